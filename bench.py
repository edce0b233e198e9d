"""Benchmark of the DCNv2 forward hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg4]

One "step" is one call of the extension op ``modulated_deform_conv_forward`` (the
drop-in boundary) on synthetic inputs that are already resident in HBM, at the
configuration the headline metric is quoted on: bf16, N=16, Cin=Cout=256,
100x152, 3x3, stride 1, pad 1.  Prints ONE JSON line on stdout; progress and the
per-stage breakdown go to stderr.  Exits with status 3, and without the line, when
the GPU output of the timed steps does not match the CPU path.

Order of the run: a first W + K calls on the idle card (`cold_start`), the CPU
baseline, the other configurations (`configs`), then the headline -- W untimed
calls, K timed ones -- and the legs that explain it.

  value       whole-op TFLOP/s (2*N*Ho*Wo*Cout*Cin/groups*kh*kw divided by the
              time of one step, re-layout and weight repack included)
  roofline    the fused main kernel alone against the dense bf16 MFMA peak,
              its launch time measured with HIP events on the stream it runs on
  cpu_baseline  the reference's own CPU path (compiled from its sources into
              oracle/_ref) or, when that is absent, the C restatement, timed on
              this host on a bounded number of samples of the same workload
  parity      max|y - y_ref| / max|y_ref| of the GPU output against the outputs the
              CPU leg has computed on the same (rounded) inputs
  configs     the other benchmark configurations (cfg 1-3, cfg 4 in fp16, the 13
              layers of cfg 5) with fewer steps: ms, TFLOP/s, fraction of the
              dtype's matrix peak, and the parity of the first and the last sample
              against the CPU path
  cold_start  the same W + K loop as the headline, run first thing on an idle card
              (whose clocks sag under the first few dozen calls and then recover)
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, 'tests'))

PEAK_TFLOPS = {'bf16': 2500.0, 'f16': 2500.0, 'f32': 157.3}
HBM_PEAK_GBS = 8000.0
# (workload, dominant kernel) -> (HBM bytes per launch from rocprofv3 counters, the profile they are in)
TRAFFIC = {
    ('cfg4', 'fused3_kernel<bf16>'): (335.0e6, 'profiles/fused3_kernel_bf16_cfg4.md (FETCH_SIZE 102 497.9 KiB x 2.00 '
                                               '+ WRITE_SIZE 122 151.7 KiB x 1.00)'),
    ('cfg4', 'fused2_kernel<bf16>'): (422.0e6, 'profiles/fused2_kernel_bf16_cfg4.md (FETCH_SIZE 130 554.5 KiB x 2.00 '
                                               '+ WRITE_SIZE 150 981.9 KiB x 1.00)'),
}
PARITY_TOL = {'f32': 1e-4, 'bf16': 2e-2, 'f16': 2e-2}

WORKLOADS = {
    'cfg1': dict(N=1, Cin=64, Cout=64, H=56, W=56, sigma=2.0, dtype='f32'),
    'cfg2': dict(N=8, Cin=256, Cout=256, H=64, W=64, sigma=4.0, dtype='f32'),
    'cfg3': dict(N=16, Cin=512, Cout=512, H=50, W=50, stride=2, deform_groups=4,
                 sigma=3.0, dtype='f32'),
    'cfg4': dict(N=16, Cin=256, Cout=256, H=100, W=152, sigma=2.0, dtype='bf16'),
    'cfg4_f16': dict(N=16, Cin=256, Cout=256, H=100, W=152, sigma=2.0, dtype='f16'),
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def cpu_baseline(case, flops_per_sample, budget_s=20.0):
    """Time the CPU path on as many samples of the workload as fit the budget.
    `case` holds fp32 CPU tensors (the values the device sees, up-cast).  Returns
    the record and the CPU output of the samples that were run."""
    import numpy as np
    import torch
    import oracle
    N = case['input'].shape[0]
    args = lambda n: dict(stride=case['stride'], padding=case['padding'],
                          dilation=case['dilation'], groups=case['groups'],
                          deform_groups=case['deform_groups'])
    use_ref = oracle.load_reference_ext() is not None

    def run(n):
        t = {k: case[k][:n] for k in ('input', 'offset', 'mask')}
        t0 = time.perf_counter()
        if use_ref:
            y = oracle.reference_forward(t['input'], t['offset'], t['mask'], case['weight'],
                                         case['bias'], **args(n))
        else:
            y = oracle.forward(t['input'].numpy(), t['offset'].numpy(), t['mask'].numpy(),
                               case['weight'].numpy(), case['bias'].numpy(), **args(n))
        return time.perf_counter() - t0, y

    t1, _ = run(1)  # also the warm-up
    n = int(max(1, min(N, budget_s // max(t1, 1e-3))))
    tn, y_ref = run(n)
    y_ref = y_ref.numpy() if hasattr(y_ref, 'numpy') else np.asarray(y_ref)
    threads = torch.get_num_threads() if use_ref else int(os.environ.get('OMP_NUM_THREADS', os.cpu_count()))
    return {
        'value': round(flops_per_sample * n / tn / 1e12, 5),
        'unit': 'TFLOP/s',
        'cores': threads,
        'kind': 'reference' if use_ref else 'port',
        'sample': (f'{n} of {N} samples of the same workload in fp32, {tn:.2f} s '
                   f'({tn / n * 1e3:.0f} ms/sample; im2col stage is single-threaded, '
                   f'GEMM uses {threads} threads)'),
        'ms_per_layer_extrapolated': round(tn / n * N * 1e3, 1),
        'host': {'cpu_count': os.cpu_count(), 'affinity': len(os.sched_getaffinity(0)),
                 'torch_threads': torch.get_num_threads()},
    }, y_ref


def cpu_forward(seen, samples):
    """The CPU path (the compiled reference when it is there, else the C restatement) on
    the given samples of `seen` (fp32 CPU tensors holding the values the device saw)."""
    import numpy as np
    import torch
    import oracle
    idx = torch.tensor(samples)
    t = {k: seen[k][idx] for k in ('input', 'offset', 'mask')}
    kw = dict(stride=seen['stride'], padding=seen['padding'], dilation=seen['dilation'],
              groups=seen['groups'], deform_groups=seen['deform_groups'])
    if oracle.load_reference_ext() is not None:
        y = oracle.reference_forward(t['input'], t['offset'], t['mask'], seen['weight'], seen['bias'], **kw)
        kind = 'reference'
    else:
        y = oracle.forward(t['input'].numpy(), t['offset'].numpy(), t['mask'].numpy(), seen['weight'].numpy(),
                           seen['bias'].numpy(), **kw)
        kind = 'port'
    return (y.numpy() if hasattr(y, 'numpy') else np.asarray(y)), kind


def parity_record(y_gpu, y_ref, dname, what):
    """max|y - y_ref| / max|y_ref| and an element-wise count against the tolerance of the dtype."""
    import numpy as np
    tol = PARITY_TOL[dname]
    err = float(np.abs(y_gpu - y_ref).max() / np.abs(y_ref).max())
    rms = float(np.sqrt(np.mean(np.square(y_ref, dtype=np.float64))))
    viol = int((np.abs(y_gpu - y_ref) > tol * np.abs(y_ref) + tol * rms).sum())
    return {'err': float(f'{err:.3e}'), 'tolerance': tol, 'ok': bool(err <= tol and np.isfinite(y_gpu).all()),
            'violating_elements': viol, 'elements': int(y_ref.size), 'against': what}


# cfg 5: DCNv2 ResNet-50 stages c3-c5 at an 800x1344 image scale, batch 16, bf16:
# (stage, channels, layers, input HxW of the first layer, output HxW)
CFG5_STAGES = [('c3', 128, 4, (200, 336), (100, 168)),
               ('c4', 256, 6, (100, 168), (50, 84)),
               ('c5', 512, 3, (50, 84), (25, 42))]


SETTLE_CALLS = 100   # calls between the first timed loop of a configuration and its second one


def time_calls(fn, warmup, steps, settle=0):
    """ms per call of `steps` calls after `warmup` untimed ones; with `settle`, also of `steps` more calls
    after that many further untimed ones (a card that idled a moment ago -- a CPU leg, tensor set-up -- runs
    its first tens of calls at lower clocks): (first, settled or None)."""
    import torch
    res = []
    for pre in ([warmup] if not settle else [warmup, settle]):
        for _ in range(pre):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        res.append(e0.elapsed_time(e1) / steps)
    return res[0], (res[1] if settle else None)


def cfg5_layers():
    """The 13 deformable 3x3 convs: (name, C, (Hin, Win), stride)."""
    layers = []
    for name, c, n, hw_in, hw_out in CFG5_STAGES:
        for i in range(n):
            layers.append((f'{name}.{i}', c, hw_in if i == 0 else hw_out, 2 if i == 0 else 1))
    return layers


def run_cfg5(a):
    """Per-layer and summed ms of the 13 layers.  Offsets and mask come from a
    default-initialised 3x3 conv on the layer input (not the Pack's zero
    initialisation, which would make every offset 0), then chunk/cat/sigmoid as
    in ModulatedDeformConv2dPack.forward; that producer is timed separately."""
    import torch
    from mmcv_amd.ops import ModulatedDeformConv2dPack
    from mmcv_amd.ops.modulated_deform_conv import ext_module
    torch.manual_seed(20245)
    N = 16
    rows, tot_dcn, tot_prod, tot_flops, tot_pack = [], 0.0, 0.0, 0.0, 0.0
    ev = lambda: torch.cuda.Event(enable_timing=True)
    for name, C, (H, W), stride in cfg5_layers():
        layer = ModulatedDeformConv2dPack(C, C, 3, stride=stride, padding=1, deform_groups=1)
        torch.nn.Conv2d.reset_parameters(layer.conv_offset)
        layer = layer.cuda().bfloat16()
        x = torch.randn(N, C, H, W, device='cuda').bfloat16()
        with torch.no_grad():
            def producer():
                raw = layer.conv_offset(x)
                o1, o2, m = torch.chunk(raw, 3, dim=1)
                return torch.cat((o1, o2), dim=1), torch.sigmoid(m)
            off, msk = producer()
            Ho, Wo = off.shape[2:]
            out = torch.empty(N, C, Ho, Wo, dtype=torch.bfloat16, device='cuda')
            empty = x.new_empty(0)
            kw = dict(kernel_h=3, kernel_w=3, stride_h=stride, stride_w=stride, pad_h=1, pad_w=1,
                      dilation_h=1, dilation_w=1, group=1, deformable_group=1, with_bias=True)
            dcn = lambda: ext_module.modulated_deform_conv_forward(
                x, layer.weight, layer.bias, empty, off, msk, out, empty, **kw)
            pack = lambda: layer(x)   # one extension call: conv_offset + split + sigmoid + DCN
            t = []
            for fn in (producer, dcn, pack):
                first, settled = time_calls(fn, a.warmup, a.steps, SETTLE_CALLS if fn is dcn else 0)
                t.append(first)
                if fn is dcn:
                    dcn_settled = settled
        flops = 2.0 * N * Ho * Wo * C * C * 9
        rows.append({'layer': name, 'C': C, 'in': [H, W], 'stride': stride,
                     'producer_ms': round(t[0], 4), 'dcn_ms': round(t[1], 4),
                     'dcn_TFLOPs': round(flops / t[1] / 1e9, 1), 'dcn_ms_settled': round(dcn_settled, 4),
                     'pack_fused_ms': round(t[2], 4)})
        if getattr(a, 'parity', False) and name.endswith('.1'):
            # one layer per stage: first and last sample of the op's output against the CPU path
            dcn()
            torch.cuda.synchronize()
            seen = dict(input=x.float().cpu(), offset=off.float().cpu(), mask=msk.float().cpu(),
                        weight=layer.weight.detach().float().cpu(), bias=layer.bias.detach().float().cpu(),
                        stride=(stride, stride), padding=(1, 1), dilation=(1, 1), groups=1, deform_groups=1)
            y_ref, kind = cpu_forward(seen, [0, N - 1])
            rows[-1]['parity'] = parity_record(out[[0, N - 1]].float().cpu().numpy(), y_ref, 'bf16',
                                               kind + ' CPU path, samples 0 and %d' % (N - 1))
        log(rows[-1])
        tot_prod += t[0]
        tot_dcn += t[1]
        tot_pack += t[2]
        tot_flops += flops
        del x, off, msk, out, layer
        torch.cuda.empty_cache()
    return rows, tot_dcn, tot_prod, tot_flops, tot_pack


def quick_config(name, steps, warmup, parity=False):
    """One of the single-layer configurations with few steps: ms per call of the
    extension op, TFLOP/s and the fraction of the dtype's matrix peak."""
    import torch
    from common import make_case, cast_case
    from mmcv_amd.ops.modulated_deform_conv import ext_module
    wl = dict(WORKLOADS[name])
    dname = wl.pop('dtype')
    dtype = {'bf16': torch.bfloat16, 'f16': torch.float16, 'f32': torch.float32}[dname]
    case = make_case(20240 + int(name[3]), **wl)
    dev = cast_case(case, dtype, 'cuda')
    x, off, msk, w, b = (dev[k] for k in ('input', 'offset', 'mask', 'weight', 'bias'))
    N, Cin, H, W = x.shape
    Cout, cin_g, kh, kw = w.shape
    (sh, sw), (ph, pw), (dh, dw) = case['stride'], case['padding'], case['dilation']
    Ho = (H + 2 * ph - (dh * (kh - 1) + 1)) // sh + 1
    Wo = (W + 2 * pw - (dw * (kw - 1) + 1)) // sw + 1
    out = torch.empty(N, Cout, Ho, Wo, dtype=dtype, device='cuda')
    empty = x.new_empty(0)
    kwargs = dict(kernel_h=kh, kernel_w=kw, stride_h=sh, stride_w=sw, pad_h=ph, pad_w=pw,
                  dilation_h=dh, dilation_w=dw, group=case['groups'],
                  deformable_group=case['deform_groups'], with_bias=True)
    fn = lambda: ext_module.modulated_deform_conv_forward(x, w, b, empty, off, msk, out, empty, **kwargs)
    ms, ms_settled = time_calls(fn, warmup, steps, SETTLE_CALLS)
    flops = 2.0 * N * Ho * Wo * Cout * cin_g * kh * kw
    tf = flops / ms / 1e9
    tf_settled = flops / ms_settled / 1e9
    rec = {'dtype': dname, 'ms_per_layer': round(ms, 4), 'TFLOPs': round(tf, 2),
           'pct_matrix_peak': round(100.0 * tf / PEAK_TFLOPS[dname], 2), 'steps': steps, 'warmup': warmup,
           # the same loop again after SETTLE_CALLS more calls: the configuration's tensors were set up on
           # the host a moment ago, and the first loop runs on a card that is still raising its clocks
           'settled': {'ms_per_layer': round(ms_settled, 4), 'TFLOPs': round(tf_settled, 2),
                       'pct_matrix_peak': round(100.0 * tf_settled / PEAK_TFLOPS[dname], 2),
                       'after_calls': warmup + steps + SETTLE_CALLS}}
    if parity:
        seen = dict(case)
        for k in ('input', 'offset', 'mask', 'weight', 'bias'):
            seen[k] = dev[k].float().cpu()
        samples = sorted({0, N - 1})
        y_ref, kind = cpu_forward(seen, samples)
        rec['parity'] = parity_record(out[samples].float().cpu().numpy(), y_ref, dname,
                                      kind + ' CPU path, samples ' + ' and '.join(map(str, samples)))
    return rec


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=200)
    ap.add_argument('--warmup', type=int, default=20)
    ap.add_argument('--workload', default='cfg4', choices=sorted(WORKLOADS) + ['cfg5'])
    ap.add_argument('--path', default='auto', choices=['auto', 'narrow', 'wide'],
                    help="forward kernels of the 16-bit fused path: the library's choice, the 128-pixel "
                         'kernel only, or the 256-pixel kernel on every whole tile')
    ap.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline leg')
    ap.add_argument('--no-configs', action='store_true',
                    help='skip the short runs of the other benchmark configurations')
    ap.add_argument('--copy-probe', action='store_true',
                    help='run a plain elementwise copy of known size instead (calibrates the '
                         'FETCH_SIZE / WRITE_SIZE counters) and exit')
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get('WORLD_SIZE', '1')) != 1:
        log('bench.py: this path is built and measured on ONE GPU; '
            'samples and pixel tiles are independent, so more GPUs only split the batch. '
            'Run with --gpus 1.')
        sys.exit(2)

    import torch
    if a.copy_probe:
        # 256 MiB read + 256 MiB written per launch by one elementwise kernel
        src = torch.ones(128 * 1024 * 1024, dtype=torch.bfloat16, device='cuda')
        dst = torch.empty_like(src)
        for _ in range(a.steps):
            torch.add(src, 1, out=dst)
        torch.cuda.synchronize()
        print(json.dumps({'copy_probe_bytes_read': src.numel() * 2,
                          'copy_probe_bytes_written': dst.numel() * 2, 'launches': a.steps}))
        return
    if a.workload == 'cfg5':
        assert torch.cuda.is_available(), 'bench.py needs a GPU'
        rows, tot_dcn, tot_prod, tot_flops, tot_pack = run_cfg5(a)
        print(json.dumps({
            'metric': 'DCNv2 fwd summed ms over 13 layers (ResNet-50 c3-c5, N=16, 800x1344 scale, bf16)',
            'value': round(tot_dcn, 4), 'unit': 'ms', 'n_gpus': 1, 'steps': a.steps,
            'warmup': a.warmup, 'ms_per_step': round(tot_dcn, 4), 'higher_is_better': False,
            'scaling': 'weak', 'vs_baseline': None, 'dtype': 'bf16', 'data': 'synthetic',
            'config': {'workload': 'cfg5: 13 DCNv2 3x3 layers, c3 4x128ch@100x168, c4 6x256ch@50x84, '
                                   'c5 3x512ch@25x42, first layer of each stage stride 2'},
            'dcn_TFLOPs': round(tot_flops / tot_dcn / 1e9, 1),
            'pct_mfma_peak': round(100.0 * tot_flops / tot_dcn / 1e9 / PEAK_TFLOPS['bf16'], 2),
            'offset_mask_producer_ms': round(tot_prod, 4),
            'summed_ms_with_producer': round(tot_dcn + tot_prod, 4),
            'summed_ms_settled': round(sum(r['dcn_ms_settled'] for r in rows), 4),
            'summed_ms_pack_fused': round(tot_pack, 4), 'layers': rows}), flush=True)
        return
    from common import make_case, cast_case
    from mmcv_amd.ops.modulated_deform_conv import ext_module

    assert torch.cuda.is_available(), 'bench.py needs a GPU'
    torch.cuda.set_device(0)
    ext_module.set_path({'auto': 0, 'narrow': 5, 'wide': 4}[a.path])  # (MDCN_PATH_AUTO / _FUSED_NARROW / _FUSED_WIDE)
    wl = dict(WORKLOADS[a.workload])
    dname = wl.pop('dtype')
    dtype = {'bf16': torch.bfloat16, 'f16': torch.float16, 'f32': torch.float32}[dname]
    seed = 20240 + int(a.workload[3])
    case = make_case(seed, **wl)
    dev = cast_case(case, dtype, 'cuda')
    N, Cin, H, W = case['input'].shape
    Cout, cin_g, kh, kw = case['weight'].shape
    x, off, msk, w, b = (dev[k] for k in ('input', 'offset', 'mask', 'weight', 'bias'))
    (sh, sw), (ph, pw), (dh, dw) = case['stride'], case['padding'], case['dilation']
    Ho = (H + 2 * ph - (dh * (kh - 1) + 1)) // sh + 1
    Wo = (W + 2 * pw - (dw * (kw - 1) + 1)) // sw + 1
    out = torch.empty(N, Cout, Ho, Wo, dtype=dtype, device='cuda')
    empty = x.new_empty(0)
    kwargs = dict(kernel_h=kh, kernel_w=kw, stride_h=sh, stride_w=sw, pad_h=ph, pad_w=pw,
                  dilation_h=dh, dilation_w=dw, group=case['groups'],
                  deformable_group=case['deform_groups'], with_bias=True)
    flops = 2.0 * N * Ho * Wo * Cout * cin_g * kh * kw
    es = 4 if dname == 'f32' else 2
    alg_bytes = es * (x.numel() + off.numel() + msk.numel() + w.numel() + b.numel() + out.numel())

    def step():
        ext_module.modulated_deform_conv_forward(x, w, b, empty, off, msk, out, empty, **kwargs)

    def timed_loop(fn, warmup, steps):
        """`warmup` untimed calls, then `steps` timed ones: (ms per call by events, by the wall clock)."""
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps, (time.perf_counter() - t0) * 1e3 / steps

    peak = PEAK_TFLOPS[dname]
    tfl = lambda ms: flops / (ms * 1e-3) / 1e12

    # ---- 1. the loop on an idle card: clocks sag under the first few dozen calls and then recover
    cold_ev, cold_wall = timed_loop(step, a.warmup, a.steps)
    cold_ms = max(cold_ev, cold_wall)
    log(f'cold start: step {cold_ms:.4f} ms')

    # ---- 2. the CPU baseline (and the reference output for the parity of the timed steps)
    cpu_rec, y_ref = None, None
    if not a.no_cpu:
        log('timing the CPU baseline ...')
        # the CPU path gets the values the device saw (rounded to the tensor dtype, up-cast)
        seen = dict(case)
        for k in ('input', 'offset', 'mask', 'weight', 'bias'):
            seen[k] = dev[k].float().cpu()
        cpu_rec, y_ref = cpu_baseline(seen, flops / N)

    # ---- 3. the other configurations, each with the parity of its first and last sample
    others = None
    if not a.no_configs:
        others = {}
        for name in sorted(WORKLOADS):
            if name != a.workload:
                others[name] = quick_config(name, max(5, min(a.steps, 50)), max(2, min(a.warmup, 10)),
                                            parity=not a.no_cpu)
                log(name, others[name])
        a5 = argparse.Namespace(steps=max(5, min(a.steps, 20)), warmup=max(2, min(a.warmup, 5)), parity=not a.no_cpu)
        rows, tot_dcn, tot_prod, tot_flops, tot_pack = run_cfg5(a5)
        others['cfg5'] = {'dtype': 'bf16', 'summed_ms': round(tot_dcn, 4),
                          'TFLOPs': round(tot_flops / tot_dcn / 1e9, 1),
                          'pct_matrix_peak': round(100.0 * tot_flops / tot_dcn / 1e9 / PEAK_TFLOPS['bf16'], 2),
                          'summed_ms_pack_fused': round(tot_pack, 4), 'steps': a5.steps, 'warmup': a5.warmup,
                          'per_layer_ms': {r['layer']: r['dcn_ms'] for r in rows},
                          # each layer's loop again after SETTLE_CALLS more calls (see quick_config)
                          'settled': {'summed_ms': round(sum(r['dcn_ms_settled'] for r in rows), 4),
                                      'pct_matrix_peak': round(100.0 * tot_flops / sum(r['dcn_ms_settled'] for r in rows)
                                                               / 1e9 / PEAK_TFLOPS['bf16'], 2),
                                      'per_layer_ms': {r['layer']: r['dcn_ms_settled'] for r in rows}},
                          'parity': {r['layer']: r['parity'] for r in rows if 'parity' in r}}

    # ---- 4. the same call on four rotating sets of buffers and through the bare C ABI (these legs also keep
    # the card under load between the CPU work above and the headline)
    sets = [(x, off, msk, out)] + [(torch.randn_like(x), off.clone(), msk.clone(), torch.empty_like(out))
                                   for _ in range(3)]
    # (four sets of input / offset / mask / output, 1.05 GB: no call finds its operands in the 256 MB last-level
    # cache; the C-ABI call has its workspace allocated once)
    rot = [0]

    def step_rot():
        i = rot[0] = (rot[0] + 1) % 4
        ext_module.modulated_deform_conv_forward(sets[i][0], w, b, empty, sets[i][1], sets[i][2], sets[i][3], empty,
                                                 **kwargs)
    rot_ms, _ = timed_loop(step_rot, 4, a.steps)
    del sets
    import ctypes
    from mmcv_amd import capi
    lib = capi.load()
    cp = capi.make_params({'f32': 0, 'f16': 1, 'bf16': 2}[dname], N, Cin, H, W, Cout, kh, kw, (sh, sw), (ph, pw),
                          (dh, dw), case['groups'], case['deform_groups'])
    cp.input, cp.offset, cp.mask, cp.weight, cp.bias, cp.output = (t.data_ptr() for t in (x, off, msk, w, b, out))
    cp.path = ext_module.get_path()
    cws = torch.empty(lib.mdcn_workspace_bytes(ctypes.byref(cp)), dtype=torch.uint8, device='cuda')
    cp.workspace, cp.workspace_bytes = cws.data_ptr(), cws.numel()
    kernels = lib.mdcn_forward_kernels(ctypes.byref(cp)).decode()  # what the library launches for this call
    cstream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def step_cabi():
        assert lib.mdcn_forward(ctypes.byref(cp), cstream) == 0
    cabi_ms, _ = timed_loop(step_cabi, 3, a.steps)
    del cws

    # ---- 5. the headline: W untimed calls, K timed ones
    ev_ms, wall_ms = timed_loop(step, a.warmup, a.steps)
    ms_per_step = max(wall_ms, ev_ms)
    y_timed = out.clone()  # what the timed steps wrote

    # dominant kernel: HIP events recorded by the library on the stream it launches on
    stage = [0.0, 0.0, 0.0, 0.0]
    for _ in range(a.steps):
        ms = ext_module.modulated_deform_conv_forward_timed(x, w, b, off, msk, out, **kwargs)
        stage = [s + m for s, m in zip(stage, ms)]
    stage = [s / a.steps for s in stage]
    main_ms = stage[2]
    log(f'{a.workload} {dname}: step {ms_per_step:.4f} ms (events {ev_ms:.4f}, wall {wall_ms:.4f}); '
        f'stages relayout {stage[0]:.4f} pack {stage[1]:.4f} main {stage[2]:.4f} ms')

    # the same step with the input handed over channels-last (read in place, no re-layout)
    x_cl = x.contiguous(memory_format=torch.channels_last)
    step_cl = lambda: ext_module.modulated_deform_conv_forward(x_cl, w, b, empty, off, msk, out, empty, **kwargs)
    cl_ms, _ = timed_loop(step_cl, a.warmup, a.steps)
    log(f'channels-last input: step {cl_ms:.4f} ms')

    # per-call distribution (one event pair per call)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(a.steps)]
    for s0, s1 in evs:
        s0.record()
        step()
        s1.record()
    torch.cuda.synchronize()
    per_call = sorted(s0.elapsed_time(s1) for s0, s1 in evs)
    # what the matrix cores of this box sustain (back-to-back MFMAs on every CU, random and zero
    # operands): context for the published peak the roofline fraction is taken against
    sustained = None
    if dname in ('bf16', 'f16'):
        scratch = torch.empty(16384, dtype=torch.uint8, device='cuda')
        tf = ctypes.c_float()
        sustained = {}
        probe = ctypes.CDLL(os.path.join(ROOT, 'bench_probe', 'libmfma_probe.so'))
        probe.mdcn_mfma_probe.restype = ctypes.c_int
        probe.mdcn_mfma_probe.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                          ctypes.c_void_p, ctypes.POINTER(ctypes.c_float)]
        for key, zero in (('random_operands', 0), ('zero_operands', 1)):
            rc = probe.mdcn_mfma_probe(2 if dname == 'bf16' else 1, 2, zero, ctypes.c_void_p(scratch.data_ptr()),
                                       cstream, ctypes.byref(tf))
            assert rc == 0, f'mdcn_mfma_probe: status {rc}'
            sustained[key] = round(tf.value, 1)
        log(f'sustained MFMA rate: {sustained}')
    log(f'per call: median {per_call[len(per_call) // 2]:.4f} min {per_call[0]:.4f} ms; rotating buffers '
        f'{rot_ms:.4f} ms; bare C ABI {cabi_ms:.4f} ms')

    # the layer's backward (all five gradients) through the same extension, for reference beside
    # the headline forward figure; not part of `value`
    gy = torch.randn(N, Cout, Ho, Wo, device='cuda').to(dtype)
    g_in, g_w, g_b = torch.empty_like(x), torch.empty_like(w), torch.empty_like(b)
    g_off, g_msk = torch.empty_like(off), torch.empty_like(msk)
    step_bwd = lambda: ext_module.modulated_deform_conv_backward(
        x, w, b, empty, off, msk, empty, g_in, g_w, g_b, g_off, g_msk, gy, **kwargs)
    bsteps = max(3, a.steps // 5)
    bwd_ms, _ = timed_loop(step_bwd, 2, bsteps)
    log(f'backward: step {bwd_ms:.4f} ms')

    value = tfl(ms_per_step)
    achieved = tfl(main_ms)
    # the kernel that does most of the main stage's work, by the library's own account
    main_kernel = kernels.split('+')[0]
    kernel_name = f'{main_kernel}<{dname}>'
    rec = {
        'metric': 'DCNv2 fwd TFLOP/s + ms/layer (N=16,C=256,100x152 bf16); % MFMA peak',
        'value': round(value, 2),
        'unit': 'TFLOP/s',
        'n_gpus': 1,
        'steps': a.steps,
        'warmup': a.warmup,
        'ms_per_step': round(ms_per_step, 4),
        'higher_is_better': True,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': dname,
        'data': 'synthetic',
        'config': {
            'workload': (f'{a.workload}: ModulatedDeformConv2d fwd N={N} Cin={Cin} Cout={Cout} '
                         f'{H}x{W} k{kh}x{kw} s{sh} p{ph} d{dh} groups={case["groups"]} '
                         f'deform_groups={case["deform_groups"]}, offsets N(0,{wl["sigma"]}) px'),
            'entry': 'mmcv_amd._ext.modulated_deform_conv_forward',
            'path': a.path,
            'flops_per_step': flops,
            'algorithmic_bytes_per_step': alg_bytes,
        },
        'ms_per_layer': round(ms_per_step, 4),
        'pct_mfma_peak': round(100.0 * value / peak, 2),
        'timed_region': ('the W untimed and K timed calls follow the cold-start loop, the CPU baseline, the other '
                         'configurations and the rotating-buffer and C-ABI legs of this run, i.e. start on a card '
                         'that is under load'),
        'cold_start': {'ms_per_step': round(cold_ms, 4), 'TFLOPs': round(tfl(cold_ms), 2),
                       'pct_mfma_peak': round(100.0 * tfl(cold_ms) / peak, 2), 'steps': a.steps, 'warmup': a.warmup,
                       'what': 'the same W + K loop run first thing in the process, on an idle card'},
        'stage_ms': {'relayout': round(stage[0], 4), 'weight_pack': round(stage[1], 4),
                     'main': round(stage[2], 4)},
        'main_stage_kernels': kernels,
        'hbm_GBs_algorithmic': round(alg_bytes / (ms_per_step * 1e-3) / 1e9, 1),
        'channels_last_input': {'ms_per_step': round(cl_ms, 4), 'TFLOPs': round(tfl(cl_ms), 2)},
        'per_call_ms': {'median': round(per_call[len(per_call) // 2], 4), 'min': round(per_call[0], 4)},
        'rotating_buffers': {'sets': 4, 'ms_per_step': round(rot_ms, 4)},
        'c_abi_call': {'entry': 'mdcn_forward', 'ms_per_step': round(cabi_ms, 4)},
        'backward': {'ms_per_step': round(bwd_ms, 4), 'steps': bsteps,
                     'TFLOPs': round(2.0 * flops / (bwd_ms * 1e-3) / 1e12, 2),
                     'what': 'grad input/offset/mask/weight/bias; two products of the forward size'},
        'roofline': {
            'bound': 'mfma',
            'kernel': kernel_name,
            'achieved': round(achieved, 2),
            'peak': peak,
            'unit': 'TFLOP/s',
            'frac': round(achieved / peak, 4),
            # HBM bytes per launch of that kernel from rocprofv3 FETCH_SIZE and WRITE_SIZE, scaled by a
            # copy kernel of known size: a figure from the named profile, not from this run
            'traffic': TRAFFIC.get((a.workload, kernel_name), (None, None))[0],
            'traffic_source': TRAFFIC.get((a.workload, kernel_name), (None, None))[1],
        },
        # measured on this box, same run: TFLOP/s of back-to-back 32x32x16 MFMAs on all CUs; the kernel's
        # share of what the matrix cores sustain on non-trivial operands
        'mfma_sustained_TFLOPs': sustained,
        'frac_of_sustained': (round(achieved / sustained['random_operands'], 4) if sustained else None),
    }
    if others is not None:
        rec['configs'] = others
    ok = True
    if cpu_rec is not None:
        import numpy as np
        rec['cpu_baseline'] = cpu_rec
        n_ref = y_ref.shape[0]
        par = parity_record(y_timed[:n_ref].float().cpu().numpy(), y_ref, dname,
                            cpu_rec['kind'] + ' CPU path on the same rounded inputs')
        par.update({'samples_checked': n_ref, 'of': N})
        rec['parity'] = par
        log('parity', par)
        ok = par['ok']
        for name, o in (others or {}).items():
            ps = [o['parity']] if 'err' in o.get('parity', {}) else list(o.get('parity', {}).values())
            ok = ok and all(q['ok'] for q in ps)
    if not ok:
        log('PARITY FAILED: the GPU output does not match the CPU path; no metric line')
        log(json.dumps(rec))
        sys.exit(3)
    print(json.dumps(rec), flush=True)


if __name__ == '__main__':
    main()
