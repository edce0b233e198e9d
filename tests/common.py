"""Helpers shared by the tests: seeded inputs, the error metric and a thin
caller of the C ABI with torch device tensors."""
import ctypes
import math

import numpy as np
import torch

from mmcv_amd import capi

TOL = {torch.float32: 1e-4, torch.float16: 2e-2, torch.bfloat16: 2e-2, torch.float64: 1e-12}
DT = {torch.float32: capi.MDCN_F32, torch.float16: capi.MDCN_F16,
      torch.bfloat16: capi.MDCN_BF16, torch.float64: capi.MDCN_F64}


def pair(v):
    return (v, v) if isinstance(v, int) else tuple(v)


def out_hw(H, W, kh, kw, stride, padding, dilation):
    (sh, sw), (ph, pw), (dh, dw) = pair(stride), pair(padding), pair(dilation)
    return ((H + 2 * ph - (dh * (kh - 1) + 1)) // sh + 1,
            (W + 2 * pw - (dw * (kw - 1) + 1)) // sw + 1)


def make_case(seed, N, Cin, Cout, H, W, k=3, stride=1, padding=1, dilation=1,
              groups=1, deform_groups=1, sigma=2.0, bias=True):
    """Seeded fp32 CPU tensors in the fixed order input, offset, mask logits,
    weight, bias: input ~ N(0,1); offset ~ N(0, sigma) pixels;
    mask = sigmoid(N(0,1)); weight Kaiming-normal (fan-in, ReLU gain);
    bias ~ N(0, 0.01)."""
    kh, kw = pair(k)
    Ho, Wo = out_hw(H, W, kh, kw, stride, padding, dilation)
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(N, Cin, H, W, generator=g)
    offset = torch.randn(N, deform_groups * 2 * kh * kw, Ho, Wo, generator=g) * sigma
    mask = torch.sigmoid(torch.randn(N, deform_groups * kh * kw, Ho, Wo, generator=g))
    fan_in = Cin // groups * kh * kw
    weight = torch.randn(Cout, Cin // groups, kh, kw, generator=g) * math.sqrt(2.0 / fan_in)
    b = torch.randn(Cout, generator=g) * 0.01 if bias else None
    return dict(input=x, offset=offset, mask=mask, weight=weight, bias=b,
                stride=pair(stride), padding=pair(padding), dilation=pair(dilation),
                groups=groups, deform_groups=deform_groups)


def rel_err(y, ref):
    """max|y - ref| / max|ref| over the whole tensor."""
    y = np.asarray(y, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    return float(np.abs(y - ref).max() / max(np.abs(ref).max(), 1e-30))


def oracle_forward(case, dtype=np.float32):
    """CPU oracle on the (possibly rounded) inputs of `case`."""
    import oracle
    f = lambda t: None if t is None else t.detach().cpu().to(torch.float64 if dtype == np.float64 else torch.float32).numpy()
    return oracle.forward(f(case['input']), f(case['offset']), f(case['mask']),
                          f(case['weight']), f(case['bias']), case['stride'],
                          case['padding'], case['dilation'], case['groups'],
                          case['deform_groups'])


def cast_case(case, dtype, device=None):
    """Round every tensor once to `dtype` (and move it)."""
    out = dict(case)
    for k in ('input', 'offset', 'mask', 'weight', 'bias'):
        if case[k] is not None:
            t = case[k].to(dtype)
            out[k] = t.to(device) if device is not None else t
    return out


def capi_forward(case, path=capi.PATH_AUTO, timed=False, unsplit=False):
    """Run the C ABI on device tensors of `case`; returns the output tensor
    (and the per-stage milliseconds when `timed`).  `unsplit`: no tile is cut
    along K (mdcn_params.no_k_split), every tile is summed by one workgroup."""
    lib = capi.load()
    x, off, msk, w, b = (case[k] for k in ('input', 'offset', 'mask', 'weight', 'bias'))
    assert x.is_cuda
    N, Cin, H, W = x.shape
    Cout, _, kh, kw = w.shape
    p = capi.make_params(DT[x.dtype], N, Cin, H, W, Cout, kh, kw, case['stride'],
                         case['padding'], case['dilation'], case['groups'],
                         case['deform_groups'], path)
    rc, Ho, Wo = capi.output_size(p)
    assert rc == 0, capi.status_string(rc)
    out = torch.empty(N, Cout, Ho, Wo, dtype=x.dtype, device=x.device)
    p.no_k_split = 1 if unsplit else 0
    ws_bytes = lib.mdcn_workspace_bytes(ctypes.byref(p))
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=x.device)
    keep = [t.contiguous() for t in (x, off, w)]
    p.input, p.offset, p.weight = (t.data_ptr() for t in keep)
    if case.get('input_nhwc'):  # hand the library the channels-last bytes of the input
        keep.append(x.permute(0, 2, 3, 1).contiguous())
        p.input, p.input_nhwc = keep[-1].data_ptr(), 1
    if msk is not None:  # None: unmodulated (DCNv1)
        keep.append(msk.contiguous())
        p.mask = keep[-1].data_ptr()
    p.bias = b.contiguous().data_ptr() if b is not None else None
    p.output = out.data_ptr()
    p.workspace = ws.data_ptr() if ws_bytes else None
    p.workspace_bytes = ws_bytes
    stream = torch.cuda.current_stream().cuda_stream
    if timed:
        ms = (ctypes.c_float * 4)()
        rc = lib.mdcn_forward_timed(ctypes.byref(p), ctypes.c_void_p(stream), ms)
        assert rc == 0, capi.status_string(rc)
        torch.cuda.synchronize()
        return out, list(ms)
    rc = lib.mdcn_forward(ctypes.byref(p), ctypes.c_void_p(stream))
    assert rc == 0, capi.status_string(rc)
    torch.cuda.synchronize()
    return out


def make_pack_case(seed, N, Cin, Cout, H, W, k=3, stride=1, padding=1, dilation=1,
                   groups=1, deform_groups=1, offset_std=0.05, unmodulated=False):
    """Seeded fp32 CPU tensors of a Pack layer: input, conv_offset weight and
    bias (random, so that offsets and mask are not trivial: the layer's own
    zero initialisation would make it a plain convolution), weight, bias."""
    kh, kw = pair(k)
    g = torch.Generator().manual_seed(seed)
    co = (2 if unmodulated else 3) * deform_groups * kh * kw
    x = torch.randn(N, Cin, H, W, generator=g)
    ow = torch.randn(co, Cin, kh, kw, generator=g) * offset_std
    ob = torch.randn(co, generator=g) * 0.5
    fan_in = Cin // groups * kh * kw
    w = torch.randn(Cout, Cin // groups, kh, kw, generator=g) * math.sqrt(2.0 / fan_in)
    b = torch.randn(Cout, generator=g) * 0.01
    return dict(input=x, offset_weight=ow, offset_bias=ob, weight=w, bias=b,
                stride=pair(stride), padding=pair(padding), dilation=pair(dilation),
                groups=groups, deform_groups=deform_groups)


def cast_pack_case(case, dtype, device=None):
    out = dict(case)
    for k in ('input', 'offset_weight', 'offset_bias', 'weight', 'bias'):
        if out[k] is not None:
            out[k] = out[k].to(dtype)
            if device is not None:
                out[k] = out[k].to(device)
    return out


def oracle_conv_offset(case):
    """conv_offset on the CPU oracle: a deformable convolution with zero offsets
    and unit mask is the plain convolution."""
    x, ow = case['input'], case['offset_weight']
    kh, kw = ow.shape[2:]
    Ho, Wo = out_hw(x.shape[2], x.shape[3], kh, kw, case['stride'], case['padding'], case['dilation'])
    N = x.shape[0]
    zero = dict(input=x, offset=torch.zeros(N, 2 * kh * kw, Ho, Wo), mask=torch.ones(N, kh * kw, Ho, Wo),
                weight=ow, bias=case['offset_bias'], stride=case['stride'], padding=case['padding'],
                dilation=case['dilation'], groups=1, deform_groups=1)
    return oracle_forward(zero)


def split_raw(raw, deform_groups, taps):
    """chunk / cat / sigmoid of ModulatedDeformConv2dPack.forward on a torch
    tensor of any dtype (each step rounds to that dtype, as in the reference)."""
    o1, o2, m = torch.chunk(raw, 3, dim=1)
    return torch.cat((o1, o2), dim=1).contiguous(), torch.sigmoid(m).contiguous()


def capi_pack_forward(case, own_conv=True, raw=None, want_raw=False, path=capi.PATH_AUTO, timed=False,
                      unmodulated=False):
    """mdcn_pack_forward through ctypes on device tensors; returns (output, raw
    or None[, ms])."""
    lib = capi.load()
    x, w, b = case['input'], case['weight'], case['bias']
    N, Cin, H, W = x.shape
    Cout, _, kh, kw = w.shape
    pp = capi.MdcnPackParams()
    pp.conv = capi.make_params(DT[x.dtype], N, Cin, H, W, Cout, kh, kw, case['stride'],
                               case['padding'], case['dilation'], case['groups'],
                               case['deform_groups'], path)
    p = pp.conv
    rc, Ho, Wo = capi.output_size(p)
    assert rc == 0, capi.status_string(rc)
    co = (2 if unmodulated else 3) * case['deform_groups'] * kh * kw
    pp.unmodulated = 1 if unmodulated else 0
    out = torch.empty(N, Cout, Ho, Wo, dtype=x.dtype, device=x.device)
    keep = [t.contiguous() for t in (x, w)]
    p.input, p.weight = (t.data_ptr() for t in keep)
    if b is not None:
        keep.append(b.contiguous())
        p.bias = keep[-1].data_ptr()
    p.output = out.data_ptr()
    raw_out = None
    if own_conv:
        keep.append(case['offset_weight'].contiguous())
        pp.offset_weight = keep[-1].data_ptr()
        if case['offset_bias'] is not None:
            keep.append(case['offset_bias'].contiguous())
            pp.offset_bias = keep[-1].data_ptr()
        if want_raw:
            raw_out = torch.empty(N, co, Ho, Wo, dtype=x.dtype, device=x.device)
            pp.raw = raw_out.data_ptr()
    else:
        keep.append(raw.contiguous())
        pp.raw = keep[-1].data_ptr()
    ws_bytes = lib.mdcn_pack_workspace_bytes(ctypes.byref(pp))
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=x.device)
    p.workspace = ws.data_ptr() if ws_bytes else None
    p.workspace_bytes = ws_bytes
    stream = torch.cuda.current_stream().cuda_stream
    if timed:
        ms = (ctypes.c_float * 5)()
        rc = lib.mdcn_pack_forward_timed(ctypes.byref(pp), ctypes.c_void_p(stream), ms)
        assert rc == 0, capi.status_string(rc)
        torch.cuda.synchronize()
        return out, raw_out, list(ms)
    rc = lib.mdcn_pack_forward(ctypes.byref(pp), ctypes.c_void_p(stream))
    assert rc == 0, capi.status_string(rc)
    torch.cuda.synchronize()
    return out, raw_out


def capi_backward(case, grad_output, want_bias=True, path=0, want_data=True, want_weight=True):
    """mdcn_backward through ctypes on device tensors of `case` (mask None:
    unmodulated); returns (grad_input, grad_offset, grad_mask or None, grad_weight,
    grad_bias or None)."""
    lib = capi.load()
    x, off, msk, w = (case[k] for k in ('input', 'offset', 'mask', 'weight'))
    N, Cin, H, W = x.shape
    Cout, _, kh, kw = w.shape
    bp = capi.MdcnBwdParams()
    bp.conv = capi.make_params(DT[x.dtype], N, Cin, H, W, Cout, kh, kw, case['stride'], case['padding'],
                               case['dilation'], case['groups'], case['deform_groups'])
    p = bp.conv
    p.path = path
    keep = [t.contiguous() for t in (x, off, w, grad_output)]
    p.input, p.offset, p.weight, bp.grad_output = (t.data_ptr() for t in keep)
    g_in, g_off, g_w = torch.full_like(x, 7.0), torch.full_like(off, 7.0), torch.full_like(w, 7.0)
    if want_data:
        bp.grad_input, bp.grad_offset = g_in.data_ptr(), g_off.data_ptr()
    if want_weight:
        bp.grad_weight = g_w.data_ptr()
    g_mask = g_b = None
    if msk is not None:
        keep.append(msk.contiguous())
        p.mask = keep[-1].data_ptr()
        g_mask = torch.full_like(msk, 7.0)
        if want_data:
            bp.grad_mask = g_mask.data_ptr()
    if want_bias:
        g_b = torch.full((Cout,), 7.0, dtype=x.dtype, device=x.device)
        bp.grad_bias = g_b.data_ptr()
    ws_bytes = lib.mdcn_backward_workspace_bytes(ctypes.byref(bp))
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=x.device)
    p.workspace = ws.data_ptr() if ws_bytes else None
    p.workspace_bytes = ws_bytes
    rc = lib.mdcn_backward(ctypes.byref(bp), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, capi.status_string(rc)
    torch.cuda.synchronize()
    return g_in, g_off, g_mask, g_w, g_b
