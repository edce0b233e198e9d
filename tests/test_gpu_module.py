"""GPU tests of the drop-in boundary: the mmcv-compatible Python API on top of
mmcv_amd._ext, the reference's own known-answer vector, the committed outputs
of the compiled reference, and the five benchmark configurations at full size.

Error metric: max|y - y_ref| / max|y_ref|; bars fp32 1e-4, bf16/fp16 2e-2."""
import json
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from mmcv_amd import capi

from common import (TOL, capi_forward, cast_case, make_case, oracle_forward,
                    rel_err)

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden')


def dcn2d(case):
    from mmcv_amd.ops import modulated_deform_conv2d
    return modulated_deform_conv2d(case['input'], case['offset'], case['mask'],
                                   case['weight'], case['bias'], case['stride'],
                                   case['padding'], case['dilation'], case['groups'],
                                   case['deform_groups'])


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16, torch.bfloat16])
def test_reference_kat_through_pack(dtype):
    """tests/test_ops/test_modulated_deform_conv.py:49-76 (forward part)."""
    from mmcv_amd.ops import ModulatedDeformConv2dPack
    with open(os.path.join(GOLD, 'reference_kats.json')) as f:
        k = json.load(f)['dcnv2_zero_offset']
    x = torch.tensor(k['input'], dtype=dtype, device='cuda')
    dcn = ModulatedDeformConv2dPack(1, 1, kernel_size=(2, 2), stride=1, padding=1,
                                    deform_groups=1, bias=False).cuda()
    dcn.weight.data.fill_(1.)
    dcn.type(dtype)
    y = dcn(x)
    assert y.dtype == dtype and y.shape == (1, 1, 4, 4)
    assert np.allclose(y.float().cpu().detach().numpy(), k['output'], 1e-2)


@pytest.mark.parametrize('input_dtype', [torch.float32, torch.float16])
def test_reference_kat_under_autocast(input_dtype):
    """tests/test_ops/test_modulated_deform_conv.py:85-128: the model stays fp32,
    autocast makes the offsets half, and the op follows offset's dtype."""
    from mmcv_amd.ops import ModulatedDeformConv2dPack
    with open(os.path.join(GOLD, 'reference_kats.json')) as f:
        k = json.load(f)['dcnv2_zero_offset']
    x = torch.tensor(k['input'], device='cuda').type(input_dtype)
    dcn = ModulatedDeformConv2dPack(1, 1, kernel_size=(2, 2), stride=1, padding=1,
                                    deform_groups=1, bias=False).cuda()
    dcn.weight.data.fill_(1.)
    with torch.autocast('cuda', dtype=torch.float16):
        y = dcn(x)
    assert y.dtype == torch.float16
    assert np.allclose(y.float().cpu().detach().numpy(), k['output'], 1e-2)


def test_dcnv1_fractional_kat():
    """tests/test_ops/test_deform_conv.py:27-35 with mask = 1 (fp32, both paths)."""
    from mmcv_amd import _ext
    with open(os.path.join(GOLD, 'reference_kats.json')) as f:
        k = json.load(f)['dcnv1_fractional']
    x = torch.tensor(k['input'], device='cuda')
    ow = torch.tensor(k['offset_weight'], device='cuda').view(8, 1, 2, 2)
    off = F.conv2d(x, ow, torch.tensor(k['offset_bias'], device='cuda'))
    w = torch.tensor(k['deform_weight'], device='cuda').view(1, 1, 2, 2)
    case = dict(input=x, offset=off, mask=torch.ones(1, 4, 2, 2, device='cuda'),
                weight=w, bias=None, stride=(1, 1), padding=(0, 0), dilation=(1, 1),
                groups=1, deform_groups=1)
    y = dcn2d(case).cpu().numpy()
    assert np.allclose(y, np.array(k['output']), rtol=0, atol=k['atol'])


@pytest.mark.parametrize('path', [capi.PATH_AUTO, capi.PATH_DIRECT])
def test_golden_outputs_of_compiled_reference(path):
    with open(os.path.join(GOLD, 'ref_cases.json')) as f:
        meta = json.load(f)
    data = np.load(os.path.join(GOLD, 'ref_cases.npz'))
    for name, kw in meta.items():
        kw = dict(kw)
        seed, dt = kw.pop('seed'), kw.pop('dtype')
        print('golden', name, flush=True)
        case = make_case(seed, **kw)
        y = capi_forward(cast_case(case, torch.float32, 'cuda'), path=path).cpu().numpy()
        assert rel_err(y, data[name]) <= 1e-4, name


def test_output_fully_written_and_inputs_untouched():
    case = cast_case(make_case(3, N=3, Cin=32, Cout=40, H=9, W=13), torch.float32, 'cuda')
    from mmcv_amd import _ext
    x, off, m, w, b = (case[k] for k in ('input', 'offset', 'mask', 'weight', 'bias'))
    keep = [t.clone() for t in (x, off, m, w, b)]
    out = torch.full((3, 40, 9, 13), float('nan'), device='cuda')
    empty = x.new_empty(0)
    _ext.modulated_deform_conv_forward(
        x, w, b, empty, off, m, out, empty, kernel_h=3, kernel_w=3, stride_h=1,
        stride_w=1, pad_h=1, pad_w=1, dilation_h=1, dilation_w=1, group=1,
        deformable_group=1, with_bias=True)
    assert torch.isfinite(out).all()
    assert empty.numel() == 0
    for a, bb in zip(keep, (x, off, m, w, b)):
        assert torch.equal(a, bb)
    assert rel_err(out.cpu().numpy(), oracle_forward(make_case(3, N=3, Cin=32, Cout=40, H=9, W=13))) <= 1e-4


def test_non_contiguous_inputs_and_side_stream():
    case = make_case(4, N=2, Cin=32, Cout=32, H=10, W=12)
    ref = oracle_forward(case)
    dev = cast_case(case, torch.float32, 'cuda')
    dev['input'] = dev['input'].permute(0, 2, 3, 1).contiguous().permute(0, 3, 1, 2)  # channels-last strides
    dev['offset'] = dev['offset'].flip(0).flip(0)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        y = dcn2d(dev)
    s.synchronize()
    assert rel_err(y.cpu().numpy(), ref) <= 1e-4


def test_device_and_shape_errors():
    from mmcv_amd.ops import modulated_deform_conv2d
    case = cast_case(make_case(5, N=1, Cin=32, Cout=32, H=8, W=8), torch.float32, 'cuda')
    # (the Python wrapper's type_as moves a stray CPU weight to the GPU, as the
    # reference's does, so the device check is exercised on the extension op)
    from mmcv_amd import _ext
    e = case['input'].new_empty(0)
    with pytest.raises(RuntimeError, match='inconsistent device'):
        _ext.modulated_deform_conv_forward(
            case['input'], case['weight'].cpu(), e, e, case['offset'], case['mask'],
            case['input'].new_empty(1, 32, 8, 8), e, kernel_h=3, kernel_w=3,
            stride_h=1, stride_w=1, pad_h=1, pad_w=1, dilation_h=1, dilation_w=1,
            group=1, deformable_group=1, with_bias=False)
    with pytest.raises(RuntimeError, match="kernel channels won't match"):
        modulated_deform_conv2d(case['input'], case['offset'], case['mask'],
                                case['weight'][:, :16].contiguous(), None, 1, 1)
    with pytest.raises(RuntimeError, match='offset must be'):
        modulated_deform_conv2d(case['input'], case['offset'][:, :9], case['mask'],
                                case['weight'], None, 1, 1)
    with pytest.raises(RuntimeError, match="not implemented for 'Int'"):
        modulated_deform_conv2d(case['input'].int(), case['offset'].int(),
                                case['mask'].int(), case['weight'].int(), None, 1, 1)
    # gradients flow (their values are checked in test_gpu_backward.py)
    x = case['input'].clone().requires_grad_(True)
    modulated_deform_conv2d(x, case['offset'], case['mask'], case['weight'], None, 1, 1).sum().backward()
    assert x.grad is not None and torch.isfinite(x.grad).all()


# ---- the benchmark configurations at full size ----------------------------------

FULL = {
    'cfg1': (dict(N=1, Cin=64, Cout=64, H=56, W=56, sigma=2.0), [torch.float32]),
    'cfg2': (dict(N=8, Cin=256, Cout=256, H=64, W=64, sigma=4.0), [torch.float32]),
    'cfg3': (dict(N=16, Cin=512, Cout=512, H=50, W=50, stride=2, deform_groups=4, sigma=3.0),
             [torch.float32]),
    'cfg4': (dict(N=16, Cin=256, Cout=256, H=100, W=152, sigma=2.0),
             [torch.bfloat16, torch.float16]),
}


@pytest.mark.parametrize('name', sorted(FULL))
def test_full_size_configs(name):
    """Full-size run; the oracle checks the first and the last sample (samples
    are independent), and size-independent properties cover the whole batch:
    every output element is written, and a batch-reversed call returns the
    batch-reversed result bit for bit."""
    kw, dtypes = FULL[name]
    case = make_case(20240 + int(name[-1]), **kw)
    N = kw['N']
    for dtype in dtypes:
        print(name, dtype, flush=True)
        dev = cast_case(case, dtype, 'cuda')
        y = capi_forward(dev, path=capi.PATH_FUSED)
        assert torch.isfinite(y).all()
        rounded = cast_case(case, dtype)
        for n in sorted({0, N - 1}):
            sub = dict(rounded)
            for k in ('input', 'offset', 'mask'):
                sub[k] = rounded[k][n:n + 1]
            err = rel_err(y[n:n + 1].float().cpu().numpy(), oracle_forward(sub))
            print(f'  sample {n}: err {err:.3e}', flush=True)
            assert err <= TOL[dtype], (name, dtype, n, err)
        rev = dict(dev)
        for k in ('input', 'offset', 'mask'):
            rev[k] = dev[k].flip(0).contiguous()
        # A tile's sum does not depend on where in the batch its image sits -- as long as one workgroup
        # forms it.  (With the split buffers in the workspace, tiles of the schedule's last round are cut
        # along K and their parts added in fp32, which rounds differently from one long sum.)
        y_one = capi_forward(dev, path=capi.PATH_FUSED, unsplit=True)
        y_rev = capi_forward(rev, path=capi.PATH_FUSED, unsplit=True)
        assert torch.equal(y_rev.flip(0), y_one)
        if name == 'cfg4':
            # the kernel with 256-pixel tiles and the one with 128-pixel tiles sum every tile in the same order
            y_wide = capi_forward(dev, path=capi.PATH_FUSED_WIDE, unsplit=True)
            assert torch.equal(y_wide, capi_forward(dev, path=capi.PATH_FUSED_NARROW, unsplit=True))
            assert torch.equal(y_wide, y_one)
        # cut tiles: same result on every run, and within an output ulp or so of the uncut sums
        assert torch.equal(capi_forward(dev, path=capi.PATH_FUSED), y)
        diff = (y.float() - y_one.float()).abs()
        assert float(diff.max() / y_one.float().abs().max()) <= (1e-5 if dtype == torch.float32 else 4e-3)


def test_full_size_zero_offset_matches_conv2d():
    """cfg 4 shape, offsets 0 and mask 1: the op is an ordinary convolution."""
    kw = dict(FULL['cfg4'][0], sigma=0.0)
    case = make_case(99, **kw)
    case['mask'] = torch.ones_like(case['mask'])
    dev = cast_case(case, torch.bfloat16, 'cuda')
    y = capi_forward(dev, path=capi.PATH_FUSED).float()
    ref = F.conv2d(dev['input'].float(), dev['weight'].float(), dev['bias'].float(), 1, 1)
    err = float((y - ref).abs().max() / ref.abs().max())
    assert err <= TOL[torch.bfloat16], err


def test_fused_matches_direct_on_cfg3_shape():
    """Two independent device implementations agree on the deform-group / stride-2 case."""
    kw = dict(FULL['cfg3'][0], N=2)
    dev = cast_case(make_case(77, **kw), torch.float32, 'cuda')
    a = capi_forward(dev, path=capi.PATH_FUSED)
    b = capi_forward(dev, path=capi.PATH_DIRECT)
    assert float((a - b).abs().max() / b.abs().max()) <= 1e-4


CFG5_SHAPES = [  # (C, Hin, Win, stride): the six distinct layer shapes of the ResNet-50 c3-c5 config
    (128, 200, 336, 2), (128, 100, 168, 1), (256, 100, 168, 2), (256, 50, 84, 1),
    (512, 50, 84, 2), (512, 25, 42, 1)]


@pytest.mark.parametrize('shape', CFG5_SHAPES, ids=lambda s: 'x'.join(map(str, s)))
def test_cfg5_layer_shapes(shape):
    """bf16, batch 16, offsets/mask from a default-initialised 3x3 conv on the
    input (chunk / cat / sigmoid as in the Pack); first and last sample against
    the fp32 oracle on the same bf16 tensors."""
    C, H, W, stride = shape
    N = 16
    torch.manual_seed(5000 + C + stride)
    conv = torch.nn.Conv2d(C, 27, 3, stride=stride, padding=1).cuda().bfloat16()
    x = torch.randn(N, C, H, W, device='cuda').bfloat16()
    g = torch.Generator().manual_seed(C)
    w = (torch.randn(C, C, 3, 3, generator=g) * (2.0 / (C * 9)) ** 0.5).bfloat16().cuda()
    b = (torch.randn(C, generator=g) * 0.01).bfloat16().cuda()
    with torch.no_grad():
        raw = conv(x)
        o1, o2, m = torch.chunk(raw, 3, dim=1)
        off, msk = torch.cat((o1, o2), dim=1).contiguous(), torch.sigmoid(m).contiguous()
    case = dict(input=x, offset=off, mask=msk, weight=w, bias=b, stride=(stride, stride),
                padding=(1, 1), dilation=(1, 1), groups=1, deform_groups=1)
    y = capi_forward(case, path=capi.PATH_FUSED)
    assert torch.isfinite(y).all()
    for n in (0, N - 1):
        sub = dict(case)
        for k in ('input', 'offset', 'mask'):
            sub[k] = case[k][n:n + 1]
        err = rel_err(y[n:n + 1].float().cpu().numpy(), oracle_forward(sub))
        print(f'  cfg5 {shape} sample {n}: err {err:.3e}', flush=True)
        assert err <= TOL[torch.bfloat16], (shape, n, err)


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_empty_batch(dtype):
    """The reference's Python layer refuses an empty batch (its _output_size counts the
    batch among the sizes that must be positive, mmcv/ops/modulated_deform_conv.py:226-229);
    its extension op loops over the samples (modulated_deform_conv.cpp:108-130, :186-246)
    and with none returns without touching anything but the zeroed parameter gradients.
    Same here at both levels."""
    from mmcv_amd import _ext
    from mmcv_amd.ops import modulated_deform_conv2d
    x = torch.zeros(0, 64, 9, 11, dtype=dtype, device='cuda')
    off = torch.zeros(0, 18, 9, 11, dtype=dtype, device='cuda')
    msk = torch.zeros(0, 9, 9, 11, dtype=dtype, device='cuda')
    w = torch.randn(32, 64, 3, 3, dtype=dtype, device='cuda')
    b = torch.randn(32, dtype=dtype, device='cuda')
    with pytest.raises(ValueError, match='convolution input is too small'):
        modulated_deform_conv2d(x, off, msk, w, b, 1, 1, 1, 1, 1)
    geo = dict(kernel_h=3, kernel_w=3, stride_h=1, stride_w=1, pad_h=1, pad_w=1, dilation_h=1, dilation_w=1,
               group=1, deformable_group=1, with_bias=True)
    out = x.new_empty(0, 32, 9, 11)
    empty = x.new_empty(0)
    _ext.modulated_deform_conv_forward(x, w, b, empty, off, msk, out, empty, **geo)
    gw, gb = torch.full_like(w, 7.0), torch.full_like(b, 7.0)
    _ext.modulated_deform_conv_backward(x, w, b, empty, off, msk, empty, torch.zeros_like(x), gw, gb,
                                        torch.zeros_like(off), torch.zeros_like(msk), out, **geo)
    assert torch.count_nonzero(gw) == 0 and torch.count_nonzero(gb) == 0
    # mismatched shapes are still refused (the reference checks before it loops)
    with pytest.raises(RuntimeError, match="kernel channels won't match"):
        _ext.modulated_deform_conv_forward(x[:, :32], w, b, empty, off, msk, out, empty, **geo)
