"""Deformable convolution without modulation (DCNv1) on the device: the C ABI with
mask == NULL, the extension op, the modules and the pack-level call, against the
CPU oracle run with a mask of ones (the reference's two samplers are the same
function) and the reference's known-answer test."""
import numpy as np
import pytest
import torch

from common import (TOL, capi, capi_forward, capi_pack_forward, cast_case, cast_pack_case, make_case,
                    make_pack_case, oracle_conv_offset, oracle_forward, rel_err)

pytestmark = pytest.mark.gpu

CASES = [
    ('c64', dict(N=2, Cin=64, Cout=64, H=13, W=17)),
    ('c128_s2_dg2', dict(N=2, Cin=128, Cout=96, H=20, W=15, stride=2, deform_groups=2)),
    ('c64_g2_dil2', dict(N=1, Cin=128, Cout=64, H=16, W=18, padding=2, dilation=2, groups=2)),
    ('c12_direct', dict(N=3, Cin=12, Cout=10, H=9, W=10, deform_groups=3)),
]
DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def _np(t):
    return t.float().cpu().numpy()


@pytest.mark.parametrize('dtype', DTYPES, ids=['f32', 'bf16', 'f16'])
@pytest.mark.parametrize('name,kw', CASES, ids=[c[0] for c in CASES])
def test_unmodulated_forward_against_oracle(name, kw, dtype):
    case = cast_case(make_case(300 + len(name), bias=False, **kw), dtype)
    ref = oracle_forward(dict(case, mask=torch.ones_like(case['mask'])))
    dev = cast_case(case, dtype, 'cuda')
    dev['mask'] = None
    for path in (capi.PATH_AUTO, capi.PATH_DIRECT):
        y = capi_forward(dev, path=path)
        err = rel_err(_np(y), ref)
        print(f'  {name} {dtype} path {path}: {err:.2e}', flush=True)
        assert err <= TOL[dtype]


# mmcv tests/test_ops/test_deform_conv.py:27-35,47: the layer's known answer
KAT_INPUT = [[[[1., 2., 3.], [0., 1., 2.], [3., 5., 2.]]]]
KAT_OFFSET_WEIGHT = [[[0.1, 0.4, 0.6, 0.1]], [[0.3, 0.2, 0.1, 0.3]], [[0.5, 0.5, 0.2, 0.8]],
                     [[0.8, 0.3, 0.9, 0.1]], [[0.3, 0.1, 0.2, 0.5]], [[0.3, 0.7, 0.5, 0.3]],
                     [[0.6, 0.2, 0.5, 0.3]], [[0.4, 0.1, 0.8, 0.4]]]
KAT_OFFSET_BIAS = [0.7, 0.1, 0.8, 0.5, 0.6, 0.5, 0.4, 0.7]
KAT_WEIGHT = [[[0.4, 0.2, 0.1, 0.9]]]
KAT_OUT = [[[[1.650, 0.], [0.000, 0.]]]]


@pytest.mark.parametrize('fuse', ['full', 'none'])
@pytest.mark.parametrize('dtype,threshold', [(torch.float32, 1e-3), (torch.float16, 1e-2), (torch.bfloat16, 3e-2)],
                         ids=['f32', 'f16', 'bf16'])
def test_reference_known_answer_through_the_pack(dtype, threshold, fuse):
    from mmcv_amd.ops import DeformConv2dPack
    batch = 10
    x = torch.tensor(np.repeat(KAT_INPUT, batch, axis=0), device='cuda', dtype=dtype)
    model = DeformConv2dPack(in_channels=1, out_channels=1, kernel_size=2, stride=1, padding=0, im2col_step=2)
    model.conv_offset.weight.data = torch.Tensor(KAT_OFFSET_WEIGHT).reshape(8, 1, 2, 2)
    model.conv_offset.bias.data = torch.Tensor(KAT_OFFSET_BIAS).reshape(8)
    model.weight.data = torch.Tensor(KAT_WEIGHT).reshape(1, 1, 2, 2)
    model.cuda().type(dtype)
    model.fuse = fuse
    with torch.no_grad():
        out = model(x)
    assert out.dtype == dtype
    assert np.allclose(_np(out), np.repeat(KAT_OUT, batch, axis=0), threshold, threshold)


@pytest.mark.parametrize('dtype', DTYPES, ids=['f32', 'bf16', 'f16'])
@pytest.mark.parametrize('kw', [dict(N=2, Cin=64, Cout=64, H=13, W=17), dict(N=1, Cin=128, Cout=64, H=12, W=9, stride=2, deform_groups=2),
                                dict(N=2, Cin=10, Cout=6, H=8, W=8)], ids=['c64', 'c128_s2_dg2', 'c10_direct'])
def test_unmodulated_pack_against_oracle(kw, dtype):
    case = cast_pack_case(make_pack_case(41, unmodulated=True, **kw), dtype)
    dev = cast_pack_case(case, dtype, 'cuda')
    dev['bias'] = None
    y, raw = capi_pack_forward(dev, want_raw=True, unmodulated=True)
    assert rel_err(_np(raw), oracle_conv_offset(case)) <= TOL[dtype]
    off = raw.cpu()
    ref = oracle_forward(dict(case, offset=off, mask=torch.ones(off.shape[0], off.shape[1] // 2, *off.shape[2:]), bias=None))
    err = rel_err(_np(y), ref)
    print(f'  {kw} {dtype}: {err:.2e}', flush=True)
    assert err <= TOL[dtype]


def test_module_behaviour():
    from mmcv_amd.ops import MODELS, DeformConv2d, DeformConv2dPack, deform_conv2d
    assert MODELS.get('DCN') is DeformConv2dPack
    torch.manual_seed(0)
    layer = DeformConv2d(64, 32, 3, padding=1, deform_groups=2).cuda()
    assert not hasattr(layer, 'bias')
    x = torch.randn(4, 64, 9, 11, device='cuda')
    offset = torch.randn(4, 2 * 2 * 9, 9, 11, device='cuda')
    with torch.no_grad():
        y = layer(x, offset)
        ref = oracle_forward(dict(input=x.cpu(), offset=offset.cpu(), mask=torch.ones(4, 18, 9, 11),
                                  weight=layer.weight.detach().cpu(), bias=None, stride=(1, 1), padding=(1, 1),
                                  dilation=(1, 1), groups=1, deform_groups=2))
    assert rel_err(_np(y), ref) <= TOL[torch.float32]
    # zero offsets: a plain convolution
    with torch.no_grad():
        y0 = layer(x, torch.zeros_like(offset))
        assert rel_err(_np(y0), _np(torch.nn.functional.conv2d(x, layer.weight, None, 1, 1))) <= TOL[torch.float32]
    # batch not divisible by im2col_step
    with pytest.raises(AssertionError, match='divisible by im2col_step'):
        deform_conv2d(x[:3], offset[:3], layer.weight, 1, 1, 1, 1, 2, False, 2)
    # an input smaller than the kernel is padded and the output cropped
    small = DeformConv2d(64, 8, 3, padding=1).cuda()
    xs = torch.randn(1, 64, 2, 5, device='cuda')
    with torch.no_grad():
        ys = small(xs, torch.zeros(1, 18, 2, 5, device='cuda'))
    assert ys.shape == (1, 8, 2, 5)
    # a gradient-requiring call takes the reference's two differentiable steps
    pack = DeformConv2dPack(64, 8, 3, padding=1).cuda()
    xg = x.clone().requires_grad_(True)
    pack(xg).sum().backward()
    assert xg.grad is not None and pack.weight.grad is not None and pack.conv_offset.bias.grad is not None
    # CPU tensors are refused
    with pytest.raises(RuntimeError, match='implementation for device cpu not found'):
        deform_conv2d(x.detach().cpu(), offset.cpu(), layer.weight.detach().cpu(), 1, 1, 1, 1, 2, False, 4)
