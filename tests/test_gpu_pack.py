"""Pack-level entry points (conv_offset + channel split + sigmoid + DCNv2) against
the CPU oracle, through the C ABI and through the module."""
import numpy as np
import pytest
import torch

from common import (TOL, capi, capi_forward, capi_pack_forward, cast_pack_case, make_pack_case,
                    oracle_conv_offset, oracle_forward, rel_err, split_raw)

pytestmark = pytest.mark.gpu

# (name, kwargs): channel counts that take the fused kernels for every dtype
# (multiples of 64) and ones that do not (direct kernels)
CASES = [
    ('c64_3x3', dict(N=2, Cin=64, Cout=64, H=13, W=17)),
    ('c128_s2', dict(N=2, Cin=128, Cout=96, H=20, W=15, stride=2)),
    ('c64_dil2', dict(N=1, Cin=64, Cout=32, H=16, W=18, padding=2, dilation=2)),
    ('c64_pad0', dict(N=1, Cin=64, Cout=64, H=9, W=11, padding=0)),
    ('c128_dg2', dict(N=2, Cin=128, Cout=128, H=10, W=12, deform_groups=2)),
    ('c256_dg4_g2', dict(N=1, Cin=256, Cout=64, H=8, W=9, deform_groups=4, groups=2)),
    ('c64_5x5', dict(N=1, Cin=64, Cout=48, H=12, W=12, k=5, padding=2)),
    ('c64_1x3', dict(N=1, Cin=64, Cout=64, H=7, W=21, k=(1, 3), padding=(0, 1))),
    ('c64_odd_tail', dict(N=3, Cin=64, Cout=64, H=11, W=13)),
    ('c64_wide_rows', dict(N=2, Cin=64, Cout=64, H=37, W=70)),
    ('c64_5x5_d3_s2_big_patch', dict(N=1, Cin=64, Cout=32, H=30, W=41, k=5, padding=6, dilation=3, stride=2)),
    ('c16_direct', dict(N=2, Cin=16, Cout=24, H=9, W=10)),
    ('c20_direct_dg2_s2', dict(N=1, Cin=20, Cout=10, H=12, W=9, stride=2, deform_groups=2)),
    # whole tiles of 256 pixels: the 256-pixel kernel reads offsets and mask logits from the raw tensor
    ('c128_wide_tiles', dict(N=2, Cin=128, Cout=128, H=24, W=24)),
    ('c256_wide_tiles', dict(N=1, Cin=256, Cout=256, H=16, W=32)),
]
DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def _np(t):
    return t.float().cpu().numpy()


@pytest.mark.parametrize('dtype', DTYPES, ids=['f32', 'bf16', 'f16'])
@pytest.mark.parametrize('name,kw', CASES, ids=[c[0] for c in CASES])
def test_pack_forward_against_oracle(name, kw, dtype):
    case = cast_pack_case(make_pack_case(900 + len(name), **kw), dtype)   # rounded, CPU
    dev = cast_pack_case(case, dtype, 'cuda')
    tol = TOL[dtype]
    y, raw = capi_pack_forward(dev, own_conv=True, want_raw=True)
    # (1) conv_offset alone
    raw_ref = oracle_conv_offset(case)
    e_raw = rel_err(_np(raw), raw_ref)
    # (2) the rest, fed with the raw tensor the device produced (already rounded)
    taps = case['weight'].shape[2] * case['weight'].shape[3]
    off, msk = split_raw(raw.cpu(), case['deform_groups'], taps)
    ref = oracle_forward(dict(case, offset=off, mask=msk))
    e_y = rel_err(_np(y), ref)
    # (3) end to end, offsets from the oracle's own conv_offset rounded to dtype
    off2, msk2 = split_raw(torch.from_numpy(raw_ref).to(dtype), case['deform_groups'], taps)
    ref2 = oracle_forward(dict(case, offset=off2, mask=msk2))
    e_e2e = rel_err(_np(y), ref2)
    print(f'  {name} {dtype}: raw {e_raw:.2e}  dcn {e_y:.2e}  end-to-end {e_e2e:.2e}', flush=True)
    assert e_raw <= tol, ('conv_offset', name, e_raw)
    assert e_y <= tol, ('dcn on device raw', name, e_y)
    assert e_e2e <= tol, ('end to end', name, e_e2e)
    # without the raw copy-out the result is the same
    y2, _ = capi_pack_forward(dev, own_conv=True, want_raw=False)
    assert torch.equal(y, y2)


@pytest.mark.parametrize('dtype', DTYPES, ids=['f32', 'bf16', 'f16'])
@pytest.mark.parametrize('name,kw', [CASES[0], CASES[4], CASES[6], CASES[9]], ids=lambda c: c if isinstance(c, str) else '')
def test_raw_input_mode_matches_unfused_sequence(name, kw, dtype):
    """raw computed by the caller: same result as chunk / cat / sigmoid by torch
    followed by the plain entry point (the only difference is the sigmoid's
    implementation, at most an ulp of dtype on a mask value)."""
    dev = cast_pack_case(make_pack_case(77, **kw), dtype, 'cuda')
    raw = torch.nn.functional.conv2d(dev['input'], dev['offset_weight'], dev['offset_bias'], dev['stride'],
                                     dev['padding'], dev['dilation'])
    taps = dev['weight'].shape[2] * dev['weight'].shape[3]
    off, msk = split_raw(raw, dev['deform_groups'], taps)
    y_ref = capi_forward(dict(dev, offset=off, mask=msk))
    y, _ = capi_pack_forward(dev, own_conv=False, raw=raw)
    err = rel_err(_np(y), _np(y_ref))
    print(f'  {name} {dtype}: fused split+sigmoid vs torch ops {err:.2e}', flush=True)
    assert err <= TOL[dtype] * 0.25


def test_module_fused_modes_agree():
    from mmcv_amd.ops import ModulatedDeformConv2dPack
    torch.manual_seed(3)
    layer = ModulatedDeformConv2dPack(64, 64, 3, stride=1, padding=1, deform_groups=1).cuda()
    torch.nn.init.normal_(layer.conv_offset.weight, std=0.05)
    torch.nn.init.normal_(layer.conv_offset.bias, std=0.5)
    x = torch.randn(2, 64, 14, 19, device='cuda')
    outs = {}
    with torch.no_grad():
        for mode in ('none', 'split', 'full'):
            layer.fuse = mode
            outs[mode] = layer(x)
    for mode in ('split', 'full'):
        err = rel_err(_np(outs[mode]), _np(outs['none']))
        print(f'  fuse={mode}: {err:.2e}', flush=True)
        assert err <= TOL[torch.float32]
    # a gradient-requiring call takes the reference sequence of differentiable ops
    layer.fuse = 'full'
    xg = x.clone().requires_grad_(True)
    y = layer(xg)
    assert rel_err(_np(y.detach()), _np(outs['none'])) == 0.0
    y.sum().backward()
    assert xg.grad is not None and layer.conv_offset.weight.grad is not None and layer.weight.grad is not None


def test_zero_init_pack_is_plain_conv():
    """conv_offset starts at zero: offsets 0, mask 0.5 (sigmoid(0)), so the layer
    is half a plain convolution plus bias (mmcv/ops/modulated_deform_conv.py:321-325)."""
    from mmcv_amd.ops import ModulatedDeformConv2dPack
    torch.manual_seed(4)
    layer = ModulatedDeformConv2dPack(64, 32, 3, padding=1).cuda()
    x = torch.randn(1, 64, 10, 12, device='cuda')
    with torch.no_grad():
        y = layer(x)
        ref = 0.5 * torch.nn.functional.conv2d(x, layer.weight, None, 1, 1) + layer.bias.view(1, -1, 1, 1)
    assert rel_err(_np(y), _np(ref)) <= TOL[torch.float32]


def test_pack_errors():
    import ctypes
    lib = capi.load()
    pp = capi.MdcnPackParams()
    pp.conv = capi.make_params(capi.MDCN_F32, 1, 64, 8, 8, 64, 3, 3, (1, 1), (1, 1))
    assert lib.mdcn_pack_forward(None, None) == -1
    # no pointers at all
    assert lib.mdcn_pack_forward(ctypes.byref(pp), None) == -1
    assert lib.mdcn_pack_workspace_bytes(ctypes.byref(pp)) > 0
