"""GPU parity: the HIP paths, called through the C ABI, against the CPU oracle
on the same seeded inputs.

Error metric everywhere: max|y - y_ref| / max|y_ref| over the whole output.
Bars: fp32 <= 1e-4; bf16 / fp16 <= 2e-2 against the fp32 oracle fed the same
(rounded) inputs."""
import numpy as np
import pytest
import torch

from mmcv_amd import capi

from common import (TOL, capi_forward, cast_case, make_case, oracle_forward,
                    rel_err)

pytestmark = pytest.mark.gpu

# name: (kwargs of make_case)
SMALL = {
    'base': dict(N=2, Cin=64, Cout=64, H=13, W=17),
    'cout_tail': dict(N=1, Cin=64, Cout=80, H=9, W=31),
    'stride2': dict(N=2, Cin=64, Cout=64, H=20, W=22, stride=2),
    'dil2': dict(N=1, Cin=64, Cout=32, H=15, W=15, dilation=2, padding=2),
    'groups2': dict(N=2, Cin=128, Cout=128, H=12, W=12, groups=2),
    'dg2': dict(N=2, Cin=128, Cout=64, H=12, W=14, deform_groups=2),
    'groups2_dg4': dict(N=1, Cin=256, Cout=256, H=10, W=11, groups=2, deform_groups=4),
    'dg3_misaligned': dict(N=1, Cin=384, Cout=64, H=9, W=10, groups=2, deform_groups=3),
    'three_slabs': dict(N=1, Cin=192, Cout=64, H=11, W=9),
    'k1': dict(N=2, Cin=64, Cout=32, H=8, W=9, k=1, padding=0),
    'k1_dg2': dict(N=1, Cin=128, Cout=32, H=8, W=9, k=1, padding=0, deform_groups=2),
    'k5': dict(N=1, Cin=64, Cout=32, H=11, W=12, k=5, padding=2),
    'k5_cout256': dict(N=1, Cin=64, Cout=256, H=7, W=8, k=5, padding=2),
    'k3x1': dict(N=1, Cin=64, Cout=32, H=11, W=12, k=(3, 1), padding=(1, 0)),
    'nobias': dict(N=1, Cin=64, Cout=192, H=16, W=16, bias=False),
    'far_offsets': dict(N=1, Cin=64, Cout=32, H=10, W=10, sigma=8.0),
    'cout256': dict(N=1, Cin=64, Cout=256, H=14, W=14),
    'cout512': dict(N=1, Cin=64, Cout=512, H=9, W=9),
    'cout384_dg2': dict(N=2, Cin=128, Cout=384, H=9, W=11, deform_groups=2),
    'cout640_s2': dict(N=1, Cin=64, Cout=640, H=13, W=15, stride=2),
    'cout1024_g2': dict(N=1, Cin=128, Cout=1024, H=8, W=10, groups=2),
    'pad0': dict(N=1, Cin=64, Cout=32, H=9, W=9, padding=0),
    'asym': dict(N=1, Cin=64, Cout=32, H=17, W=12, stride=(2, 1), padding=(0, 2), dilation=(1, 2)),
    'odd_plane': dict(N=3, Cin=64, Cout=64, H=7, W=9),
    'many_tiles': dict(N=5, Cin=64, Cout=64, H=33, W=35),
}

ODD = {  # shapes only the direct kernel covers
    'c3': dict(N=2, Cin=3, Cout=5, H=7, W=8),
    'c1': dict(N=1, Cin=1, Cout=1, H=3, W=3, k=2, padding=1),
    'c24_g3': dict(N=1, Cin=24, Cout=9, H=9, W=8, groups=3, deform_groups=2),
    'c32': dict(N=1, Cin=32, Cout=32, H=9, W=8),
}


def run_case(kw, dtype, path, seed=7):
    case = make_case(seed, **kw)
    dev = cast_case(case, dtype, 'cuda')
    y = capi_forward(dev, path=path).float().cpu().numpy()
    ref = oracle_forward(cast_case(case, dtype))  # fp32 oracle on the rounded inputs
    return rel_err(y, ref)


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('name', sorted(SMALL))
def test_fused_small(name, dtype):
    print(f'case={name} dtype={dtype}', flush=True)
    err = run_case(SMALL[name], dtype, capi.PATH_FUSED)
    assert err <= TOL[dtype], err


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('name', sorted(SMALL) + sorted(ODD))
def test_direct_small(name, dtype):
    print(f'case={name} dtype={dtype}', flush=True)
    kw = SMALL.get(name) or ODD[name]
    err = run_case(kw, dtype, capi.PATH_DIRECT)
    assert err <= TOL[dtype], err


def test_auto_picks_direct_for_odd_channels():
    lib = capi.load()
    import ctypes
    p = capi.make_params(capi.MDCN_F32, 1, 3, 7, 8, 5, 3, 3, (1, 1), (1, 1))
    assert lib.mdcn_fused_eligible(ctypes.byref(p)) == 0
    assert lib.mdcn_workspace_bytes(ctypes.byref(p)) == 0
    p.path = capi.PATH_FUSED
    x = torch.zeros(1, device='cuda')
    p.input = p.offset = p.mask = p.weight = p.output = x.data_ptr()
    assert lib.mdcn_forward(ctypes.byref(p), None) == -5  # MDCN_ERR_PATH


# Shapes that reach the eight-wave streaming kernel (16-bit tensors, more than 128 output channels per group,
# one deformable group, at least 18 K steps), chosen so that workgroups walk several tiles, tiles end inside
# an image, images end inside a tile and the padded step count differs from the real one.
STREAM = {
    'many_tiles': dict(N=4, Cin=128, Cout=256, H=96, W=96),                 # 288 tiles on 256 workgroups
    'ragged': dict(N=3, Cin=192, Cout=200, H=61, W=53, sigma=3.0),          # 27 steps padded to 30, odd plane
    'stride2_groups': dict(N=2, Cin=256, Cout=512, H=37, W=41, stride=2, groups=2),
    'dilated_far': dict(N=1, Cin=128, Cout=384, H=30, W=34, dilation=2, padding=2, sigma=9.0),
    'k1x3': dict(N=2, Cin=384, Cout=256, H=20, W=24, k=(1, 3), padding=(0, 1)),
}


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('name', sorted(STREAM))
def test_streaming_kernel(name, dtype):
    """Default fused path (streaming kernel) against the oracle and against the
    specialised-wave kernel on the same inputs."""
    print(f'case={name} dtype={dtype}', flush=True)
    case = make_case(11, **STREAM[name])
    dev = cast_case(case, dtype, 'cuda')
    y = capi_forward(dev, path=capi.PATH_FUSED)
    y_split = capi_forward(dev, path=capi.PATH_FUSED_SPLIT)
    ref = oracle_forward(cast_case(case, dtype))
    assert rel_err(y.float().cpu().numpy(), ref) <= TOL[dtype]
    assert rel_err(y_split.float().cpu().numpy(), ref) <= TOL[dtype]
    assert rel_err(y.float().cpu().numpy(), y_split.float().cpu().numpy()) <= TOL[dtype]


@pytest.mark.parametrize('path', [capi.PATH_FUSED, capi.PATH_FUSED_SPLIT, capi.PATH_DIRECT])
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_outside_taps_never_touch_the_image(path, dtype):
    """A tap whose position lies outside (-1, H) x (-1, W) adds nothing in the
    reference (cpu/modulated_deform_conv.cpp:160-164), whatever the image holds:
    Inf / NaN in the corner pixels must not leak into outputs whose taps that
    would touch them are all outside."""
    kw = dict(N=2, Cin=128, Cout=256, H=24, W=28)
    case = make_case(5, **kw)
    # every tap of every pixel far outside, except the lower right quarter of the plane, which samples
    # around its own position (away from the poisoned corner)
    off = case['offset']
    off[:] = 1000.0
    off[:, :, 12:, 14:] = torch.randn(off[:, :, 12:, 14:].shape, generator=torch.Generator().manual_seed(3)) * 0.5
    case['input'][:, :, 0:2, 0:2] = float('inf')
    case['input'][:, 1::2, 0, 0] = float('nan')
    clean = dict(case)
    clean['input'] = case['input'].clone()
    clean['input'][:, :, 0:2, 0:2] = 0.0  # nothing in the oracle run may depend on these pixels
    ref = oracle_forward(cast_case(clean, dtype))
    y = capi_forward(cast_case(case, dtype, 'cuda'), path=path).float().cpu().numpy()
    assert np.isfinite(y).all()
    assert rel_err(y, ref) <= TOL[dtype]


@pytest.mark.parametrize('path', [capi.PATH_FUSED, capi.PATH_FUSED_SPLIT, capi.PATH_DIRECT])
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
def test_non_finite_offsets_are_outside(path, dtype):
    """An offset that is NaN or infinite fails the reference's position test
    (cpu/modulated_deform_conv.cpp:160: every comparison with NaN is false), so
    the tap adds nothing and nothing is read for it.  A third of the taps get
    such offsets here; the rest sample normally."""
    kw = dict(N=2, Cin=128, Cout=256, H=20, W=26, sigma=1.5)
    print(f'path={path} dtype={dtype} non-finite offsets', flush=True)
    case = make_case(9, **kw)
    off = case['offset']
    g = torch.Generator().manual_seed(4)
    kind = torch.randint(0, 9, off.shape, generator=g)
    off[kind == 0] = float('nan')
    off[kind == 1] = float('inf')
    off[kind == 2] = float('-inf')
    ref = oracle_forward(cast_case(case, dtype))
    assert np.isfinite(ref).all()
    y = capi_forward(cast_case(case, dtype, 'cuda'), path=path).float().cpu().numpy()
    assert np.isfinite(y).all()
    assert rel_err(y, ref) <= TOL[dtype]


# Tiles of the schedule's last round cut along K (both fused kernels): shapes whose tile counts give
# two, three and four parts per tile on a 256-CU grid, and one with whole rounds in front of the cut one.
CUT = {
    'eight_wave_4_parts': (dict(N=1, Cin=256, Cout=256, H=12, W=20), [torch.bfloat16, torch.float16]),       # 2 tiles
    'eight_wave_3_parts': (dict(N=5, Cin=256, Cout=256, H=32, W=64), [torch.bfloat16]),                       # 80 tiles: 10 per XCD
    'eight_wave_2_parts': (dict(N=8, Cin=256, Cout=256, H=32, W=56), [torch.bfloat16]),                       # 112 tiles: 14 per XCD
    'eight_wave_rounds_then_cut': (dict(N=16, Cin=256, Cout=256, H=48, W=50), [torch.bfloat16]),              # 300 tiles: 32 + 6 per XCD
    'eight_wave_two_ctiles': (dict(N=2, Cin=128, Cout=512, H=16, W=24), [torch.float16]),                      # 6 x 2 tiles
    'specialised_fp32_4_parts': (dict(N=1, Cin=256, Cout=256, H=16, W=16), [torch.float32]),                   # 72 steps
    'specialised_fp32_dg4_s2': (dict(N=2, Cin=512, Cout=512, H=20, W=20, stride=2, deform_groups=4), [torch.float32]),
    'specialised_c128': (dict(N=4, Cin=128, Cout=128, H=24, W=40), [torch.bfloat16, torch.float32]),
    'specialised_c64_25_taps': (dict(N=2, Cin=128, Cout=64, H=16, W=16, k=5, padding=2), [torch.float16]),
}


@pytest.mark.parametrize('name', sorted(CUT))
def test_tiles_cut_along_k(name):
    """Cut and uncut runs both meet the oracle, agree with one another to fp32 rounding of the sums, and the
    cut run gives the same bits every time (the parts are added in a fixed order)."""
    kw, dtypes = CUT[name]
    for dtype in dtypes:
        case = make_case(31, **kw)
        dev = cast_case(case, dtype, 'cuda')
        ref = oracle_forward(cast_case(case, dtype))
        y_cut = capi_forward(dev, path=capi.PATH_FUSED)
        y_one = capi_forward(dev, path=capi.PATH_FUSED, unsplit=True)
        assert rel_err(y_cut.float().cpu().numpy(), ref) <= TOL[dtype]
        assert rel_err(y_one.float().cpu().numpy(), ref) <= TOL[dtype]
        diff = float((y_cut.float() - y_one.float()).abs().max() / y_one.float().abs().max())
        print(f'  {name} {dtype}: cut vs uncut {diff:.2e}', flush=True)
        assert diff <= (1e-5 if dtype == torch.float32 else 8e-3)
        for _ in range(3):
            assert torch.equal(capi_forward(dev, path=capi.PATH_FUSED), y_cut)


# Shapes that have the kernel with 256-pixel tiles (16-bit tensors, one deformable group, whole channel
# tiles of 256, an even number of K steps, planes of whole 16-byte runs): workgroups that walk several
# tiles, waves whose 64 pixels cross an image boundary, two groups, two channel tiles, stride 2, and a
# pixel count that leaves a rest for the 128-pixel kernel launched beside it.
WIDE = {
    'tiles_and_rest': dict(N=2, Cin=256, Cout=256, H=24, W=24),            # 4 tiles of 256 + 128 pixels
    'one_tile': dict(N=1, Cin=128, Cout=256, H=16, W=16),                  # 18 K steps, exactly one tile
    'images_inside_a_wave': dict(N=3, Cin=256, Cout=256, H=20, W=24, sigma=4.0),
    'two_groups': dict(N=2, Cin=512, Cout=512, H=16, W=24, groups=2),
    'two_channel_tiles': dict(N=2, Cin=128, Cout=512, H=16, W=16),
    'stride2': dict(N=2, Cin=128, Cout=256, H=33, W=32, stride=2),
    'several_tiles_per_workgroup': dict(N=9, Cin=128, Cout=256, H=96, W=88),  # 297 tiles on 256 workgroups
    'channel_tile_128': dict(N=2, Cin=128, Cout=128, H=24, W=24),           # the 128-channel variant of the tile
    'channel_tile_128_two_groups': dict(N=3, Cin=256, Cout=256, H=16, W=24, groups=2, sigma=3.0),
    'channel_tile_128_stride2': dict(N=2, Cin=256, Cout=128, H=31, W=32, stride=2, bias=False),
    'no_bias_k1x3': dict(N=2, Cin=512, Cout=256, H=16, W=24, k=(1, 3), padding=(0, 1), bias=False),  # 24 K steps
}


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('name', sorted(WIDE))
def test_wide_tile_kernel(name, dtype):
    """Every whole tile of 256 pixels through the 256-pixel kernel: against the oracle, and bit for bit
    against the 128-pixel kernel (the two sum a tile's K range in the same order)."""
    print(f'case={name} dtype={dtype}', flush=True)
    case = make_case(777, **WIDE[name])
    dev = cast_case(case, dtype, 'cuda')
    ref = oracle_forward(cast_case(case, dtype))
    y = capi_forward(dev, path=capi.PATH_FUSED_WIDE, unsplit=True)
    y_narrow = capi_forward(dev, path=capi.PATH_FUSED_NARROW, unsplit=True)
    assert rel_err(y.float().cpu().numpy(), ref) <= TOL[dtype]
    assert torch.equal(y, y_narrow)
    # (... and with the rest's tiles cut along K by the 128-pixel kernel)
    y_cut = capi_forward(dev, path=capi.PATH_FUSED_WIDE)
    assert rel_err(y_cut.float().cpu().numpy(), ref) <= TOL[dtype]


def test_wide_tile_kernel_needs_its_shape():
    """MDCN_PATH_FUSED_WIDE is an error where the shape has no 256-pixel kernel (fp32; channel tiles that
    are not whole; several deformable groups); the default path takes such shapes elsewhere."""
    import ctypes
    lib = capi.load()
    x = torch.zeros(1, device='cuda')
    for dt, kw in ((capi.MDCN_F32, dict(Cin=256, Cout=256)), (capi.MDCN_BF16, dict(Cin=256, Cout=200)),
                   (capi.MDCN_BF16, dict(Cin=256, Cout=256, dg=2)), (capi.MDCN_BF16, dict(Cin=64, Cout=256))):
        p = capi.make_params(dt, 1, kw['Cin'], 16, 16, kw['Cout'], 3, 3, (1, 1), (1, 1), (1, 1), 1, kw.get('dg', 1),
                             capi.PATH_FUSED_WIDE)
        p.input = p.offset = p.mask = p.weight = p.output = x.data_ptr()
        assert lib.mdcn_workspace_bytes(ctypes.byref(p)) == 0
        assert lib.mdcn_forward(ctypes.byref(p), None) == -5, kw  # MDCN_ERR_PATH
