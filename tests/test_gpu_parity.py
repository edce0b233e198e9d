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
