"""Seeded sweep over random geometries: kernel size, stride, padding, dilation,
groups, deformable groups, channel counts on and off the fused paths' grid,
plane sizes that are not multiples of any tile.  Forward (automatic path choice
and the direct kernel), pack-level forward and backward (automatic choice and
forced tiled kernels) against the CPU oracle."""
import random

import pytest
import torch

import oracle
from mmcv_amd import capi
from common import (TOL, capi_backward, capi_forward, capi_pack_forward, cast_case, cast_pack_case, make_case,
                    make_pack_case, oracle_conv_offset, oracle_forward, rel_err, split_raw)

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def random_geometry(rng, max_px=400):
    """A valid layer geometry with at least one output pixel."""
    while True:
        kh, kw = rng.choice([(1, 1), (3, 3), (3, 3), (3, 3), (1, 3), (3, 1), (2, 2), (5, 5)])
        groups = rng.choice([1, 1, 1, 2, 4])
        dgroups = rng.choice([1, 1, 2, 3, 4])
        unit = groups * dgroups // __import__('math').gcd(groups, dgroups)
        base = rng.choice([1, 2, 4, 8, 16, 32, 64])
        Cin = unit * base
        if Cin > 384:
            continue
        Cout = groups * rng.choice([1, 3, 8, 16, 32, 64, 80])
        if Cout > 320:
            continue
        stride = (rng.choice([1, 1, 2]), rng.choice([1, 1, 2]))
        dilation = (rng.choice([1, 1, 2]), rng.choice([1, 1, 2]))
        padding = (rng.randint(0, 2), rng.randint(0, 2))
        H, W = rng.randint(2, 26), rng.randint(2, 26)
        Ho = (H + 2 * padding[0] - (dilation[0] * (kh - 1) + 1)) // stride[0] + 1
        Wo = (W + 2 * padding[1] - (dilation[1] * (kw - 1) + 1)) // stride[1] + 1
        if Ho < 1 or Wo < 1 or Ho * Wo > max_px:
            continue
        return dict(N=rng.randint(1, 3), Cin=Cin, Cout=Cout, H=H, W=W, k=(kh, kw), stride=stride, padding=padding,
                    dilation=dilation, groups=groups, deform_groups=dgroups,
                    sigma=rng.choice([0.5, 2.0, 2.0, 5.0]))


def _np(t):
    return t.float().cpu().numpy()


@pytest.mark.parametrize('seed', range(72))
def test_forward_random_geometry(seed):
    rng = random.Random(1000 + seed)
    kw = random_geometry(rng)
    dtype = DTYPES[seed % 3]
    case = cast_case(make_case(seed, bias=rng.random() < 0.7, **kw), dtype)
    ref = oracle_forward(case)
    dev = cast_case(case, dtype, 'cuda')
    print(f'  {kw} {dtype}', flush=True)
    for path in (capi.PATH_AUTO, capi.PATH_DIRECT):
        err = rel_err(_np(capi_forward(dev, path=path)), ref)
        assert err <= TOL[dtype], (path, err)
    if rng.random() < 0.5:  # without a mask
        ref1 = oracle_forward(dict(case, mask=torch.ones_like(case['mask'])))
        err = rel_err(_np(capi_forward(dict(dev, mask=None))), ref1)
        assert err <= TOL[dtype], ('dcnv1', err)


@pytest.mark.parametrize('seed', range(36))
def test_pack_forward_random_geometry(seed):
    rng = random.Random(2000 + seed)
    kw = random_geometry(rng)
    kw.pop('sigma')
    dtype = DTYPES[seed % 3]
    unmodulated = seed % 2 == 1
    case = cast_pack_case(make_pack_case(seed, unmodulated=unmodulated, **kw), dtype)
    dev = cast_pack_case(case, dtype, 'cuda')
    print(f'  {kw} {dtype} unmodulated={unmodulated}', flush=True)
    y, raw = capi_pack_forward(dev, want_raw=True, unmodulated=unmodulated)
    assert rel_err(_np(raw), oracle_conv_offset(case)) <= TOL[dtype]
    # the main stage against the oracle fed with the device's own conv_offset output
    if unmodulated:
        off = raw.cpu()
        msk = torch.ones(off.shape[0], off.shape[1] // 2, *off.shape[2:])
    else:
        off, msk = split_raw(raw.cpu(), kw['deform_groups'], kw['k'][0] * kw['k'][1])
    ref = oracle_forward(dict(case, offset=off, mask=msk))
    err = rel_err(_np(y), ref)
    assert err <= TOL[dtype], err


@pytest.mark.parametrize('seed', range(48))
def test_backward_random_geometry(seed):
    rng = random.Random(3000 + seed)
    while True:
        kw = random_geometry(rng, max_px=300)
        if kw['Cin'] <= 128:   # (the oracle's backward is a scalar loop nest)
            break
    if seed % 2 == 0:          # every other case on the matrix-core kernels' channel grid
        kw['groups'] = rng.choice([1, 2])
        kw['deform_groups'] = rng.choice([1, 2, 4])
        kw['Cin'] = 64 * kw['groups']
        kw['Cout'] = 64 * kw['groups'] * rng.choice([1, 2])
    dtype = DTYPES[(seed // 2) % 3]
    modulated = seed % 3 != 0
    case = cast_case(make_case(seed, bias=False, **kw), dtype)
    if not modulated:
        case['mask'] = torch.ones_like(case['mask'])
    Ho, Wo = case['offset'].shape[2:]
    gy = torch.randn(kw['N'], kw['Cout'], Ho, Wo, generator=torch.Generator().manual_seed(seed)).to(dtype)
    geo = dict(stride=case['stride'], padding=case['padding'], dilation=case['dilation'],
               groups=case['groups'], deform_groups=case['deform_groups'])
    ref = oracle.backward(*[case[k].float().numpy() for k in ('input', 'offset', 'mask', 'weight')],
                          gy.float().numpy(), True, **geo)
    dev = cast_case(case, dtype, 'cuda')
    if not modulated:
        dev['mask'] = None
    print(f'  {kw} {dtype} modulated={modulated}', flush=True)
    lib = capi.load()
    for path in (capi.PATH_AUTO, capi.PATH_FUSED):
        try:
            got = capi_backward(dev, gy.cuda(), path=path)
        except AssertionError as e:   # the forced tiled kernels do not cover every geometry
            assert path == capi.PATH_FUSED and 'not covered' in str(e), e
            continue
        for nm, r, o in zip(('grad_input', 'grad_offset', 'grad_mask', 'grad_weight', 'grad_bias'), ref, got):
            if o is None:
                continue
            err = rel_err(_np(o), r)
            assert err <= TOL[dtype], (path, nm, err)
