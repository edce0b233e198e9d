"""Pins the CPU oracle (oracle/mdcn_oracle.c) before anything is compared with it.

Independent anchors, chosen so that a dropped term, a swapped (dy, dx), a wrong
tap order, a clamped instead of zeroed corner or a transposed weight fails one:
  * the reference's own known-answer vectors (tests/golden/reference_kats.json),
  * outputs of the reference's compiled C++ (tests/golden/ref_cases.npz, and
    oracle/_ref live when it is built),
  * zero offsets + unit mask  ==  zero-padded F.conv2d,
  * general case == F.grid_sample(bilinear, zeros, align_corners=True) + einsum,
  * a float64 brute-force loop over the definition on tiny shapes,
  * sampler edge cases on and next to the (-1, H) x (-1, W) boundary.
"""
import json
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from common import make_case, out_hw, pair, rel_err

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden')


def np_case(case, dtype):
    f = lambda t: None if t is None else t.numpy().astype(dtype)
    return (f(case['input']), f(case['offset']), f(case['mask']), f(case['weight']),
            f(case['bias']), case['stride'], case['padding'], case['dilation'],
            case['groups'], case['deform_groups'])


# ---- independent definitions ------------------------------------------------

def brute_force(x, offset, mask, weight, bias, stride, padding, dilation, groups,
                dg):
    """float64 loops straight from the definition: y-offset first, taps
    row-major, each of the 4 corners contributes only when inside the image."""
    x = x.astype(np.float64)
    N, Cin, H, W = x.shape
    Cout, cin_g, kh, kw = weight.shape
    (sh, sw), (ph, pw), (dh, dw) = pair(stride), pair(padding), pair(dilation)
    Ho, Wo = out_hw(H, W, kh, kw, stride, padding, dilation)
    cout_g = Cout // groups
    cpd = Cin // dg
    y = np.zeros((N, Cout, Ho, Wo))

    def px(n, c, yy, xx):
        return x[n, c, yy, xx] if (0 <= yy < H and 0 <= xx < W) else 0.0

    for n in range(N):
        for ho in range(Ho):
            for wo in range(Wo):
                for co in range(Cout):
                    g = co // cout_g
                    acc = 0.0
                    for cl in range(cin_g):
                        c = g * cin_g + cl
                        d = c // cpd
                        for i in range(kh):
                            for j in range(kw):
                                t = i * kw + j
                                oy = float(offset[n, d * 2 * kh * kw + 2 * t, ho, wo])
                                ox = float(offset[n, d * 2 * kh * kw + 2 * t + 1, ho, wo])
                                m = float(mask[n, d * kh * kw + t, ho, wo])
                                py = ho * sh - ph + i * dh + oy
                                pxx = wo * sw - pw + j * dw + ox
                                y0, x0 = int(np.floor(py)), int(np.floor(pxx))
                                ly, lx = py - y0, pxx - x0
                                s = ((1 - ly) * (1 - lx) * px(n, c, y0, x0) +
                                     (1 - ly) * lx * px(n, c, y0, x0 + 1) +
                                     ly * (1 - lx) * px(n, c, y0 + 1, x0) +
                                     ly * lx * px(n, c, y0 + 1, x0 + 1))
                                acc += float(weight[co, cl, i, j]) * s * m
                    y[n, co, ho, wo] = acc + (float(bias[co]) if bias is not None else 0.0)
    return y


def grid_sample_forward(x, offset, mask, weight, bias, stride, padding, dilation,
                        groups, dg):
    """Library-routine formulation in float64: per tap, zero-padded bilinear
    F.grid_sample at the absolute positions, times mask; then a grouped
    contraction with weight.flatten(1)."""
    x = torch.as_tensor(x, dtype=torch.float64)
    offset = torch.as_tensor(offset, dtype=torch.float64)
    mask = torch.as_tensor(mask, dtype=torch.float64)
    weight = torch.as_tensor(weight, dtype=torch.float64)
    N, Cin, H, W = x.shape
    Cout, cin_g, kh, kw = weight.shape
    (sh, sw), (ph, pw), (dh, dw) = pair(stride), pair(padding), pair(dilation)
    Ho, Wo = out_hw(H, W, kh, kw, stride, padding, dilation)
    cpd = Cin // dg
    ys = (torch.arange(Ho, dtype=torch.float64) * sh - ph).view(1, Ho, 1)
    xs = (torch.arange(Wo, dtype=torch.float64) * sw - pw).view(1, 1, Wo)
    col = torch.zeros(N, Cin, kh * kw, Ho, Wo, dtype=torch.float64)
    for d in range(dg):
        for i in range(kh):
            for j in range(kw):
                t = i * kw + j
                py = ys + i * dh + offset[:, d * 2 * kh * kw + 2 * t]
                px = xs + j * dw + offset[:, d * 2 * kh * kw + 2 * t + 1]
                grid = torch.stack([2 * px / (W - 1) - 1, 2 * py / (H - 1) - 1], dim=-1)
                s = F.grid_sample(x[:, d * cpd:(d + 1) * cpd], grid, mode='bilinear',
                                  padding_mode='zeros', align_corners=True)
                col[:, d * cpd:(d + 1) * cpd, t] = s * mask[:, d * kh * kw + t].unsqueeze(1)
    col = col.view(N, groups, cin_g * kh * kw, Ho * Wo)
    w = weight.view(groups, Cout // groups, cin_g * kh * kw)
    y = torch.einsum('gok,ngkp->ngop', w, col).reshape(N, Cout, Ho, Wo)
    if bias is not None:
        y = y + torch.as_tensor(bias, dtype=torch.float64).view(1, -1, 1, 1)
    return y.numpy()


# ---- reference-held vectors -------------------------------------------------

@pytest.fixture(scope='module')
def kats():
    with open(os.path.join(GOLD, 'reference_kats.json')) as f:
        return json.load(f)


@pytest.mark.parametrize('dtype', [np.float32, np.float64])
def test_kat_dcnv2_zero_offset(kats, dtype):
    k = kats['dcnv2_zero_offset']
    x = np.array(k['input'], dtype=dtype)
    kh, kw = k['kernel']
    Ho, Wo = out_hw(3, 3, kh, kw, k['stride'], k['padding'], 1)
    w = np.full((1, 1, kh, kw), k['weight_fill'], dtype=dtype)
    off = np.zeros((1, 2 * kh * kw, Ho, Wo), dtype=dtype)
    m = np.full((1, kh * kw, Ho, Wo), k['mask_fill'], dtype=dtype)
    y = oracle.forward(x, off, m, w, None, k['stride'], k['padding'])
    assert np.allclose(y, np.array(k['output']), rtol=k['rtol'], atol=0)
    assert np.array_equal(y, np.array(k['output'], dtype=dtype))  # exact in binary fp


@pytest.mark.parametrize('dtype', [np.float32, np.float64])
def test_kat_dcnv1_fractional(kats, dtype):
    k = kats['dcnv1_fractional']
    x = torch.tensor(k['input'], dtype=torch.float64)
    ow = torch.tensor(k['offset_weight'], dtype=torch.float64).view(8, 1, 2, 2)
    ob = torch.tensor(k['offset_bias'], dtype=torch.float64)
    off = F.conv2d(x, ow, ob).numpy().astype(dtype)  # (1, 8, 2, 2)
    w = np.array(k['deform_weight'], dtype=dtype).reshape(1, 1, 2, 2)
    m = np.ones((1, 4, 2, 2), dtype=dtype)
    xin = np.array(k['input'], dtype=dtype)
    y = oracle.forward(xin, off, m, w, None, k['stride'], k['padding'])
    assert np.allclose(y, np.array(k['output']), rtol=0, atol=k['atol'])
    # the four sampled values at output (0, 0) are the reference's weight gradient
    col = oracle.im2col(xin[0], off[0], m[0], (2, 2), 1, 0, 1, 1)
    assert np.allclose(col[:, 0], np.array(k['samples_at_00']), rtol=0, atol=1e-6)


def test_golden_reference_outputs():
    """Outputs of the reference's compiled C++ (committed fixtures)."""
    with open(os.path.join(GOLD, 'ref_cases.json')) as f:
        meta = json.load(f)
    data = np.load(os.path.join(GOLD, 'ref_cases.npz'))
    assert set(meta) == set(data.files)
    for name, kw in meta.items():
        kw = dict(kw)
        seed, dt = kw.pop('seed'), kw.pop('dtype')
        case = make_case(seed, **kw)
        y = oracle.forward(*np_case(case, np.float64 if dt == 'float64' else np.float32))
        # only the GEMM summation order (BLAS vs plain loop) may differ
        tol = 1e-13 if dt == 'float64' else 5e-6
        assert rel_err(y, data[name]) <= tol, (name, rel_err(y, data[name]))


CASES = [
    dict(N=2, Cin=8, Cout=6, H=7, W=9),
    dict(N=1, Cin=8, Cout=8, H=9, W=8, stride=2, dilation=2, padding=2),
    dict(N=2, Cin=12, Cout=8, H=6, W=7, groups=2, deform_groups=3, sigma=4.0),
    dict(N=1, Cin=4, Cout=4, H=5, W=6, k=(2, 3), padding=(1, 0), stride=(1, 2), bias=False),
    dict(N=1, Cin=4, Cout=2, H=8, W=8, k=1, padding=0, deform_groups=4),
]


@pytest.mark.parametrize('idx', range(len(CASES)))
def test_against_live_reference(idx):
    if oracle.load_reference_ext() is None:
        pytest.skip('oracle/_ref not built (needs the reference tree)')
    case = make_case(300 + idx, **CASES[idx])
    for dt, npdt, tol in ((torch.float32, np.float32, 5e-6), (torch.float64, np.float64, 1e-13)):
        t = {k: (v.to(dt) if torch.is_tensor(v) else v) for k, v in case.items()}
        ref = oracle.reference_forward(t['input'], t['offset'], t['mask'], t['weight'],
                                       t['bias'], t['stride'], t['padding'],
                                       t['dilation'], t['groups'], t['deform_groups']).numpy()
        y = oracle.forward(*np_case(case, npdt))
        assert rel_err(y, ref) <= tol


# ---- what the mathematics fixes ---------------------------------------------

@pytest.mark.parametrize('kw', [
    dict(stride=1, padding=1, dilation=1, groups=1),
    dict(stride=2, padding=2, dilation=2, groups=2),
    dict(stride=(1, 2), padding=(0, 1), dilation=1, groups=4),
])
def test_zero_offset_is_conv2d(kw):
    case = make_case(11, N=2, Cin=8, Cout=12, H=9, W=10, sigma=0.0, **kw)
    args = list(np_case(case, np.float64))
    args[2] = np.ones_like(args[2])  # mask = 1
    y = oracle.forward(*args)
    ref = F.conv2d(case['input'].double(), case['weight'].double(), case['bias'].double(),
                   kw['stride'], kw['padding'], kw['dilation'], kw['groups']).numpy()
    assert rel_err(y, ref) <= 1e-14
    # constant mask m scales the bias-free part by m
    args[2] = np.full_like(args[2], 0.25)
    args[4] = None
    y2 = oracle.forward(*args)
    ref2 = 0.25 * F.conv2d(case['input'].double(), case['weight'].double(), None,
                           kw['stride'], kw['padding'], kw['dilation'], kw['groups']).numpy()
    assert rel_err(y2, ref2) <= 1e-14


@pytest.mark.parametrize('idx', range(len(CASES)))
def test_grid_sample_formulation(idx):
    case = make_case(500 + idx, **CASES[idx])
    args = np_case(case, np.float64)
    assert rel_err(oracle.forward(*args), grid_sample_forward(*args)) <= 1e-12


def test_brute_force_tiny():
    for seed, kw in ((1, dict(N=1, Cin=2, Cout=2, H=4, W=5, sigma=2.0)),
                     (2, dict(N=2, Cin=4, Cout=4, H=4, W=4, groups=2, deform_groups=2,
                              stride=2, sigma=3.0)),
                     (3, dict(N=1, Cin=2, Cout=3, H=5, W=4, k=2, padding=1, dilation=2,
                              bias=False))):
        case = make_case(seed, **kw)
        args = np_case(case, np.float64)
        assert rel_err(oracle.forward(*args), brute_force(*args)) <= 1e-13


def test_integer_offsets_are_shifted_taps():
    """Integer offsets pick single pixels: a brute-force shifted gather."""
    N, C, H, W = 1, 3, 6, 7
    g = torch.Generator().manual_seed(5)
    x = torch.randn(N, C, H, W, generator=g, dtype=torch.float64).numpy()
    off = torch.randint(-3, 4, (N, 18, H, W), generator=g).double().numpy()
    m = np.ones((N, 9, H, W))
    w = torch.randn(2, C, 3, 3, generator=g, dtype=torch.float64).numpy()
    y = oracle.forward(x, off, m, w, None, 1, 1)
    ref = np.zeros((N, 2, H, W))
    for ho in range(H):
        for wo in range(W):
            for i in range(3):
                for j in range(3):
                    t = i * 3 + j
                    yy = ho - 1 + i + int(off[0, 2 * t, ho, wo])
                    xx = wo - 1 + j + int(off[0, 2 * t + 1, ho, wo])
                    if 0 <= yy < H and 0 <= xx < W:
                        ref[0, :, ho, wo] += w[:, :, i, j] @ x[0, :, yy, xx]
    assert rel_err(y, ref) <= 1e-14


def test_sampler_boundaries():
    plane = np.arange(12, dtype=np.float64).reshape(3, 4) + 1.0
    H, W = plane.shape
    s = lambda h, w: oracle.sample(plane, h, w)
    assert s(0.0, 0.0) == plane[0, 0] and s(2.0, 3.0) == plane[2, 3]
    assert s(1.5, 2.25) == pytest.approx(
        0.5 * (0.75 * plane[1, 2] + 0.25 * plane[1, 3]) + 0.5 * (0.75 * plane[2, 2] + 0.25 * plane[2, 3]))
    # the open box: exactly -1 or H/W is outside; just inside blends with a zero border
    assert s(-1.0, 1.0) == 0.0 and s(1.0, -1.0) == 0.0
    assert s(float(H), 1.0) == 0.0 and s(1.0, float(W)) == 0.0
    assert s(-0.5, 0.0) == pytest.approx(0.5 * plane[0, 0])
    assert s(H - 0.5, W - 1.0) == pytest.approx(0.5 * plane[H - 1, W - 1])
    assert s(0.0, W - 0.75) == pytest.approx(0.75 * plane[0, W - 1])
    assert s(-0.25, -0.25) == pytest.approx(0.75 * 0.75 * plane[0, 0])
    assert s(float('nan'), 0.0) == 0.0
    # float32 twin agrees
    p32 = plane.astype(np.float32)
    assert oracle.sample(p32, 1.5, 2.25) == pytest.approx(s(1.5, 2.25), rel=1e-6)


def test_linearity_and_bias():
    case = make_case(21, N=1, Cin=8, Cout=4, H=6, W=6, deform_groups=2)
    x, off, m, w, b, *rest = np_case(case, np.float64)
    f = lambda x_, m_, w_, b_: oracle.forward(x_, off, m_, w_, b_, *rest)
    base = f(x, m, w, None)
    assert rel_err(f(2 * x, m, w, None), 2 * base) <= 1e-14
    assert rel_err(f(x, 0.5 * m, w, None), 0.5 * base) <= 1e-14
    assert rel_err(f(x, m, -3 * w, None), -3 * base) <= 1e-14
    assert rel_err(f(x, m, w, b), base + b.reshape(1, -1, 1, 1)) <= 1e-14


def test_all_taps_outside_gives_zero():
    case = make_case(22, N=1, Cin=4, Cout=4, H=5, W=5, bias=False)
    x, off, m, w, b, *rest = np_case(case, np.float32)
    off = np.full_like(off, 100.0)
    assert np.all(oracle.forward(x, off, m, w, None, *rest) == 0.0)


def test_channel_mismatch_raises():
    x = np.zeros((1, 4, 5, 5), np.float32)
    w = np.zeros((2, 3, 3, 3), np.float32)
    with pytest.raises(RuntimeError):
        oracle.forward(x, np.zeros((1, 18, 5, 5), np.float32),
                       np.zeros((1, 9, 5, 5), np.float32), w, None, 1, 1)
