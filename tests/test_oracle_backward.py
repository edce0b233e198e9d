"""Pins of the CPU oracle's backward: the reference's known-answer gradients, the
compiled reference itself, and central differences of the (already pinned)
forward oracle in float64."""
import numpy as np
import pytest
import torch

import oracle
from common import make_case


def _chain_through_pack(x, ow, ob, w, b, stride, padding, kh_kw, dtype=np.float64):
    """Gradients of sum(DCNv2Pack(x)) w.r.t. x, the DCN weight and conv_offset's
    parameters: torch autograd around the oracle's forward/backward."""
    class Op(torch.autograd.Function):
        @staticmethod
        def forward(ctx, inp, off, msk, wt):
            ctx.save_for_backward(inp, off, msk, wt)
            y = oracle.forward(inp.numpy(), off.numpy(), msk.numpy(), wt.numpy(), None, stride, padding)
            return torch.from_numpy(y)

        @staticmethod
        def backward(ctx, gy):
            inp, off, msk, wt = ctx.saved_tensors
            gi, go, gm, gw, _ = oracle.backward(inp.numpy(), off.numpy(), msk.numpy(), wt.numpy(),
                                                gy.contiguous().numpy(), False, stride, padding)
            return tuple(torch.from_numpy(a) for a in (gi, go, gm, gw))

    raw = torch.nn.functional.conv2d(x, ow, ob, stride, padding)
    o1, o2, m = torch.chunk(raw, 3, dim=1)
    y = Op.apply(x, torch.cat((o1, o2), 1), torch.sigmoid(m), w)
    return y


def test_reference_known_answer_gradients_dcnv2():
    """mmcv tests/test_ops/test_modulated_deform_conv.py:28-46: zero-initialised
    conv_offset, weight 1, loss = output.sum()."""
    t = torch.float64
    x = torch.tensor([[[[1., 2., 3.], [1., 2., 3.], [1., 2., 3.]]]], dtype=t, requires_grad=True)
    ow = torch.zeros(12, 1, 2, 2, dtype=t, requires_grad=True)
    ob = torch.zeros(12, dtype=t, requires_grad=True)
    w = torch.ones(1, 1, 2, 2, dtype=t, requires_grad=True)
    y = _chain_through_pack(x, ow, ob, w, None, 1, 1, (2, 2))
    y.sum().backward()
    assert np.allclose(y.detach().numpy(), [[[[0.5, 1.5, 2.5, 1.5], [1.0, 3.0, 5.0, 3.0], [1.0, 3.0, 5.0, 3.0],
                                               [0.5, 1.5, 2.5, 1.5]]]], 1e-2)
    assert np.allclose(x.grad.numpy(), np.full((1, 1, 3, 3), 2.0), 1e-2)
    assert np.allclose(w.grad.numpy(), np.full((1, 1, 2, 2), 9.0), 1e-2)
    kat_ow = [[[[-7.0, -4.0], [0.0, 0.0]]], [[[-9.0, 7.5], [-6.0, 5.0]]], [[[-4.0, -7.0], [0.0, 0.0]]],
              [[[-7.5, -9.0], [-5.0, -6.0]]], [[[-7.0, -4.0], [-7.0, -4.0]]], [[[-6.0, 5.0], [-9.0, 7.5]]],
              [[[-4.0, -7.0], [-4.0, -7.0]]], [[[-5.0, -6.0], [-7.5, -9.0]]], [[[10.5, 6.0], [7.0, 4.0]]],
              [[[6.0, 10.5], [4.0, 7.0]]], [[[7.0, 4.0], [10.5, 6.0]]], [[[4.0, 7.0], [6.0, 10.5]]]]
    kat_ob = [-3.0, -1.5, -3.0, -1.5, -3.0, -1.5, -3.0, -1.5, 4.5, 4.5, 4.5, 4.5]
    assert np.allclose(ow.grad.numpy(), kat_ow, 1e-2)
    assert np.allclose(ob.grad.numpy(), kat_ob, 1e-2)


def test_reference_known_answer_gradients_dcnv1():
    """mmcv tests/test_ops/test_deform_conv.py:27-47 (fractional offsets, mask 1):
    the DCNv1 layer's gradients equal the modulated ones with a mask of ones."""
    t = torch.float64
    x = torch.tensor([[[[1., 2., 3.], [0., 1., 2.], [3., 5., 2.]]]], dtype=t, requires_grad=True)
    ow = torch.tensor([[[0.1, 0.4, 0.6, 0.1]], [[0.3, 0.2, 0.1, 0.3]], [[0.5, 0.5, 0.2, 0.8]], [[0.8, 0.3, 0.9, 0.1]],
                       [[0.3, 0.1, 0.2, 0.5]], [[0.3, 0.7, 0.5, 0.3]], [[0.6, 0.2, 0.5, 0.3]], [[0.4, 0.1, 0.8, 0.4]]],
                      dtype=t).reshape(8, 1, 2, 2).requires_grad_(True)
    ob = torch.tensor([0.7, 0.1, 0.8, 0.5, 0.6, 0.5, 0.4, 0.7], dtype=t, requires_grad=True)
    w = torch.tensor([[[0.4, 0.2, 0.1, 0.9]]], dtype=t).reshape(1, 1, 2, 2).requires_grad_(True)

    class Op(torch.autograd.Function):
        @staticmethod
        def forward(ctx, inp, off, wt):
            ctx.save_for_backward(inp, off, wt)
            ones = np.ones((1, 4, 2, 2))
            return torch.from_numpy(oracle.forward(inp.numpy(), off.numpy(), ones, wt.numpy(), None, 1, 0))

        @staticmethod
        def backward(ctx, gy):
            inp, off, wt = ctx.saved_tensors
            gi, go, _, gw, _ = oracle.backward(inp.numpy(), off.numpy(), np.ones((1, 4, 2, 2)), wt.numpy(),
                                               gy.contiguous().numpy(), False, 1, 0)
            return torch.from_numpy(gi), torch.from_numpy(go), torch.from_numpy(gw)

    y = Op.apply(x, torch.nn.functional.conv2d(x, ow, ob), w)
    y.backward(torch.ones_like(y))
    thr = 1e-3
    assert np.allclose(y.detach().numpy(), [[[[1.650, 0.], [0.000, 0.]]]], thr, thr)
    assert np.allclose(x.grad.numpy(), [[[[-0.666, 0.204, 0.000], [0.030, -0.416, 0.012], [0.000, 0.252, 0.129]]]],
                       thr, thr)
    kat_ow = [[[[1.44, 2.88], [0.00, 1.44]]], [[[-0.72, -1.44], [0.00, -0.72]]], [[[0.00, 0.00], [0.00, 0.00]]],
              [[[0.00, 0.00], [0.00, 0.00]]], [[[-0.10, -0.20], [0.00, -0.10]]], [[[-0.08, -0.16], [0.00, -0.08]]],
              [[[-0.54, -1.08], [0.00, -0.54]]], [[[-0.54, -1.08], [0.00, -0.54]]]]
    assert np.allclose(ow.grad.numpy(), kat_ow, thr, thr)
    assert np.allclose(ob.grad.numpy(), [1.44, -0.72, 0., 0., -0.10, -0.08, -0.54, -0.54], thr, thr)
    assert np.allclose(w.grad.numpy(), [[[[3.62, 0.], [0.40, 0.18]]]], thr, thr)


CASES = [
    dict(N=2, Cin=4, Cout=6, H=7, W=9, sigma=1.5),
    dict(N=1, Cin=8, Cout=4, H=9, W=8, stride=2, groups=2, deform_groups=2, sigma=2.5),
    dict(N=2, Cin=6, Cout=6, H=8, W=8, padding=2, dilation=2, deform_groups=3, sigma=3.0),
    dict(N=1, Cin=3, Cout=5, H=6, W=7, k=(1, 3), padding=(0, 1), sigma=1.0),
    dict(N=1, Cin=4, Cout=4, H=5, W=5, padding=0, sigma=6.0),   # many taps outside
]


@pytest.mark.parametrize('dtype', [np.float32, np.float64], ids=['f32', 'f64'])
@pytest.mark.parametrize('kw', CASES, ids=lambda c: 'x'.join(f'{k}{v}' for k, v in c.items() if k != 'sigma'))
def test_against_the_compiled_reference(kw, dtype):
    if oracle.load_reference_ext() is None or not hasattr(oracle.load_reference_ext(), 'modulated_deform_conv_backward'):
        pytest.skip('oracle/_ref not built')
    case = make_case(11, **kw)
    td = torch.float32 if dtype == np.float32 else torch.float64
    g = torch.Generator().manual_seed(5)
    Ho, Wo = case['offset'].shape[2:]
    gy = torch.randn(case['input'].shape[0], case['weight'].shape[0], Ho, Wo, generator=g)
    args = [case[k].to(td) for k in ('input', 'offset', 'mask', 'weight')] + [gy.to(td)]
    geo = dict(stride=case['stride'], padding=case['padding'], dilation=case['dilation'], groups=case['groups'],
               deform_groups=case['deform_groups'])
    ref = oracle.reference_backward(*args, with_bias=True, **geo)
    got = oracle.backward(*[a.numpy() for a in args], with_bias=True, **geo)
    tol = 2e-5 if dtype == np.float32 else 1e-12
    for name, r, o in zip(('grad_input', 'grad_offset', 'grad_mask', 'grad_weight', 'grad_bias'), ref, got):
        r = r.numpy()
        scale = max(np.abs(r).max(), 1e-30)
        assert np.abs(o - r).max() / scale <= tol, (name, np.abs(o - r).max() / scale)


def test_against_central_differences_of_the_forward():
    """float64, loss = sum(forward * G): the analytic gradients equal central
    differences of the forward oracle for input, weight, mask (exactly linear) and,
    away from integer sampling positions, for the offsets."""
    case = make_case(23, N=1, Cin=4, Cout=3, H=6, W=7, deform_groups=2, sigma=1.3)
    a = {k: case[k].double().numpy() for k in ('input', 'offset', 'mask', 'weight')}
    b = case['bias'].double().numpy()
    geo = dict(stride=(1, 1), padding=(1, 1), dilation=(1, 1), groups=1, deform_groups=2)
    rng = np.random.default_rng(3)
    G = rng.standard_normal((1, 3, 6, 7))
    # keep sampling positions away from the integer grid, where the sampler has kinks
    frac = a['offset'] - np.floor(a['offset'])
    a['offset'] = np.floor(a['offset']) + 0.2 + 0.6 * frac
    loss = lambda **over: float((oracle.forward(**{**a, **over}, bias=b, **geo) * G).sum())
    gi, go, gm, gw, gb = oracle.backward(a['input'], a['offset'], a['mask'], a['weight'], G, True, **geo)
    for name, grad, eps in (('input', gi, 1e-3), ('weight', gw, 1e-3), ('mask', gm, 1e-3), ('offset', go, 1e-6)):
        flat = a[name].reshape(-1)
        for idx in rng.choice(flat.size, size=40, replace=False):
            up, dn = a[name].copy().reshape(-1), a[name].copy().reshape(-1)
            up[idx] += eps
            dn[idx] -= eps
            num = (loss(**{name: up.reshape(a[name].shape)}) - loss(**{name: dn.reshape(a[name].shape)})) / (2 * eps)
            assert abs(num - grad.reshape(-1)[idx]) <= 1e-6 * max(1.0, abs(num)), (name, idx, num, grad.reshape(-1)[idx])
    assert np.allclose(gb, G.sum(axis=(0, 2, 3)), rtol=1e-12, atol=1e-12)
