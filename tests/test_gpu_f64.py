"""Double precision on the device: the reference dispatches its kernels over double
(mmcv/ops/csrc/pytorch/cuda/modulated_deform_conv_cuda.cu:16) and its own test
runs the layer in torch.double (tests/test_ops/test_modulated_deform_conv.py:148-160).
Forward and backward through the C ABI against the float64 oracle, the compiled
reference's committed float64 output, and the reference's known answers through
the Pack module."""
import json
import os

import numpy as np
import pytest
import torch

import oracle
from common import TOL, capi_backward, capi_forward, cast_case, make_case, oracle_forward, rel_err

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), 'golden')
F64 = torch.float64

CASES = [
    ('c8', dict(N=2, Cin=8, Cout=6, H=7, W=9, sigma=1.5)),
    ('c64', dict(N=2, Cin=64, Cout=64, H=12, W=13, sigma=2.0)),
    ('s2_g2_dg2', dict(N=1, Cin=16, Cout=12, H=11, W=10, stride=2, groups=2, deform_groups=2, sigma=2.5)),
    ('dil2_dg3', dict(N=2, Cin=12, Cout=8, H=9, W=9, padding=2, dilation=2, deform_groups=3, sigma=3.0)),
    ('k1x3_nobias', dict(N=1, Cin=6, Cout=10, H=6, W=17, k=(1, 3), padding=(0, 1), sigma=1.0, bias=False)),
    ('far_offsets', dict(N=1, Cin=8, Cout=8, H=5, W=5, padding=0, sigma=6.0)),
]


@pytest.mark.parametrize('name,kw', CASES, ids=[c[0] for c in CASES])
def test_forward_f64_against_oracle(name, kw):
    case = cast_case(make_case(300 + len(name), **kw), F64)
    ref = oracle_forward(case, np.float64)
    y = capi_forward(cast_case(case, F64, 'cuda'))
    assert y.dtype == F64
    err = rel_err(y.cpu().numpy(), ref)
    print(f'  {name}: {err:.2e}', flush=True)
    assert err <= TOL[F64]
    # DCNv1: no mask
    dev = cast_case(case, F64, 'cuda')
    dev['mask'], dev['bias'] = None, None
    ones = dict(case, mask=torch.ones_like(case['mask']), bias=None)
    assert rel_err(capi_forward(dev).cpu().numpy(), oracle_forward(ones, np.float64)) <= TOL[F64]


def test_forward_f64_golden_of_compiled_reference():
    with open(os.path.join(GOLD, 'ref_cases.json')) as f:
        kw = dict(json.load(f)['g_f64'])
    seed, dt = kw.pop('seed'), kw.pop('dtype')
    assert dt == 'float64'
    case = cast_case(make_case(seed, **kw), F64, 'cuda')
    y = capi_forward(case).cpu().numpy()
    assert rel_err(y, np.load(os.path.join(GOLD, 'ref_cases.npz'))['g_f64']) <= 1e-12


@pytest.mark.parametrize('modulated', [True, False], ids=['dcnv2', 'dcnv1'])
@pytest.mark.parametrize('name,kw', CASES, ids=[c[0] for c in CASES])
def test_backward_f64_against_oracle(name, kw, modulated):
    case = cast_case(make_case(500 + len(name), **kw), F64)
    if not modulated:
        case['mask'] = torch.ones_like(case['mask'])
    g = torch.Generator().manual_seed(11)
    Ho, Wo = case['offset'].shape[2:]
    gy = torch.randn(case['input'].shape[0], case['weight'].shape[0], Ho, Wo, generator=g, dtype=F64)
    geo = dict(stride=case['stride'], padding=case['padding'], dilation=case['dilation'],
               groups=case['groups'], deform_groups=case['deform_groups'])
    ref = oracle.backward(*[case[k].numpy() for k in ('input', 'offset', 'mask', 'weight')], gy.numpy(), True, **geo)
    dev = cast_case(case, F64, 'cuda')
    if not modulated:
        dev['mask'] = None
    got = capi_backward(dev, gy.cuda())
    for nm, r, o in zip(('grad_input', 'grad_offset', 'grad_mask', 'grad_weight', 'grad_bias'), ref, got):
        if o is None:
            assert nm == 'grad_mask' and not modulated
            continue
        assert o.dtype == F64
        err = rel_err(o.cpu().numpy(), r)
        print(f'  {name} {nm}: {err:.2e}', flush=True)
        assert err <= 1e-11, (nm, err)


def test_reference_known_answer_in_double():
    """mmcv tests/test_ops/test_modulated_deform_conv.py:49-76 with dtype=torch.double
    (test_mdconv_double)."""
    from mmcv_amd.ops import ModulatedDeformConv2dPack
    x = torch.tensor([[[[1., 2., 3.], [1., 2., 3.], [1., 2., 3.]]]], dtype=F64, device='cuda', requires_grad=True)
    dcn = ModulatedDeformConv2dPack(1, 1, kernel_size=(2, 2), stride=1, padding=1, deform_groups=1, bias=False).cuda()
    dcn.weight.data.fill_(1.)
    dcn.type(F64)
    out = dcn(x)
    assert out.dtype == F64
    out.sum().backward()
    n = lambda t: t.detach().cpu().numpy()
    assert np.allclose(n(out), [[[[0.5, 1.5, 2.5, 1.5], [1.0, 3.0, 5.0, 3.0], [1.0, 3.0, 5.0, 3.0],
                                  [0.5, 1.5, 2.5, 1.5]]]], 1e-2)
    assert np.allclose(n(x.grad), np.full((1, 1, 3, 3), 2.0), 1e-2)
    assert np.allclose(n(dcn.weight.grad), np.full((1, 1, 2, 2), 9.0), 1e-2)
    assert np.allclose(n(dcn.conv_offset.bias.grad),
                       [-3.0, -1.5, -3.0, -1.5, -3.0, -1.5, -3.0, -1.5, 4.5, 4.5, 4.5, 4.5], 1e-2)
    # without gradients the Pack takes the same tensor-op sequence (no fused pack-level call in double)
    with torch.no_grad():
        assert torch.equal(dcn(x.detach()), out.detach())


def test_f64_gradcheck_through_the_function():
    """torch.autograd.gradcheck of the op itself: analytic backward against central
    differences of the forward, both on the device, in double."""
    from mmcv_amd.ops import modulated_deform_conv2d
    case = cast_case(make_case(77, N=1, Cin=4, Cout=3, H=5, W=6, sigma=0.7), F64, 'cuda')
    # keep sampling positions away from the integer grid, where the op is not differentiable
    off = case['offset']
    frac = off - torch.floor(off)
    off = torch.floor(off) + frac.clamp(0.15, 0.85)
    leaves = [case['input'].requires_grad_(True), off.requires_grad_(True), case['mask'].requires_grad_(True),
              case['weight'].requires_grad_(True), case['bias'].requires_grad_(True)]
    fn = lambda x, o, m, w, b: modulated_deform_conv2d(x, o, m, w, b, 1, 1, 1, 1, 1)
    assert torch.autograd.gradcheck(fn, leaves, eps=1e-6, atol=1e-7, rtol=1e-6, nondet_tol=1e-12)


def test_f64_is_refused_where_it_has_no_kernel():
    import ctypes
    from mmcv_amd import capi
    lib = capi.load()
    p = capi.make_params(capi.MDCN_F64, 1, 64, 8, 8, 64, 3, 3, (1, 1), (1, 1), (1, 1), 1, 1)
    assert lib.mdcn_fused_eligible(ctypes.byref(p)) == 0
    assert lib.mdcn_workspace_bytes(ctypes.byref(p)) == 0
    case = cast_case(make_case(5, N=1, Cin=64, Cout=64, H=8, W=8), F64, 'cuda')
    with pytest.raises(AssertionError, match='not covered by the fused path'):
        capi_forward(case, path=capi.PATH_FUSED)
