"""Backward on the device against the CPU oracle's backward (itself pinned against
the reference's gradient known answers, the compiled reference and central
differences) and the reference's known-answer tests through the modules."""
import numpy as np
import pytest
import torch

import oracle
from mmcv_amd import capi
from common import TOL, capi_backward, cast_case, make_case, rel_err

pytestmark = pytest.mark.gpu

CASES = [
    ('c8', dict(N=2, Cin=8, Cout=6, H=7, W=9, sigma=1.5)),
    ('c64_fused_shape', dict(N=2, Cin=64, Cout=64, H=12, W=13, sigma=2.0)),
    ('s2_g2_dg2', dict(N=1, Cin=16, Cout=12, H=11, W=10, stride=2, groups=2, deform_groups=2, sigma=2.5)),
    ('dil2_dg3', dict(N=2, Cin=12, Cout=8, H=9, W=9, padding=2, dilation=2, deform_groups=3, sigma=3.0)),
    ('k1x3', dict(N=1, Cin=6, Cout=10, H=6, W=17, k=(1, 3), padding=(0, 1), sigma=1.0)),
    ('cout300_g1', dict(N=1, Cin=20, Cout=300, H=6, W=7, sigma=1.0)),
    ('far_offsets', dict(N=1, Cin=8, Cout=8, H=5, W=5, padding=0, sigma=6.0)),
    ('odd_plane', dict(N=3, Cin=10, Cout=7, H=7, W=11, sigma=2.0)),
]
DTYPES = [torch.float32, torch.bfloat16, torch.float16]
NAMES = ('grad_input', 'grad_offset', 'grad_mask', 'grad_weight', 'grad_bias')


def _np(t):
    return t.float().cpu().numpy()


@pytest.mark.parametrize('modulated', [True, False], ids=['dcnv2', 'dcnv1'])
@pytest.mark.parametrize('dtype', DTYPES, ids=['f32', 'bf16', 'f16'])
@pytest.mark.parametrize('name,kw', CASES, ids=[c[0] for c in CASES])
def test_backward_against_oracle(name, kw, dtype, modulated):
    case = cast_case(make_case(700 + len(name), **kw), dtype)
    if not modulated:
        case['mask'] = torch.ones_like(case['mask'])
    g = torch.Generator().manual_seed(9)
    Ho, Wo = case['offset'].shape[2:]
    gy = torch.randn(case['input'].shape[0], case['weight'].shape[0], Ho, Wo, generator=g).to(dtype)
    geo = dict(stride=case['stride'], padding=case['padding'], dilation=case['dilation'],
               groups=case['groups'], deform_groups=case['deform_groups'])
    ref = oracle.backward(*[case[k].float().numpy() for k in ('input', 'offset', 'mask', 'weight')],
                          gy.float().numpy(), True, **geo)
    dev = cast_case(case, dtype, 'cuda')
    if not modulated:
        dev['mask'] = None
    got = capi_backward(dev, gy.cuda())
    for nm, r, o in zip(NAMES, ref, got):
        if o is None:
            assert nm == 'grad_mask' and not modulated
            continue
        err = rel_err(_np(o), r)
        print(f'  {name} {dtype} {nm}: {err:.2e}', flush=True)
        assert err <= TOL[dtype], (nm, err)


def test_reference_known_answer_dcnv2_module():
    """mmcv tests/test_ops/test_modulated_deform_conv.py:28-80."""
    from mmcv_amd.ops import ModulatedDeformConv2dPack
    for dtype, tol in ((torch.float32, 1e-2), (torch.float16, 1e-2)):
        x = torch.tensor([[[[1., 2., 3.], [1., 2., 3.], [1., 2., 3.]]]], dtype=dtype, device='cuda', requires_grad=True)
        dcn = ModulatedDeformConv2dPack(1, 1, kernel_size=(2, 2), stride=1, padding=1, deform_groups=1, bias=False).cuda()
        dcn.weight.data.fill_(1.)
        dcn.type(dtype)
        out = dcn(x)
        out.sum().backward()
        assert np.allclose(_np(out.detach()), [[[[0.5, 1.5, 2.5, 1.5], [1.0, 3.0, 5.0, 3.0], [1.0, 3.0, 5.0, 3.0],
                                                  [0.5, 1.5, 2.5, 1.5]]]], tol)
        assert np.allclose(_np(x.grad), np.full((1, 1, 3, 3), 2.0), tol)
        assert np.allclose(_np(dcn.weight.grad), np.full((1, 1, 2, 2), 9.0), tol)
        kat_ow = [[[[-7.0, -4.0], [0.0, 0.0]]], [[[-9.0, 7.5], [-6.0, 5.0]]], [[[-4.0, -7.0], [0.0, 0.0]]],
                  [[[-7.5, -9.0], [-5.0, -6.0]]], [[[-7.0, -4.0], [-7.0, -4.0]]], [[[-6.0, 5.0], [-9.0, 7.5]]],
                  [[[-4.0, -7.0], [-4.0, -7.0]]], [[[-5.0, -6.0], [-7.5, -9.0]]], [[[10.5, 6.0], [7.0, 4.0]]],
                  [[[6.0, 10.5], [4.0, 7.0]]], [[[7.0, 4.0], [10.5, 6.0]]], [[[4.0, 7.0], [6.0, 10.5]]]]
        assert np.allclose(_np(dcn.conv_offset.weight.grad), kat_ow, tol)
        assert np.allclose(_np(dcn.conv_offset.bias.grad),
                           [-3.0, -1.5, -3.0, -1.5, -3.0, -1.5, -3.0, -1.5, 4.5, 4.5, 4.5, 4.5], tol)


def test_reference_known_answer_dcnv1_module():
    """mmcv tests/test_ops/test_deform_conv.py:27-113 (batch of 10, im2col_step 2)."""
    from mmcv_amd.ops import DeformConv2dPack
    from test_gpu_dcnv1 import KAT_INPUT, KAT_OFFSET_BIAS, KAT_OFFSET_WEIGHT, KAT_OUT, KAT_WEIGHT
    batch = 10
    for dtype, thr in ((torch.float32, 1e-3), (torch.float16, 1e-2)):
        x = torch.tensor(np.repeat(KAT_INPUT, batch, axis=0), device='cuda', dtype=dtype, requires_grad=True)
        model = DeformConv2dPack(in_channels=1, out_channels=1, kernel_size=2, stride=1, padding=0, im2col_step=2)
        model.conv_offset.weight.data = torch.Tensor(KAT_OFFSET_WEIGHT).reshape(8, 1, 2, 2)
        model.conv_offset.bias.data = torch.Tensor(KAT_OFFSET_BIAS).reshape(8)
        model.weight.data = torch.Tensor(KAT_WEIGHT).reshape(1, 1, 2, 2)
        model.cuda().type(dtype)
        out = model(x)
        out.backward(torch.ones_like(out))
        assert np.allclose(_np(out.detach()), np.repeat(KAT_OUT, batch, axis=0), thr, thr)
        gt_x = [[[[-0.666, 0.204, 0.000], [0.030, -0.416, 0.012], [0.000, 0.252, 0.129]]]]
        assert np.allclose(_np(x.grad), np.repeat(gt_x, batch, axis=0), thr, thr)
        gt_ow = [[[[1.44, 2.88], [0.00, 1.44]]], [[[-0.72, -1.44], [0.00, -0.72]]], [[[0.00, 0.00], [0.00, 0.00]]],
                 [[[0.00, 0.00], [0.00, 0.00]]], [[[-0.10, -0.20], [0.00, -0.10]]], [[[-0.08, -0.16], [0.00, -0.08]]],
                 [[[-0.54, -1.08], [0.00, -0.54]]], [[[-0.54, -1.08], [0.00, -0.54]]]]
        # fp16 sums ten images' gradients in half precision inside torch's conv backward
        wthr = thr if dtype == torch.float32 else 3e-2
        assert np.allclose(_np(model.conv_offset.weight.grad) / batch, gt_ow, wthr, wthr)
        assert np.allclose(_np(model.conv_offset.bias.grad) / batch, [1.44, -0.72, 0., 0., -0.10, -0.08, -0.54, -0.54],
                           wthr, wthr)
        assert np.allclose(_np(model.weight.grad) / batch, [[[[3.62, 0.], [0.40, 0.18]]]], wthr, wthr)


# shapes the matrix-core column-gradient path covers (channels in whole 128-byte
# slabs, 32-channel blocks per tap), forced onto the tiled kernels at test size
TILED_CASES = [
    ('c64', dict(N=2, Cin=64, Cout=64, H=20, W=19, sigma=2.0)),
    ('c128_g2_dg2', dict(N=1, Cin=128, Cout=128, H=18, W=21, groups=2, deform_groups=2, sigma=2.5)),
    ('c64_co192', dict(N=2, Cin=64, Cout=192, H=23, W=17, sigma=1.5)),
    ('c64_co128_s2', dict(N=2, Cin=64, Cout=128, H=23, W=37, stride=2, sigma=1.5)),
    ('c128_s2_dil2_dg2', dict(N=1, Cin=128, Cout=64, H=30, W=21, stride=2, padding=2, dilation=2, deform_groups=2, sigma=2.5)),
    ('c64_dil2_dg4', dict(N=1, Cin=64, Cout=64, H=17, W=17, padding=2, dilation=2, deform_groups=4, sigma=3.0)),
    ('c192_k1x3', dict(N=1, Cin=192, Cout=64, H=9, W=33, k=(1, 3), padding=(0, 1), sigma=1.0)),
    ('c96_f32_only', dict(N=1, Cin=96, Cout=32, H=16, W=16, sigma=6.0)),
    ('c40_window_only', dict(N=2, Cin=40, Cout=24, H=18, W=17, deform_groups=2, sigma=2.0)),
]


@pytest.mark.parametrize('modulated', [True, False], ids=['dcnv2', 'dcnv1'])
@pytest.mark.parametrize('dtype', DTYPES, ids=['f32', 'bf16', 'f16'])
@pytest.mark.parametrize('name,kw', TILED_CASES, ids=[c[0] for c in TILED_CASES])
def test_tiled_backward_against_oracle(name, kw, dtype, modulated):
    case = cast_case(make_case(900 + len(name), **kw), dtype)
    if not modulated:
        case['mask'] = torch.ones_like(case['mask'])
    g = torch.Generator().manual_seed(11)
    Ho, Wo = case['offset'].shape[2:]
    gy = torch.randn(case['input'].shape[0], case['weight'].shape[0], Ho, Wo, generator=g).to(dtype)
    geo = dict(stride=case['stride'], padding=case['padding'], dilation=case['dilation'],
               groups=case['groups'], deform_groups=case['deform_groups'])
    ref = oracle.backward(*[case[k].float().numpy() for k in ('input', 'offset', 'mask', 'weight')],
                          gy.float().numpy(), True, **geo)
    dev = cast_case(case, dtype, 'cuda')
    if not modulated:
        dev['mask'] = None
    got = capi_backward(dev, gy.cuda(), path=capi.PATH_FUSED)
    direct = capi_backward(dev, gy.cuda(), path=capi.PATH_DIRECT)
    for nm, r, o, d in zip(NAMES, ref, got, direct):
        if o is None:
            assert nm == 'grad_mask' and not modulated
            continue
        err, err_d = rel_err(_np(o), r), rel_err(_np(d), r)
        print(f'  {name} {dtype} {nm}: tiled {err:.2e} per-tap {err_d:.2e}', flush=True)
        assert err <= TOL[dtype] and err_d <= TOL[dtype], (nm, err, err_d)


@pytest.mark.parametrize('dtype', DTYPES, ids=['f32', 'bf16', 'f16'])
def test_tiled_backward_partial_requests(dtype):
    """Only the data gradients, or only grad_weight (the two calls of the unmodulated
    layer's backward): the same values as the full call, the rest untouched."""
    case = cast_case(make_case(77, N=2, Cin=64, Cout=128, H=14, W=24, deform_groups=2, sigma=2.0), dtype, 'cuda')
    gy = torch.randn(2, 128, 14, 24, generator=torch.Generator().manual_seed(3)).to(dtype).cuda()
    full = capi_backward(case, gy, path=capi.PATH_FUSED)
    data = capi_backward(case, gy, path=capi.PATH_FUSED, want_weight=False, want_bias=False)
    wonly = capi_backward(case, gy, path=capi.PATH_FUSED, want_data=False)
    tol = 1e-5 if dtype == torch.float32 else 4e-3  # (atomics: the order of the sums varies; one 16-bit ulp)
    for i in range(3):
        assert rel_err(_np(data[i]), _np(full[i])) <= tol
        assert torch.all(wonly[i] == 7.0)
    assert torch.all(data[3] == 7.0)
    assert rel_err(_np(wonly[3]), _np(full[3])) <= tol
    assert rel_err(_np(wonly[4]), _np(full[4])) <= tol


def test_full_size_layer_gradients_spot_check():
    """cfg-4-like layer at reduced batch (bf16, 256 channels, 100x152): first image
    of the batch against the oracle."""
    dtype = torch.bfloat16
    case = cast_case(make_case(4242, N=2, Cin=256, Cout=256, H=100, W=152, sigma=2.0), dtype)
    g = torch.Generator().manual_seed(1)
    gy = torch.randn(2, 256, 100, 152, generator=g).to(dtype)
    got = capi_backward(cast_case(case, dtype, 'cuda'), gy.cuda(), path=capi.PATH_FUSED)
    sub = {k: (case[k][:1] if k in ('input', 'offset', 'mask') else case[k]) for k in case}
    ref = oracle.backward(*[sub[k].float().numpy() for k in ('input', 'offset', 'mask', 'weight')],
                          gy[:1].float().numpy(), True, stride=(1, 1), padding=(1, 1), dilation=(1, 1), groups=1,
                          deform_groups=1)
    for nm, r, o in zip(NAMES[:3], ref[:3], got[:3]):
        err = rel_err(_np(o[:1]), r)
        print(f'  {nm}: {err:.2e}', flush=True)
        assert err <= TOL[dtype], (nm, err)


def test_full_size_grad_weight_and_bias_at_cfg4_shape():
    """grad_weight / grad_bias at the full cfg-4 shape (N = 16, 243 200 pixels: the 256-tile split-K
    product and its fixed-order reduction).  With zero offsets and unit mask the layer is a plain
    convolution, whose weight gradient torch computes in fp32; grad_bias is the sum of grad_output."""
    dtype = torch.bfloat16
    case = make_case(99, N=16, Cin=256, Cout=256, H=100, W=152, sigma=0.0)
    case['mask'] = torch.ones_like(case['mask'])
    dev = cast_case(case, dtype, 'cuda')
    gy = torch.randn(16, 256, 100, 152, generator=torch.Generator().manual_seed(2)).to(dtype).cuda()
    got = capi_backward(dev, gy, path=capi.PATH_FUSED)
    gw_ref = torch.nn.grad.conv2d_weight(dev['input'].float(), dev['weight'].shape, gy.float(), stride=1, padding=1)
    gb_ref = gy.double().sum(dim=(0, 2, 3))
    gi_ref = torch.nn.grad.conv2d_input(dev['input'].shape, dev['weight'].float(), gy.float(), stride=1, padding=1)
    for nm, o, r in (('grad_weight', got[3], gw_ref), ('grad_bias', got[4], gb_ref), ('grad_input', got[0], gi_ref)):
        err = rel_err(_np(o), r.float().cpu().numpy())
        print(f'  {nm}: {err:.2e}', flush=True)
        assert err <= TOL[dtype], (nm, err)


def test_full_size_grad_weight_adds_up_over_batch_halves():
    """Random offsets at the cfg-4 shape: the weight and bias gradients of the whole batch are the sums of
    those of its two halves (each a call of its own, with its own K-range shares)."""
    dtype = torch.bfloat16
    case = cast_case(make_case(4243, N=16, Cin=256, Cout=256, H=100, W=152, sigma=2.0), dtype, 'cuda')
    gy = torch.randn(16, 256, 100, 152, generator=torch.Generator().manual_seed(5)).to(dtype).cuda()
    full = capi_backward(case, gy, path=capi.PATH_FUSED, want_data=False)

    def half(sl):
        sub = dict(case)
        for k in ('input', 'offset', 'mask'):
            sub[k] = case[k][sl].contiguous()
        return capi_backward(sub, gy[sl].contiguous(), path=capi.PATH_FUSED, want_data=False)

    a, b = half(slice(0, 8)), half(slice(8, 16))
    for i, nm in ((3, 'grad_weight'), (4, 'grad_bias')):
        err = rel_err(_np(full[i]), _np(a[i]) + _np(b[i]))
        print(f'  {nm}: {err:.2e}', flush=True)
        assert err <= 8e-3, (nm, err)  # (three roundings to bf16 instead of one)


def test_full_size_all_five_gradients_against_oracle():
    """cfg-4-shaped layer, N = 2: every gradient of the whole call against the oracle."""
    dtype = torch.bfloat16
    case = cast_case(make_case(4244, N=2, Cin=256, Cout=256, H=100, W=152, sigma=2.0), dtype)
    gy = torch.randn(2, 256, 100, 152, generator=torch.Generator().manual_seed(7)).to(dtype)
    got = capi_backward(cast_case(case, dtype, 'cuda'), gy.cuda(), path=capi.PATH_FUSED)
    ref = oracle.backward(*[case[k].float().numpy() for k in ('input', 'offset', 'mask', 'weight')],
                          gy.float().numpy(), True, stride=(1, 1), padding=(1, 1), dilation=(1, 1), groups=1,
                          deform_groups=1)
    for nm, r, o in zip(NAMES, ref, got):
        err = rel_err(_np(o), r)
        print(f'  {nm}: {err:.2e}', flush=True)
        assert err <= TOL[dtype], (nm, err)


def test_fixed_point_window_with_wide_dynamic_range():
    """16-bit tensors sum grad_input in a 32-bit fixed-point window scaled by the largest column
    gradient of the call.  With grad_output spanning six decades, the gradient as a whole stays
    within tolerance of the oracle (error against the largest element), and the region whose
    contributions are a million times smaller than the largest carries an absolute error of at most
    a few window quanta, i.e. far below the 16-bit rounding of the large elements -- but not a
    small relative error of its own, which is what the window gives up."""
    dtype = torch.bfloat16
    case = cast_case(make_case(606, N=1, Cin=64, Cout=64, H=40, W=48, sigma=1.0), dtype)
    g = torch.Generator().manual_seed(8)
    gy = torch.randn(1, 64, 40, 48, generator=g) * 1e-5
    gy[:, :, 2:6, 2:6] = torch.randn(1, 64, 4, 4, generator=g) * 10.0
    gy = gy.to(dtype)
    got = capi_backward(cast_case(case, dtype, 'cuda'), gy.cuda(), path=capi.PATH_FUSED)
    ref = oracle.backward(*[case[k].float().numpy() for k in ('input', 'offset', 'mask', 'weight')],
                          gy.float().numpy(), True, stride=(1, 1), padding=(1, 1), dilation=(1, 1), groups=1,
                          deform_groups=1)
    gi, gi_ref = _np(got[0]), ref[0]
    big = float(np.abs(gi_ref).max())
    assert rel_err(gi, gi_ref) <= TOL[dtype]
    far = np.abs(gi - gi_ref)[:, :, 20:, 24:]   # sampled only by pixels with tiny grad_output
    assert float(np.abs(gi_ref[:, :, 20:, 24:]).max()) < 1e-4 * big
    print(f'  far region: max abs err {far.max():.3e}, largest element of the gradient {big:.3e}', flush=True)
    assert float(far.max()) <= 2e-5 * big
    for nm, r, o in zip(NAMES[1:], ref[1:], got[1:]):
        assert rel_err(_np(o), r) <= TOL[dtype], nm
