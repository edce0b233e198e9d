"""Channels-last input read in place (no re-laid-out copy): the C ABI's input_nhwc
flag and torch.channels_last tensors through the extension, against the oracle
and against the bordered-copy path."""
import pytest
import torch

from common import TOL, capi, capi_forward, cast_case, make_case, oracle_forward, rel_err

pytestmark = pytest.mark.gpu

CASES = [
    ('c64', dict(N=2, Cin=64, Cout=64, H=13, W=17, sigma=2.0)),
    ('c128_far_offsets', dict(N=2, Cin=128, Cout=96, H=9, W=8, sigma=6.0)),        # many edge and outside taps
    ('c128_s2_dg2', dict(N=1, Cin=128, Cout=128, H=20, W=15, stride=2, deform_groups=2, sigma=3.0)),
    ('c64_g2_dil2', dict(N=1, Cin=128, Cout=64, H=16, W=18, padding=2, dilation=2, groups=2, sigma=2.0)),
    ('c64_2x2_image', dict(N=3, Cin=64, Cout=32, H=2, W=2, sigma=1.0)),
    ('c256_5x5', dict(N=1, Cin=256, Cout=48, H=12, W=12, k=5, padding=2, sigma=2.0)),
    # shapes with whole tiles of 256 pixels: the 256-pixel kernel reads the tensor in place as well
    ('wide_c256', dict(N=2, Cin=256, Cout=256, H=24, W=24, sigma=3.0)),
    ('wide_c128_far_offsets', dict(N=3, Cin=128, Cout=128, H=16, W=16, sigma=6.0)),
    ('wide_s2_g2', dict(N=2, Cin=256, Cout=512, H=33, W=32, stride=2, groups=2, sigma=2.0)),
]
DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def _np(t):
    return t.float().cpu().numpy()


@pytest.mark.parametrize('dtype', DTYPES, ids=['f32', 'bf16', 'f16'])
@pytest.mark.parametrize('name,kw', CASES, ids=[c[0] for c in CASES])
def test_in_place_channels_last_against_oracle(name, kw, dtype):
    case = cast_case(make_case(500 + len(name), **kw), dtype)
    ref = oracle_forward(case)
    dev = cast_case(case, dtype, 'cuda')
    y_copy = capi_forward(dev, path=capi.PATH_FUSED)
    y = capi_forward(dict(dev, input_nhwc=True), path=capi.PATH_FUSED)
    err = rel_err(_np(y), ref)
    both = rel_err(_np(y), _np(y_copy))
    print(f'  {name} {dtype}: vs oracle {err:.2e}, vs bordered-copy path {both:.2e}', flush=True)
    assert err <= TOL[dtype]
    assert both <= TOL[dtype] * 0.1
    if name.startswith('wide') and dtype != torch.float32:
        import ctypes
        N, Cin, H, W = case['input'].shape
        Cout, _, kh, kw = case['weight'].shape
        p = capi.make_params(capi.MDCN_BF16, N, Cin, H, W, Cout, kh, kw, case['stride'], case['padding'],
                             case['dilation'], case['groups'], case['deform_groups'], capi.PATH_FUSED_WIDE)
        p.input_nhwc = 1
        p.input = dev['input'].data_ptr()
        assert capi.load().mdcn_forward_kernels(ctypes.byref(p)).decode().startswith('fused3_kernel')
        y_wide = capi_forward(dict(dev, input_nhwc=True), path=capi.PATH_FUSED_WIDE, unsplit=True)
        y_narrow = capi_forward(dict(dev, input_nhwc=True), path=capi.PATH_FUSED_NARROW, unsplit=True)
        assert torch.equal(y_wide, y_narrow)   # the two kernels sum a tile's K range in the same order


def test_extension_takes_channels_last_tensors_in_place():
    from mmcv_amd.ops import modulated_deform_conv2d
    case = cast_case(make_case(77, N=2, Cin=64, Cout=64, H=14, W=11, sigma=2.0), torch.bfloat16, 'cuda')
    args = (case['offset'], case['mask'], case['weight'], case['bias'], 1, 1)
    y_nchw = modulated_deform_conv2d(case['input'], *args)
    x_cl = case['input'].contiguous(memory_format=torch.channels_last)
    assert not x_cl.is_contiguous()
    y_cl = modulated_deform_conv2d(x_cl, *args)
    assert y_cl.is_contiguous() and rel_err(_np(y_cl), _np(y_nchw)) <= TOL[torch.bfloat16] * 0.1
    # shapes the fused kernel does not cover fall back to a dense copy
    small = cast_case(make_case(78, N=1, Cin=8, Cout=8, H=6, W=6), torch.float32, 'cuda')
    ys = modulated_deform_conv2d(small['input'].contiguous(memory_format=torch.channels_last), small['offset'],
                                 small['mask'], small['weight'], small['bias'], 1, 1)
    assert rel_err(_np(ys), oracle_forward(cast_case(small, torch.float32, 'cpu'))) <= TOL[torch.float32]


def test_direct_path_and_other_entry_points_refuse_the_flag():
    import ctypes
    lib = capi.load()
    p = capi.make_params(capi.MDCN_F32, 1, 8, 6, 6, 8, 3, 3, (1, 1), (1, 1))
    p.input_nhwc = 1
    assert lib.mdcn_fused_eligible(ctypes.byref(p)) == 0
    assert lib.mdcn_workspace_bytes(ctypes.byref(p)) == 0
    dev = cast_case(make_case(79, N=1, Cin=8, Cout=8, H=6, W=6), torch.float32, 'cuda')
    with pytest.raises(AssertionError, match='not covered by the fused path'):
        capi_forward(dict(dev, input_nhwc=True))


@pytest.mark.parametrize('layer', ['dcnv2', 'dcnv1'])
def test_backward_through_channels_last_tensors(layer):
    """Training with channels_last input / offset / mask: gradients come out dense
    and equal those of the NCHW run."""
    from mmcv_amd.ops import deform_conv2d, modulated_deform_conv2d
    case = cast_case(make_case(91, N=2, Cin=64, Cout=64, H=12, W=10, sigma=1.5), torch.float32, 'cuda')
    gy = torch.randn(2, 64, 12, 10, device='cuda', generator=torch.Generator('cuda').manual_seed(1))

    def run(fmt):
        leaves = [case[k].clone().contiguous(memory_format=fmt).requires_grad_(True)
                  for k in ('input', 'offset', 'mask')]
        w = case['weight'].clone().requires_grad_(True)
        if layer == 'dcnv2':
            y = modulated_deform_conv2d(leaves[0], leaves[1], leaves[2], w, case['bias'], 1, 1)
        else:
            y = deform_conv2d(leaves[0], leaves[1], w, 1, 1)
        y.backward(gy)
        used = leaves if layer == 'dcnv2' else leaves[:2]
        return [t.grad for t in used] + [w.grad]

    ref = run(torch.contiguous_format)
    got = run(torch.channels_last)
    for a, b in zip(got, ref):
        assert a.shape == b.shape
        assert rel_err(_np(a), _np(b)) <= 1e-5
