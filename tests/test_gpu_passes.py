"""Large batches run in passes of whole images (forward: 32-bit offsets into the
input copy; backward: bounded column-gradient scratch).  With the limits lowered
through mdcn_set_pass_limits the pass loops run at test size; results must equal
the single-pass ones."""
import pytest
import torch

from mmcv_amd import capi
from common import (capi_backward, capi_forward, capi_pack_forward, cast_case, cast_pack_case, make_case,
                    make_pack_case, rel_err)

pytestmark = pytest.mark.gpu


@pytest.fixture
def limits():
    lib = capi.load()
    yield lambda fwd, bwd: lib.mdcn_set_pass_limits(fwd, bwd)
    lib.mdcn_set_pass_limits(0, 0)


def _np(t):
    return t.float().cpu().numpy()


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16], ids=['f32', 'bf16'])
@pytest.mark.parametrize('nhwc', [False, True], ids=['nchw', 'nhwc'])
def test_forward_passes(limits, dtype, nhwc):
    kw = dict(N=5, Cin=128, Cout=96, H=11, W=13, deform_groups=2, sigma=2.0)
    dev = cast_case(make_case(31, **kw), dtype, 'cuda')
    dev = dict(dev, input_nhwc=nhwc)
    one = capi_forward(dev, path=capi.PATH_FUSED)
    img = 13 * 15 * 128 * dev['input'].element_size()   # one zero-bordered image of the copy
    for images in (1, 2):
        limits(images * img, 0)
        got = capi_forward(dev, path=capi.PATH_FUSED)
        assert torch.equal(got, one), images


@pytest.mark.parametrize('unmodulated', [False, True], ids=['dcnv2', 'dcnv1'])
def test_pack_forward_passes(limits, unmodulated):
    dtype = torch.bfloat16
    dev = cast_pack_case(make_pack_case(5, N=4, Cin=64, Cout=64, H=12, W=9, unmodulated=unmodulated), dtype, 'cuda')
    one, raw_one = capi_pack_forward(dev, want_raw=True, unmodulated=unmodulated)
    limits(2 * 14 * 11 * 64 * 2, 0)
    got, raw = capi_pack_forward(dev, want_raw=True, unmodulated=unmodulated)
    assert torch.equal(raw, raw_one) and torch.equal(got, one)


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16], ids=['f32', 'bf16'])
def test_backward_passes(limits, dtype):
    kw = dict(N=5, Cin=64, Cout=64, H=12, W=22, groups=2, sigma=2.0)
    dev = cast_case(make_case(32, **kw), dtype, 'cuda')
    gy = torch.randn(5, 64, 12, 22, generator=torch.Generator().manual_seed(5)).to(dtype).cuda()
    one = capi_backward(dev, gy, path=capi.PATH_FUSED)
    d_img = 9 * 64 * 12 * 22 * dev['input'].element_size()   # column gradient of one image
    tol = 1e-5 if dtype == torch.float32 else 4e-3           # (atomics: summation order varies)
    for images in (1, 2):
        limits(0, images * d_img)
        got = capi_backward(dev, gy, path=capi.PATH_FUSED)
        for a, b in zip(got, one):
            assert rel_err(_np(a), _np(b)) <= tol, images
