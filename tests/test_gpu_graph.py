"""The forward enqueues kernels only (no allocation of its own, no synchronisation,
no memset nodes), so a caller may capture it into a HIP graph.  Replays with new
contents in the captured tensors must match eager calls."""
import pytest
import torch

from common import TOL, cast_case, make_case, rel_err

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16], ids=['f32', 'bf16'])
def test_forward_in_a_captured_graph(dtype):
    from mmcv_amd.ops import modulated_deform_conv2d
    kw = dict(N=2, Cin=64, Cout=96, H=19, W=23, sigma=2.0)
    cases = [cast_case(make_case(50 + i, **kw), dtype, 'cuda') for i in range(4)]
    static = {k: cases[0][k].clone() for k in ('input', 'offset', 'mask', 'weight', 'bias')}
    call = lambda c: modulated_deform_conv2d(c['input'], c['offset'], c['mask'], c['weight'], c['bias'], 1, 1, 1, 1, 1)
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):   # warm up on the capture stream, as torch's recipe asks
            for _ in range(2):
                call(static)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = call(static)
        for i in (1, 2, 3, 0):
            for k in static:
                static[k].copy_(cases[i][k])
            graph.replay()
            torch.cuda.synchronize()
            got = out.clone()
            eager = call(cases[i])          # (eager work and a synchronisation between replays)
            torch.cuda.synchronize()
            assert torch.equal(got, eager), i
