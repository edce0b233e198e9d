"""The allocation-free entry point mdcn_forward_noalloc() against mdcn_forward():
same kernels, scratch inside the library instead of a caller workspace.  Collected
last (file name) so that a failure here hides no other test."""
import ctypes

import pytest
import torch

from mmcv_amd import capi
from common import DT, capi_forward, cast_case, make_case

pytestmark = pytest.mark.gpu


def noalloc_forward(case):
    """mdcn_forward_noalloc through ctypes; every tensor is allocated before the call."""
    lib = capi.load()
    x, off, msk, w, b = (case[k] for k in ('input', 'offset', 'mask', 'weight', 'bias'))
    N, Cin, H, W = x.shape
    Cout, _, kh, kw = w.shape
    p = capi.make_params(DT[x.dtype], N, Cin, H, W, Cout, kh, kw, case['stride'], case['padding'],
                         case['dilation'], case['groups'], case['deform_groups'])
    rc, Ho, Wo = capi.output_size(p)
    assert rc == 0
    out = torch.full((N, Cout, Ho, Wo), 7.0, dtype=x.dtype, device=x.device)
    keep = [t.contiguous() for t in (x, off, msk, w, b)]
    p.input, p.offset, p.mask, p.weight, p.bias = (t.data_ptr() for t in keep)
    p.output = out.data_ptr()
    p.workspace, p.workspace_bytes = None, 0
    need = lib.mdcn_workspace_bytes(ctypes.byref(p))
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()['allocation.all.allocated']
    rc = lib.mdcn_forward_noalloc(ctypes.byref(p), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    after = torch.cuda.memory_stats()['allocation.all.allocated']
    torch.cuda.synchronize()
    return rc, out, need, after - before


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32])
def test_two_calls_in_a_row_match_the_workspace_entry_point(dtype):
    dev = torch.device('cuda:0')
    # fused-path shapes; the second is smaller, so it reuses a scratch that still holds the first one's data
    big = cast_case(make_case(11, 2, 128, 96, 40, 52, sigma=3.0), dtype, dev)
    small = cast_case(make_case(12, 1, 64, 64, 17, 23, stride=2, sigma=2.0), dtype, dev)
    for case in (big, small):
        ref = capi_forward(case)
        rc, out, need, allocs = noalloc_forward(case)
        assert rc == 0, capi.status_string(rc)
        assert 0 < need <= capi.NOALLOC_SCRATCH_BYTES
        assert allocs == 0
        assert torch.equal(out, ref)  # same kernels on the same inputs: bit-equal


def test_scratch_limit_is_reported_and_nothing_runs():
    dev = torch.device('cuda:0')
    case = cast_case(make_case(13, 9, 256, 64, 100, 152), torch.bfloat16, dev)  # 72.7 MB input copy
    rc, out, need, _ = noalloc_forward(case)
    assert need > capi.NOALLOC_SCRATCH_BYTES
    assert rc == -8 and 'scratch' in capi.status_string(rc)
    assert bool((out == 7.0).all())


def test_direct_path_shapes_need_no_scratch():
    dev = torch.device('cuda:0')
    case = cast_case(make_case(14, 1, 3, 5, 9, 11), torch.float32, dev)  # 3 channels: one thread per output
    rc, out, need, _ = noalloc_forward(case)
    assert rc == 0 and need == 0
    assert torch.equal(out, capi_forward(case))


def _free_device_bytes():
    hip = ctypes.CDLL('libamdhip64.so')
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


def test_in_a_captured_graph_after_one_warm_up_call():
    """After one ordinary call on the device (which resolves the scratch address and the CU count)
    the entry point only enqueues kernels: it can be captured into a HIP graph, replays match
    mdcn_forward() on new contents of the captured tensors, and the device's free memory does
    not move over the calls."""
    lib = capi.load()
    dev = torch.device('cuda:0')
    kw = dict(N=2, Cin=128, Cout=256, H=24, W=32, sigma=2.0)
    cases = [cast_case(make_case(60 + i, **kw), torch.bfloat16, dev) for i in range(3)]
    static = {k: cases[0][k].clone().contiguous() for k in ('input', 'offset', 'mask', 'weight', 'bias')}
    N, Cin, H, W = static['input'].shape
    Cout = static['weight'].shape[0]
    p = capi.make_params(capi.MDCN_BF16, N, Cin, H, W, Cout, 3, 3, (1, 1), (1, 1), (1, 1), 1, 1)
    out = torch.zeros(N, Cout, H, W, dtype=torch.bfloat16, device=dev)
    p.input, p.offset, p.mask, p.weight, p.bias = (static[k].data_ptr() for k in ('input', 'offset', 'mask', 'weight', 'bias'))
    p.output = out.data_ptr()
    side = torch.cuda.Stream()
    call = lambda: lib.mdcn_forward_noalloc(ctypes.byref(p), ctypes.c_void_p(side.cuda_stream))
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        assert call() == 0          # the warm-up call, outside any capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        assert call() == 0
    for i in (1, 2, 0):
        for k in static:
            static[k].copy_(cases[i][k])
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        ref = capi_forward(cases[i])    # (eager work and a synchronisation between the replays)
        assert torch.equal(got, ref), i
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        free1 = _free_device_bytes()
        assert call() == 0
        side.synchronize()
        assert _free_device_bytes() == free1   # an eager call allocates nothing on the device either
