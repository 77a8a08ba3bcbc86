"""`dk_sample_depthwise_backward_filter_static`: the filter gradient for callers that cannot
allocate (its partial sums live in a buffer inside the library's device image).  It runs the
kernels of `dk_sample_depthwise_backward_filter`, so its result has to be bit-identical to that
entry point's -- also on a second call with a smaller input, which finds the buffer full of the
first call's partial sums (where the generic kernel runs, whose LDS atomics
make the last bits vary from launch to launch: equal to the float64 bar of 1e-11) -- and it has to refuse, launching nothing, what does not fit."""
import pytest
import torch

from _cases import make_local, rel_err

pytestmark = pytest.mark.gpu

# (N, C, H, W, scope, stride, dtype): the first needs most of the static buffer, the second little
CASES = [
    (16, 144, 56, 56, (4, 4), 1, torch.float32),
    (3, 40, 28, 28, (4, 4), 1, torch.float32),
    (2, 24, 30, 30, (5, 5), 2, torch.bfloat16),
    (2, 6, 9, 11, (3, 3), 1, torch.float64),   # generic kernels
]


def _both(L, _lib, case, seed):
    N, C, H, W, S, stride, dtype = case
    dev = torch.device("cuda:0")
    x, wt, rot, gout, cfg = make_local(N, C, H, W, 3, S, stride, 1, 1, 1, 1.0, seed=seed, dtype=dtype)
    xg, wg, rg, gg = [t.to(dev) for t in (x, wt, rot, gout)]
    desc = _lib.conv_desc(xg, wg, cfg["kernel_size"], cfg["stride"], cfg["padding"], cfg["dilation"], 1)
    P = _lib.ptr
    s = torch.cuda.current_stream().cuda_stream
    need = L.dk_sample_depthwise_backward_filter_workspace(desc)
    ws, nbytes = _lib.workspace(need, dev)
    want = torch.full_like(wg, float("nan"))
    _lib.check(L.dk_sample_depthwise_backward_filter(desc, P(gg), P(xg), P(rg), P(want), P(ws), nbytes, s), "filter")
    got = torch.full_like(wg, float("nan"))
    _lib.check(L.dk_sample_depthwise_backward_filter_static(desc, P(gg), P(xg), P(rg), P(got), s), "filter_static")
    torch.cuda.synchronize()
    return got, want, need


def test_static_scratch_filter_gradient_equals_the_workspace_entry_point_on_consecutive_calls():
    from deformable_kernels.ops.deform_kernel import _lib
    L = _lib.lib()
    sizes = []
    for i, case in enumerate(CASES):
        print("case", case, flush=True)
        got, want, need = _both(L, _lib, case, seed=300 + i)
        sizes.append(need)
        assert torch.isfinite(want).all()
        if case[-1] == torch.float64:
            # the generic kernel adds into LDS with hardware atomics: the order of the additions, and
            # with it the last bits, differ from launch to launch
            assert rel_err(got.cpu(), want.cpu()) < 1e-11, case
        else:
            assert torch.equal(got, want), case
    assert sizes[0] > sizes[1] > 0  # the second call is the smaller one and reuses the buffer


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    from deformable_kernels.ops.deform_kernel import _lib
    L, P = _lib.lib(), _lib.ptr
    dev = torch.device("cuda:0")
    # 1024 channels with a 5 x 5 scope: one partial buffer per workgroup comes to 13 MB
    x = torch.zeros(8, 1024, 14, 14, device=dev)
    wt = torch.zeros(1024, 1, 5, 5, device=dev)
    rot = torch.zeros(8, 18, 14, 14, device=dev)
    desc = _lib.conv_desc(x, wt, (3, 3), (1, 1), (1, 1), (1, 1), 1)
    need = L.dk_sample_depthwise_backward_filter_workspace(desc)
    assert need > (8 << 20), need
    gw = torch.full_like(wt, 7.0)
    rc = L.dk_sample_depthwise_backward_filter_static(desc, P(x), P(x), P(rot), P(gw), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == -8 and b"static" in L.dk_status_string(rc)
    assert bool((gw == 7.0).all())  # nothing was launched


def test_static_scratch_entry_point_in_a_graph_after_a_warm_up_call():
    """The first call for a (device, shape) looks the buffer's address up and sets a kernel attribute, which a
    capturing stream may refuse; after one ordinary call the entry point is launches only and can be captured.
    The graph is replayed three times with eager work of the library in between (another shape through the same
    buffer), and every replay must give the workspace entry point's bits."""
    from deformable_kernels.ops.deform_kernel import _lib
    L, P = _lib.lib(), _lib.ptr
    dev = torch.device("cuda:0")
    N, C, H, W, S, stride, dtype = CASES[1]
    x, wt, rot, gout, cfg = make_local(N, C, H, W, 3, S, stride, 1, 1, 1, 1.0, seed=77, dtype=dtype)
    xg, wg, rg, gg = [t.to(dev) for t in (x, wt, rot, gout)]
    desc = _lib.conv_desc(xg, wg, cfg["kernel_size"], cfg["stride"], cfg["padding"], cfg["dilation"], 1)
    need = L.dk_sample_depthwise_backward_filter_workspace(desc)
    ws, nbytes = _lib.workspace(need, dev)
    want = torch.empty_like(wg)
    s0 = torch.cuda.current_stream().cuda_stream
    _lib.check(L.dk_sample_depthwise_backward_filter(desc, P(gg), P(xg), P(rg), P(want), P(ws), nbytes, s0), "filter")
    got = torch.zeros_like(wg)
    _lib.check(L.dk_sample_depthwise_backward_filter_static(desc, P(gg), P(xg), P(rg), P(got), s0), "warm-up")
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = L.dk_sample_depthwise_backward_filter_static(desc, P(gg), P(xg), P(rg), P(got), side.cuda_stream)
    assert rc == 0
    for i in range(3):
        got.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want), "replay %d" % i
        other, other_want, _ = _both(L, _lib, CASES[2], seed=500 + i)  # eager use of the same buffer in between
        assert torch.equal(other, other_want)
