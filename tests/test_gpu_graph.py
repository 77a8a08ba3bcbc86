"""The operator entry points under HIP graph capture: the local operator, the deformable operator
and the N-d sampler (its sort of the points by cell included) launch kernels and copies only (no
memset nodes, no synchronisation, no allocation), so a captured forward + backward replays correctly.  Each graph is replayed several times, with eager work,
new input values and synchronisations between the replays, and every replay is compared with
the same calls issued eagerly."""
import pytest
import torch

from _cases import make_deform, make_local

pytestmark = pytest.mark.gpu


def _fresh(tensors, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(t.shape, generator=g) * float(t.std()) for t in tensors]


def test_local_operator_forward_and_backward_replay_from_a_graph():
    from deformable_kernels.ops.deform_kernel import _lib
    L, P = _lib.lib(), _lib.ptr
    dev = torch.device("cuda:0")
    x, wt, rot, gout, cfg = make_local(4, 48, 28, 28, 3, (4, 4), 1, 1, 1, 1, 0.7, seed=21)
    xg, wg, rg, gg = [t.to(dev) for t in (x, wt, rot, gout)]
    desc = _lib.conv_desc(xg, wg, cfg["kernel_size"], cfg["stride"], cfg["padding"], cfg["dilation"], 1)
    ws, nbytes = _lib.workspace(L.dk_sample_depthwise_backward_workspace(desc), dev)
    outs = [torch.empty_like(gg), torch.empty_like(xg), torch.empty_like(rg), torch.empty_like(wg)]

    def calls():
        s = torch.cuda.current_stream().cuda_stream
        _lib.check(L.dk_sample_depthwise_forward(desc, P(xg), P(rg), P(wg), P(outs[0]), s), "forward")
        _lib.check(L.dk_sample_depthwise_backward(desc, P(gg), P(xg), P(rg), P(wg), P(outs[1]), P(outs[2]),
                                                  P(outs[3]), P(ws), nbytes, s), "backward")

    calls()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        calls()
    for replay in range(3):
        for dst, src in zip((xg, rg, gg), _fresh((x, rot, gout), 100 + replay)):
            dst.copy_(src.to(dev))
        for o in outs:
            o.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        calls()  # eager, same inputs
        torch.cuda.synchronize()
        for g_, e_ in zip(got, outs):
            assert torch.equal(g_, e_), "replay %d" % replay


def test_deformable_operator_forward_and_backward_replay_from_a_graph():
    from deformable_kernels.ops.deform_kernel import _lib
    L, P = _lib.lib(), _lib.ptr
    dev = torch.device("cuda:0")
    x, wt, rot, off, gout, cfg = make_deform(3, 32, 28, 28, 3, (4, 4), 2, 1, 1, 1, 0.5, 2.0, seed=22)
    xg, wg, rg, og, gg = [t.to(dev) for t in (x, wt, rot, off, gout)]
    desc = _lib.conv_desc(xg, wg, cfg["kernel_size"], cfg["stride"], cfg["padding"], cfg["dilation"], 1)
    need = max(L.dk_deformable_sample_depthwise_backward_data_workspace(desc),
               L.dk_deformable_sample_depthwise_backward_offset_workspace(desc),
               L.dk_deformable_sample_depthwise_backward_rotation_workspace(desc),
               L.dk_deformable_sample_depthwise_backward_filter_workspace(desc))
    ws, nbytes = _lib.workspace(need, dev)
    outs = [torch.empty_like(gg), torch.empty_like(xg), torch.empty_like(og), torch.empty_like(rg),
            torch.empty_like(wg)]

    def calls():
        s = torch.cuda.current_stream().cuda_stream
        _lib.check(L.dk_deformable_sample_depthwise_forward(desc, P(xg), P(og), P(rg), P(wg), P(outs[0]), s), "fwd")
        _lib.check(L.dk_deformable_sample_depthwise_backward_data(desc, P(gg), P(og), P(rg), P(wg), P(outs[1]),
                                                                  P(ws), nbytes, s), "data")
        _lib.check(L.dk_deformable_sample_depthwise_backward_offset(desc, P(gg), P(xg), P(og), P(rg), P(wg),
                                                                    P(outs[2]), P(ws), nbytes, s), "offset")
        _lib.check(L.dk_deformable_sample_depthwise_backward_rotation(desc, P(gg), P(xg), P(og), P(rg), P(wg),
                                                                      P(outs[3]), P(ws), nbytes, s), "rotation")
        _lib.check(L.dk_deformable_sample_depthwise_backward_filter(desc, P(gg), P(xg), P(og), P(rg), P(outs[4]),
                                                                    P(ws), nbytes, s), "filter")

    calls()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        calls()
    for replay in range(3):
        for dst, src in zip((xg, og, gg), _fresh((x, off, gout), 200 + replay)):
            dst.copy_(src.to(dev))
        for o in outs:
            o.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        calls()
        torch.cuda.synchronize()
        for g_, e_ in zip(got, outs):
            assert torch.equal(g_, e_), "replay %d" % replay


def test_nd_sampler_sorted_by_cell_replays_from_a_graph():
    """70000 points in an 8 x 8 x 8 volume take the sorted path: order, forward, both gradients."""
    from deformable_kernels.ops.deform_kernel import _lib
    from _cases import rel_err
    L, P = _lib.lib(), _lib.ptr
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(23)
    data = torch.randn(64, 8, 8, 8, generator=g).to(dev)
    coord = (torch.rand(70000, 3, generator=g) * 10.0 - 1.5).to(dev)
    gout = torch.randn(70000, 64, generator=g).to(dev)
    desc = _lib.nd_desc(data, coord)
    assert L.dk_nd_linear_sample_order_bytes(desc) > 0
    order = torch.empty(L.dk_nd_linear_sample_order_bytes(desc), dtype=torch.uint8, device=dev)
    need = max(L.dk_nd_linear_sample_order_workspace(desc), L.dk_nd_linear_sample_forward_workspace(desc),
               L.dk_nd_linear_sample_backward_data_workspace(desc), L.dk_nd_linear_sample_backward_coord_workspace(desc))
    ws, nbytes = _lib.workspace(need, dev)
    outs = [torch.empty(70000, 64, device=dev), torch.empty_like(data), torch.empty_like(coord)]

    def calls():
        s = torch.cuda.current_stream().cuda_stream
        _lib.check(L.dk_nd_linear_sample_order(desc, P(coord), P(order), P(ws), nbytes, s), "order")
        _lib.check(L.dk_nd_linear_sample_forward(desc, P(data), P(coord), P(order), P(outs[0]), P(ws), nbytes, s), "fwd")
        _lib.check(L.dk_nd_linear_sample_backward_data(desc, P(gout), P(coord), P(order), P(outs[1]), P(ws), nbytes, s),
                   "data")
        _lib.check(L.dk_nd_linear_sample_backward_coord(desc, P(gout), P(data), P(coord), P(order), P(outs[2]), P(ws),
                                                        nbytes, s), "coord")

    calls()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        calls()
    for replay in range(3):
        gen = torch.Generator().manual_seed(300 + replay)
        coord.copy_((torch.rand(70000, 3, generator=gen) * 10.0 - 1.5).to(dev))
        gout.copy_(torch.randn(70000, 64, generator=gen).to(dev))
        for o in outs:
            o.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        calls()  # eager, same inputs
        torch.cuda.synchronize()
        assert torch.equal(got[0], outs[0]), "replay %d" % replay
        assert rel_err(got[1].cpu(), outs[1].cpu()) < 1e-5, "replay %d" % replay   # atomic sums: order differs
        assert torch.equal(got[2], outs[2]), "replay %d" % replay
