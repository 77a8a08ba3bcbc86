"""GPU parity of the N-d linear sampler (forward, grad-data, grad-coord) against the CPU
oracle.  fp32: forward 1e-5 against the fp32 oracle, gradients 1e-4 against the fp64 oracle;
fp64 1e-11; fp16 / bf16 1e-2 against the fp32 oracle on the rounded inputs."""
import numpy as np
import pytest
import torch

from _cases import rel_err
from oracle import dk_oracle as orc

pytestmark = pytest.mark.gpu


def _inputs(shape, C, B, seed, dtype, lo=-1.5, extra=1.5):
    g = torch.Generator().manual_seed(seed)
    data = torch.randn(C, *shape, generator=g)
    hi = torch.tensor(shape, dtype=torch.float32)
    coord = torch.rand(B, len(shape), generator=g) * (hi + extra - lo) + lo  # spills outside on both sides
    gout = torch.randn(B, C, generator=g)
    return data.to(dtype), coord.to(dtype), gout.to(dtype)


def _run(data, coord, gout):
    from deformable_kernels.ops.deform_kernel.functions import nd_linear_sample
    dev = torch.device("cuda:0")
    dg, cg = data.to(dev).requires_grad_(), coord.to(dev).requires_grad_()
    out = nd_linear_sample(dg, cg)
    out.backward(gout.to(dev))
    torch.cuda.synchronize()
    return out.detach().cpu(), dg.grad.cpu(), cg.grad.cpu()


def _oracle(data, coord, gout, np_dtype):
    a = [t.to(torch.float64).numpy().astype(np_dtype) for t in (data, coord, gout)]
    out = orc.nd_linear_sample_forward(a[0], a[1])
    gd, gc = orc.nd_linear_sample_backward(a[2], a[0], a[1])
    return out, gd, gc


@pytest.mark.parametrize("shape,C,B", [((9,), 5, 70), ((5, 5), 256, 1152), ((4, 5, 6), 7, 333),
                                       ((3, 4, 2, 5), 3, 200), ((2, 2), 1, 1),
                                       ((9,), 40, 3000), ((6, 7, 5), 100, 1001), ((5, 4), 16, 4097)])
def test_fp32_matches_oracle(shape, C, B):
    data, coord, gout = _inputs(shape, C, B, seed=41, dtype=torch.float32)
    got = _run(data, coord, gout)
    o32, o64 = _oracle(data, coord, gout, np.float32), _oracle(data, coord, gout, np.float64)
    assert got[0].shape == (B, C)
    assert rel_err(got[0], o32[0]) < 1e-5
    assert rel_err(got[1], o64[1]) < 1e-4
    assert rel_err(got[2], o64[2]) < 1e-4


@pytest.mark.parametrize("shape,C,B,lo,hi", [
    ((8, 8, 8), 64, 65536 + 37, -1.5, 9.5),    # many points per cell: the sorted-by-cell kernels; ragged last wave
    ((16, 12), 80, 70001, -1.5, 17.0),         # two channel passes (64 + 16)
    ((40,), 16, 66000, -2.0, 42.0),            # one dimension
    ((8, 8, 8), 32, 65536, -1.0, 1.0),         # config 5's coordinate range: every point in the 8 corner cells
    ((6, 5, 4), 64, 65536, 2.2, 2.9),          # every point in one cell
    ((10, 9), 128, 66000, -1.5, 10.5),         # two dimensions, two 64-channel blocks of the matrix-core kernels
    ((50,), 64, 66000, -2.0, 52.0),            # one dimension on the matrix-core kernels
    ((5, 6, 7), 192, 65536, -1.5, 7.5),        # three 64-channel blocks
])
def test_many_points_per_cell_match_oracle(shape, C, B, lo, hi):
    g = torch.Generator().manual_seed(45)
    data = torch.randn(C, *shape, generator=g)
    coord = torch.rand(B, len(shape), generator=g) * (hi - lo) + lo
    gout = torch.randn(B, C, generator=g)
    got = _run(data, coord, gout)
    o32, o64 = _oracle(data, coord, gout, np.float32), _oracle(data, coord, gout, np.float64)
    assert rel_err(got[0], o32[0]) < 1e-5
    assert rel_err(got[1], o64[1]) < 1e-4
    assert rel_err(got[2], o64[2]) < 1e-4


def test_many_points_on_grid_nodes_and_half_way_between():
    # fractional positions of exactly 0 and 0.5: a corner with interpolation weight 0 still
    # enters the coordinate gradient
    g = torch.Generator().manual_seed(47)
    data = torch.randn(32, 7, 6, 5, generator=g)
    hi = torch.tensor([7.0, 6.0, 5.0])
    coord = torch.round((torch.rand(65536, 3, generator=g) * (hi + 2.0) - 1.0) * 2.0) / 2.0
    gout = torch.randn(65536, 32, generator=g)
    got = _run(data, coord, gout)
    o32, o64 = _oracle(data, coord, gout, np.float32), _oracle(data, coord, gout, np.float64)
    assert rel_err(got[0], o32[0]) < 1e-5
    assert rel_err(got[1], o64[1]) < 1e-4
    assert rel_err(got[2], o64[2]) < 1e-4


def test_sorted_and_unsorted_kernels_agree(switch_off):
    g = torch.Generator().manual_seed(46)
    data = torch.randn(64, 8, 8, 8, generator=g)
    coord = torch.rand(70000, 3, generator=g) * 10.0 - 1.0
    gout = torch.randn(70000, 64, generator=g)
    a = _run(data, coord, gout)
    switch_off("DK_NO_ND_BINS")
    b = _run(data, coord, gout)
    assert rel_err(a[0], b[0]) < 1e-6  # the same eight products per point and channel, summed in another order
    assert rel_err(a[1], b[1]) < 1e-5
    assert rel_err(a[2], b[2]) < 1e-5


def test_sorted_kernels_with_and_without_the_matrix_cores_agree(switch_off):
    """64 channels in fp32 take the matrix-core kernels; switched off, the VALU kernels serve the same call."""
    g = torch.Generator().manual_seed(47)
    data = torch.randn(64, 7, 9, 8, generator=g)
    coord = torch.rand(66000, 3, generator=g) * 11.0 - 1.5
    gout = torch.randn(66000, 64, generator=g)
    a = _run(data, coord, gout)
    switch_off("DK_NO_ND_MFMA")
    b = _run(data, coord, gout)
    want = _oracle(data, coord, gout, np.float64)
    for x, y, w in zip(a, b, want):
        assert rel_err(x, y) < 1e-5
        assert rel_err(y, w) < 1e-4


@pytest.mark.parametrize("dtype,C,B", [(torch.float32, 256, 1152), (torch.float16, 64, 4096), (torch.bfloat16, 100, 700)])
def test_channel_last_kernels_on_few_points_over_a_tiny_volume(dtype, C, B, switch_off):
    """Few points on a volume of at most 64 cells take the direct kernels and the one-launch grad
    data; with that path switched off the channel-last kernels serve the same call."""
    data, coord, gout = _inputs((5, 5), C, B, seed=44, dtype=dtype)
    small = _run(data, coord, gout)
    switch_off("DK_NO_ND_SMALL")
    general = _run(data, coord, gout)
    want = _oracle(data, coord, gout, np.float64)
    tol = (1e-5, 1e-4, 1e-4) if dtype == torch.float32 else (1e-2, 1e-2, 1e-2)
    for a, b, w, t in zip(small, general, want, tol):
        assert rel_err(a.float(), w) < t
        assert rel_err(b.float(), w) < t


def test_fp64_matches_oracle():
    data, coord, gout = _inputs((4, 5, 6), 9, 257, seed=42, dtype=torch.float64)
    got = _run(data, coord, gout)
    want = _oracle(data, coord, gout, np.float64)
    for g, w in zip(got, want):
        assert rel_err(g, w) < 1e-11


@pytest.mark.parametrize("points", [300, 4096, 65536])   # direct path / channel-last path / sorted by cell
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_half_precisions_match_fp32_oracle(dtype, points):
    data, coord, gout = _inputs((5, 5), 64, points, seed=43, dtype=dtype)
    got = _run(data, coord, gout)
    want = _oracle(data, coord, gout, np.float32)
    for g, w in zip(got, want):
        assert g.dtype == dtype
        assert rel_err(g.float(), w) < 1e-2


def test_zero_rule_and_fade_bands_on_gpu():
    data = torch.ones(1, 4, 4)
    pts = torch.tensor([[-1.0, 1.0], [1.0, -1.0], [4.0, 1.0], [1.0, 4.0], [-0.5, 1.0], [3.5, 3.5], [3.0, 3.0]])
    out, _, gc = _run(data, pts, torch.ones(7, 1))
    assert out[:4, 0].tolist() == [0, 0, 0, 0]
    assert torch.allclose(out[4:, 0], torch.tensor([0.5, 0.25, 1.0]))
    assert torch.count_nonzero(gc[:4]).item() == 0


def test_trilinear_volume_slice_of_config5():
    """Config 5's standalone case at reduced point count: data [64, 32, 32, 32], coordinates
    uniform in [-1, 1]^3 as written there (half the points in the fade band) and uniform over
    the whole volume."""
    g = torch.Generator().manual_seed(44)
    data = torch.randn(64, 32, 32, 32, generator=g)
    for lo, hi in ((-1.0, 1.0), (-1.0, 32.0)):
        coord = torch.rand(4096, 3, generator=g) * (hi - lo) + lo
        gout = torch.randn(4096, 64, generator=g)
        got = _run(data, coord, gout)
        o32, o64 = _oracle(data, coord, gout, np.float32), _oracle(data, coord, gout, np.float64)
        assert rel_err(got[0], o32[0]) < 1e-5
        assert rel_err(got[1], o64[1]) < 1e-4
        assert rel_err(got[2], o64[2]) < 1e-4
