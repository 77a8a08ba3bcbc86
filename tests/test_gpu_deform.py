"""GPU parity of the deformable variant (kernel-space + image-space offsets):
forward, grad-input, grad-offset, grad-rotation, grad-filter against the CPU
oracle, through the Python Function and the C ABI.

Tolerances relative to the largest expected magnitude: fp32 forward 1e-5
against the fp32 oracle; the four gradients 1e-4 against the fp64 oracle
(grad-input is an atomic scatter, the others are reductions, so summation order
differs from the oracle's); fp64 1e-11; fp16 / bf16 1e-2 against the fp32
oracle on the rounded inputs."""
import numpy as np
import pytest
import torch

from _cases import mixed_err, clipped_rotation, make_deform, rel_err
from oracle import dk_oracle as orc

pytestmark = pytest.mark.gpu

# N, C, H, W, k, S, stride, pad, dil, groups, rot_std, off_std
CASES = [
    (2, 16, 14, 14, 3, (4, 4), 2, 1, 1, 1, 0.5, 2.0),     # benchmark configuration 4 geometry, small
    (2, 12, 13, 11, 3, (4, 4), 1, 1, 1, 1, 1.0, 2.0),
    (2, 12, 9, 10, 3, (4, 4), 1, 2, 2, 3, 0.7, 3.0),      # dilation, rotation groups
    (1, 8, 12, 12, 3, (3, 3), 1, 1, 1, 1, 0.0, 1.5),      # DeformConv2d: scope == kernel, zero rotation
    (2, 6, 8, 8, (2, 3), (4, 5), (1, 2), (0, 1), 1, 3, 0.7, 1.0),
    (1, 3, 6, 5, 1, (2, 2), 1, 0, 1, 1, 0.6, 3.0),
    (1, 20, 24, 24, 3, (4, 4), 1, 1, 1, 2, 0.7, 2.0),     # 576 output pixels: three pixel tiles, two groups
    (1, 6, 33, 60, 3, (5, 5), 1, 1, 1, 1, 1.0, 2.5),      # wide plane (16 staging passes), scope 5, > 1024 output pixels
    (2, 80, 10, 10, 3, (3, 3), 1, 1, 1, 1, 0.8, 1.0),     # many channels: several channel chunks per image
    (1, 8, 20, 18, 3, (4, 4), 2, 1, 1, 1, 0.5, 6.0),      # large offsets: many samples outside the image
    (2, 10, 40, 36, 3, (4, 4), 1, 1, 1, 2, 0.7, 2.0),     # 1440 output pixels: tiled grad input, 5 channels per group (partial chunk)
    (2, 27, 14, 14, 3, (4, 4), 2, 1, 1, 1, 0.5, 2.0),     # three chunks of 9 channels: the four-channel tuples end in a single channel
    (1, 9, 16, 17, 3, (5, 5), 1, 1, 1, 1, 1.0, 2.0),      # scope 5 on the channel-interleaved kernels
    (1, 9, 56, 56, 3, (4, 4), 1, 1, 1, 1, 0.7, 2.0),      # 56 x 56: 512-thread channel-interleaved kernels, 7 tiles of 7 waves
    (1, 6, 64, 64, 3, (5, 5), 2, 1, 1, 1, 1.0, 2.5),      # the largest plane they take, stride 2
    (2, 10, 45, 50, 3, (3, 3), 1, 1, 1, 2, 0.6, 3.0),     # 5 tiles of 512, the last one ragged; two groups, scope 3; one sample on a grid line in fp32
    (1, 5, 112, 112, 3, (4, 4), 1, 1, 1, 1, 0.7, 2.0),    # 112 x 112: wider than 64 columns, row-window staging, one 64-bit plane per workgroup in grad input
    (1, 4, 40, 130, 3, (3, 3), 1, 1, 1, 2, 0.6, 3.0),     # 130 columns: 256 lanes per staged row, two groups
    (2, 6, 112, 112, 3, (4, 4), 2, 1, 1, 1, 0.5, 8.0),    # 112 x 112 stride 2 with offsets that spread a tile's samples over most of the plane
    (1, 3, 100, 30, 3, (5, 5), 1, 1, 1, 1, 1.0, 2.5),     # narrow but taller than the 256-thread staging covers; scope 5
    (1, 20, 60, 40, 3, (4, 4), 1, 1, 1, 2, 0.7, 10.0),    # row-window grad filter: offsets of ten rows spread a tile's samples over three windows of 24 rows; two channel blocks, the second partial
    (2, 33, 56, 56, 3, (5, 5), 1, 1, 1, 1, 1.0, 2.0),     # row-window grad filter, scope 5 (two launches of 16 cells), three channel blocks
    (1, 6, 120, 100, 3, (4, 4), 1, 1, 1, 1, 0.7, 15.0),   # row-window channel-interleaved kernels (100 columns): offsets of fifteen rows, four windows of 32 rows per tile; two channel tuples
    (2, 9, 70, 96, 3, (3, 3), 1, 1, 1, 3, 0.6, 2.0),      # the same kernels in one pass: three groups of three channels, scope 3
    (1, 10, 224, 224, 3, (4, 4), 1, 1, 1, 1, 0.7, 2.0),   # 224 x 224: no padded plane fits LDS; grad input in bands of 20 rows (a chunk of 8 channels and one of 2), row windows with the smaller margin
    (1, 6, 150, 200, 3, (4, 4), 2, 1, 1, 2, 0.6, 12.0),   # the band form at stride 2 with offsets of twelve rows (every band walks many tiles), two groups of three channels
    (4, 40, 56, 56, 3, (4, 4), 1, 1, 1, 1, 0.7, 2.0),     # row-window grad filter with more (tile, channel block) units than persistent workgroups: 300 units on 256, runs that start and end inside a tile
    (1, 40, 112, 112, 3, (4, 4), 1, 1, 1, 1, 0.7, 2.0),   # the same for the rows-and-columns-window grad filter: 98 tiles x 3 channel blocks
]
NAMES = ("forward", "grad input", "grad offset", "grad rotation", "grad filter")


def _run(case, dtype, seed=0):
    from deformable_kernels.ops.deform_kernel.functions import deform_sample_depthwise
    N, C, H, W, k, S, s, p, d, G, rs, os_ = case
    x, wt, rot, off, gout, cfg = make_deform(N, C, H, W, k, S, s, p, d, G, rs, os_, seed=seed, dtype=dtype)
    dev = torch.device("cuda:0")
    xg, og, rg, wg = [t.to(dev).requires_grad_() for t in (x, off, rot, wt)]
    out = deform_sample_depthwise(xg, og, rg, wg, cfg["kernel_size"], cfg["stride"], cfg["padding"],
                                  cfg["dilation"], cfg["groups"])
    out.backward(gout.to(dev))
    torch.cuda.synchronize()
    return (x, wt, rot, off, gout, cfg), [t.detach().cpu() for t in (out, xg.grad, og.grad, rg.grad, wg.grad)]


def _oracle(inputs, np_dtype):
    x, wt, rot, off, gout, cfg = inputs
    a = [t.to(torch.float64).numpy().astype(np_dtype) for t in (x, off, rot, wt, gout)]
    out = orc.deform_sample_depthwise_forward(a[0], a[1], a[2], a[3], **cfg)
    return (out,) + tuple(orc.deform_sample_depthwise_backward(a[4], a[0], a[1], a[2], a[3], **cfg))


def assert_fp32_parity(got, o32, o64):
    assert rel_err(got[0], o32[0]) < 1e-5, NAMES[0]
    # grad input: fixed-point sums, exact on a grid of 2^-24 of the largest term or finer
    assert mixed_err(got[1], o64[1]) < 1e-5, NAMES[1]
    for i in (3, 4):
        assert rel_err(got[i], o64[i]) < 1e-4, NAMES[i]
    # The offset gradient is the slope of the bilinear patch a sample falls in, so it jumps where a
    # sampling position crosses a grid line; a position that fp32 rounds onto the line (36 + 0.9999987
    # = 37.0f) lies in the next patch than in fp64.  Each element must match one of the two oracles,
    # and all but a few the fp64 one (a few per million samples: the bound grows with the tensor).
    g = got[2].double().numpy()
    err = np.minimum(np.abs(g - o64[2]), np.abs(g - o32[2].astype(np.float64)))
    assert err.max() / np.abs(o64[2]).max() < 1e-4, NAMES[2]
    assert np.count_nonzero(np.abs(g - o64[2]) > 1e-4 * np.abs(o64[2]).max()) <= 2 + g.size // 250000, NAMES[2]


@pytest.mark.parametrize("case", CASES)
def test_fp32_matches_oracle(case):
    inputs, got = _run(case, torch.float32)
    assert_fp32_parity(got, _oracle(inputs, np.float32), _oracle(inputs, np.float64))


@pytest.mark.parametrize("case", CASES[:3])
def test_fp64_matches_oracle(case):
    inputs, got = _run(case, torch.float64)
    want = _oracle(inputs, np.float64)
    for g, w, name in zip(got, want, NAMES):
        assert rel_err(g, w) < 1e-11, name


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", CASES[:3] + [CASES[10], CASES[13], CASES[14], CASES[16], CASES[17], CASES[24], CASES[26], CASES[27]])   # planes above 30 x 30; wider than 64 columns; 224 x 224; persistent grad filter
def test_half_precisions_match_fp32_oracle(case, dtype):
    inputs, got = _run(case, dtype)
    want = _oracle(inputs, np.float32)
    for g, w, name in zip(got, want, NAMES):
        assert g.dtype == dtype
        assert rel_err(g.float(), w) < 1e-2, name


@pytest.mark.parametrize("clip", [(-0.5, 0.25), 'scope'])
@pytest.mark.parametrize("case", [CASES[0], CASES[2], CASES[4], CASES[6]])
def test_rotation_clip_inside_the_operator(case, clip):
    # the operator clamping the kernel-space offsets itself == clamping the tensor first
    from deformable_kernels.ops.deform_kernel.functions import deform_sample_depthwise
    N, C, H, W, k, S, s, p, d, G, rs, os_ = case
    x, wt, rot, off, gout, cfg = make_deform(N, C, H, W, k, S, s, p, d, G, 2.0 * rs, os_, seed=7)
    dev = torch.device("cuda:0")
    xg, og, rg, wg = [t.to(dev).requires_grad_() for t in (x, off, rot, wt)]
    out = deform_sample_depthwise(xg, og, rg, wg, cfg["kernel_size"], cfg["stride"], cfg["padding"],
                                  cfg["dilation"], cfg["groups"], clip)
    out.backward(gout.to(dev))
    got = [t.detach().cpu() for t in (out, xg.grad, og.grad, rg.grad, wg.grad)]
    rot_c, open_ = clipped_rotation(rot, clip, cfg["kernel_size"], S, G)
    assert 0.02 < 1.0 - open_.float().mean().item() < 0.9
    inputs = (x, wt, rot_c, off, gout, cfg)
    o32, o64 = _oracle(inputs, np.float32), _oracle(inputs, np.float64)
    assert rel_err(got[0], o32[0]) < 1e-5, NAMES[0]
    for i in (1, 2, 4):
        assert rel_err(got[i], o64[i]) < 1e-4, NAMES[i]
    assert rel_err(got[3], torch.as_tensor(o64[3]) * open_) < 1e-4, NAMES[3]
    assert (got[3][~open_] == 0).all()


# 14 x 14: one workgroup per output plane; 40 x 36 with 11 channels: the tiled kernel (planes above 1024 pixels:
# a plane per channel and two walks over the tiles when an element collects more than 64 samples, last chunk ragged)
@pytest.mark.parametrize("case", [(2, 12, 14, 14, 3, (4, 4), 1, 1, 1, 1, 0.5, 0.0),
                                  (1, 11, 40, 36, 3, (4, 4), 1, 1, 1, 1, 0.5, 0.0)])
def test_grad_input_when_every_sample_lands_on_one_input_element(case):
    # all 9 x P samples of an image within one input cell: the grad-input kernel's fixed-point
    # scale has to leave room for that many terms in one sum
    from deformable_kernels.ops.deform_kernel.functions import deform_sample_depthwise
    N, C, H, W, k, S, s, p, d, G, rs, os_ = case
    x, wt, rot, off, gout, cfg = make_deform(N, C, H, W, k, S, s, p, d, G, rs, os_, seed=9)
    g = torch.Generator().manual_seed(1)
    oh, ow = torch.meshgrid(torch.arange(H), torch.arange(W), indexing="ij")
    for t in range(9):
        # tap position oh - 1 + t // 3, ow - 1 + t % 3; target (6.3, 7.6) plus a little jitter
        off[:, 2 * t] = 6.3 - (oh - 1 + t // 3) + 0.2 * torch.rand(N, H, W, generator=g)
        off[:, 2 * t + 1] = 7.6 - (ow - 1 + t % 3) + 0.2 * torch.rand(N, H, W, generator=g)
    dev = torch.device("cuda:0")
    xg, og, rg, wg = [t_.to(dev).requires_grad_() for t_ in (x, off, rot, wt)]
    out = deform_sample_depthwise(xg, og, rg, wg, cfg["kernel_size"], cfg["stride"], cfg["padding"],
                                  cfg["dilation"], cfg["groups"])
    out.backward(gout.to(dev))
    got = [t_.detach().cpu() for t_ in (out, xg.grad, og.grad, rg.grad, wg.grad)]
    inputs = (x, wt, rot, off, gout, cfg)
    o32, o64 = _oracle(inputs, np.float32), _oracle(inputs, np.float64)
    assert rel_err(got[0], o32[0]) < 1e-5, NAMES[0]
    assert rel_err(got[1], o64[1]) < 1e-5, NAMES[1]
    for i in range(2, 5):
        assert rel_err(got[i], o64[i]) < 1e-4, NAMES[i]


def test_zero_image_offsets_equal_the_local_operator_on_gpu():
    from deformable_kernels.ops.deform_kernel.functions import deform_sample_depthwise, sample_depthwise
    x, wt, rot, off, gout, cfg = make_deform(2, 16, 12, 12, 3, (4, 4), 1, 1, 1, 1, 1.0, 0.0, seed=3)
    dev = torch.device("cuda:0")
    args = (cfg["kernel_size"], cfg["stride"], cfg["padding"], cfg["dilation"], cfg["groups"])
    a = deform_sample_depthwise(x.to(dev), off.to(dev), rot.to(dev), wt.to(dev), *args)
    b = sample_depthwise(x.to(dev), rot.to(dev), wt.to(dev), *args)
    assert rel_err(a.cpu(), b.cpu()) < 1e-6


def test_samples_outside_the_image_give_exact_zeros():
    from deformable_kernels.ops.deform_kernel.functions import deform_sample_depthwise
    x, wt, rot, off, gout, cfg = make_deform(1, 4, 8, 8, 3, (4, 4), 1, 1, 1, 1, 0.3, 0.0, seed=4)
    dev = torch.device("cuda:0")
    for shift in (-30.0, 30.0):
        ts = [t.to(dev).requires_grad_() for t in (x, off + shift, rot, wt)]
        out = deform_sample_depthwise(*ts, (3, 3), (1, 1), (1, 1), (1, 1), 1)
        out.backward(gout.to(dev))
        for t in [out] + [t.grad for t in ts]:
            assert torch.count_nonzero(t).item() == 0


def test_config4_shape_on_a_batch_slice():
    """benchmark configuration 4 geometry at full channel count (C=512, 28x28 -> 14x14, stride 2) on 4
    images: forward and all four gradients against the oracle."""
    case = (4, 512, 28, 28, 3, (4, 4), 2, 1, 1, 1, 0.5, 2.0)
    inputs, got = _run(case, torch.float32)
    o32, o64 = _oracle(inputs, np.float32), _oracle(inputs, np.float64)
    assert rel_err(got[0], o32[0]) < 1e-5
    for i in range(1, 5):
        assert rel_err(got[i], o64[i]) < 1e-4, NAMES[i]


def test_config4_properties_at_full_size():
    """benchmark configuration 4 (N=64, C=512, 28x28 -> 14x14, stride 2, fp32) at full size: the oracle on
    two images; the whole batch through properties that need no oracle -- the operator is linear
    in the input and in the filter, so <gout, F> = <grad_input, x> = <grad_filter, Wt>, and it is
    independent per image."""
    from deformable_kernels.ops.deform_kernel.functions import deform_sample_depthwise
    case = (64, 512, 28, 28, 3, (4, 4), 2, 1, 1, 1, 0.5, 2.0)
    (x, wt, rot, off, gout, cfg), got = _run(case, torch.float32)
    out, gin, goff, grot, gw = got
    for n in (0, 63):
        sl = slice(n, n + 1)
        a = [t[sl].double().numpy() for t in (x, off, rot)] + [wt.double().numpy(), gout[sl].double().numpy()]
        want = orc.deform_sample_depthwise_forward(a[0], a[1], a[2], a[3], **cfg)
        w_gin, w_goff, w_grot, _ = orc.deform_sample_depthwise_backward(a[4], a[0], a[1], a[2], a[3], **cfg)
        assert rel_err(out[sl], want) < 1e-5
        assert rel_err(gin[sl], w_gin) < 1e-4
        assert rel_err(goff[sl], w_goff) < 1e-4
        assert rel_err(grot[sl], w_grot) < 1e-4
    lhs = (gout.double() * out.double()).sum().item()
    via_x = (gin.double() * x.double()).sum().item()
    via_w = (gw.double() * wt.double()).sum().item()
    assert abs(lhs - via_x) < 1e-5 * max(abs(lhs), 1.0)
    assert abs(lhs - via_w) < 1e-5 * max(abs(lhs), 1.0)
    # batch independence: images 10..13 alone give the same rows
    dev = torch.device("cuda:0")
    sl = slice(10, 14)
    with torch.no_grad():
        part = deform_sample_depthwise(x[sl].to(dev), off[sl].to(dev), rot[sl].to(dev), wt.to(dev), cfg["kernel_size"],
                                       cfg["stride"], cfg["padding"], cfg["dilation"], cfg["groups"])
    assert torch.equal(part.cpu(), out[sl])


@pytest.mark.parametrize("switch,case", [("DK_NO_DEFORM_CH", CASES[0]), ("DK_NO_DEFORM_MFMA", CASES[0]),
                                         ("DK_NO_DEFORM_CH_BIG", CASES[7]), ("DK_NO_DEFORM_WINDOW", CASES[13]),
                                         ("DK_NO_DEFORM_WINDOW", CASES[20]), ("DK_NO_DEFORM_WINDOW", CASES[16]),
                                         ("DK_NO_DEFORM_WINDOW", CASES[22]), ("DK_NO_DEFORM_WINDOW", CASES[25]),
                                         ("DK_FORCE_WIN2", CASES[13]),
                                         ("DK_FORCE_WIN2", CASES[20]), ("DK_FORCE_WIN2", CASES[21]),
                                         ("DK_FORCE_WIN2", CASES[9])])
def test_one_plane_kernels_on_a_shape_the_newer_ones_cover(switch_off, switch, case):
    """Without the channel-interleaved kernels (those for small planes and those for large ones) / the
    matrix-core grad filter / the row-window forms, the one-plane kernels serve the shape; and the grad filter with
    a window in rows and columns on shapes that its row-window form takes by default."""
    switch_off(switch)
    inputs, got = _run(case, torch.float32)
    assert_fp32_parity(got, _oracle(inputs, np.float32), _oracle(inputs, np.float64))


def test_generic_kernels_on_a_shape_the_tuned_ones_cover(switch_off):
    """With the tuned deformable kernels switched off the generic ones serve the same shape."""
    switch_off("DK_NO_DEFORM_FAST")
    inputs, got = _run(CASES[0], torch.float32)
    o32, o64 = _oracle(inputs, np.float32), _oracle(inputs, np.float64)
    assert rel_err(got[0], o32[0]) < 1e-5
    for i in range(1, 5):
        assert rel_err(got[i], o64[i]) < 1e-4, NAMES[i]


@pytest.mark.parametrize("case", [CASES[0], CASES[10], CASES[24]])  # one plane per workgroup; tiled planes above 1024 pixels; bands of rows
@pytest.mark.parametrize("poison", [float("inf"), float("nan")])
@pytest.mark.parametrize("where", ["out_grad", "filter"])
def test_non_finite_values_reach_the_input_gradient(case, poison, where):
    """The tuned grad-input kernels add fixed-point integers whose scale comes from max|out_grad| and
    max|filter[c]|; an infinity or a NaN there must not come back as finite numbers (the reference's
    float atomics carry it to the elements it touches; loss scaling only asks whether any gradient
    is non-finite).  out_grad: the whole input gradient is NaN; filter: at least the poisoned
    channel's planes are, and the planes of other channel chunks stay finite."""
    from deformable_kernels.ops.deform_kernel import _lib
    L, P = _lib.lib(), _lib.ptr
    N, C, H, W, k, S, s, p, d, G, rs, os_ = case
    x, wt, rot, off, gout, cfg = make_deform(N, C, H, W, k, S, s, p, d, G, rs, os_, seed=9)
    if where == "out_grad":
        gout[N - 1, C // 2, 3, 4] = poison
    else:
        wt[1, 0, 2, 1] = poison
    dev = torch.device("cuda:0")
    wg, rg, og, gg = [t.to(dev) for t in (wt, rot, off, gout)]
    xs = torch.empty(N, C, H, W, device=dev)
    desc = _lib.conv_desc(xs, wg, cfg["kernel_size"], cfg["stride"], cfg["padding"], cfg["dilation"], G)
    ws, nbytes = _lib.workspace(L.dk_deformable_sample_depthwise_backward_data_workspace(desc), dev)
    gin = torch.zeros_like(xs)
    _lib.check(L.dk_deformable_sample_depthwise_backward_data(
        desc, P(gg), P(og), P(rg), P(wg), P(gin), P(ws), nbytes, torch.cuda.current_stream().cuda_stream), "data")
    torch.cuda.synchronize()
    bad = ~torch.isfinite(gin)
    if where == "out_grad":
        assert bool(bad[N - 1, C // 2].any())   # where the reference's atomics would have put it
    else:
        assert bool(bad[:, 1].any())


# ---- no rotation tensor (DeformKernelConv2d / DeformConv2d: rotation = None) ----------------------

NO_ROTATION_CASES = [
    (2, 16, 14, 14, 3, (3, 3), 2, 1, 1, 1, 0.0, 2.0),    # DeformConv2d: scope == kernel, stride 2
    (1, 9, 56, 56, 3, (3, 3), 1, 1, 1, 1, 0.0, 2.0),     # 56 x 56 planes, the 1024-thread kernels
    (2, 12, 13, 11, 3, (4, 4), 1, 1, 1, 1, 0.0, 2.0),    # DeformKernelConv2d with a scope larger than the kernel
    (2, 6, 8, 8, (2, 3), (4, 5), (1, 2), (0, 1), 1, 3, 0.0, 1.0),  # the general kernels
    (1, 3, 5, 70, 3, (3, 3), 1, 1, 1, 1, 0.0, 1.5),      # wider than the tuned kernels take
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16])
@pytest.mark.parametrize("case", NO_ROTATION_CASES)
def test_without_a_rotation_tensor_equals_the_oracle_with_zero_rotation(case, dtype):
    """rotation = None (a NULL pointer at the C ABI) is the reference's call with a tensor of zeros
    (ops/deform_kernel/modules/filter_sample_depthwise.py:163-168), without that tensor."""
    from deformable_kernels.ops.deform_kernel.functions import deform_sample_depthwise
    N, C, H, W, k, S, s, p, d, G, rs, os_ = case
    x, wt, rot, off, gout, cfg = make_deform(N, C, H, W, k, S, s, p, d, G, 0.0, os_, seed=7, dtype=dtype)
    assert float(rot.abs().max()) == 0.0
    dev = torch.device("cuda:0")
    xg, og, wg = [t.to(dev).requires_grad_() for t in (x, off, wt)]
    out = deform_sample_depthwise(xg, og, None, wg, cfg["kernel_size"], cfg["stride"], cfg["padding"],
                                  cfg["dilation"], cfg["groups"])
    out.backward(gout.to(dev))
    torch.cuda.synchronize()
    got = [t.detach().cpu() for t in (out, xg.grad, og.grad, wg.grad)]
    o64 = _oracle((x, wt, rot, off, gout, cfg), np.float64)
    want = [o64[i] for i in (0, 1, 2, 4)]
    tol = {torch.float32: (1e-5, 1e-5, 1e-4, 1e-4), torch.float64: (1e-11,) * 4, torch.bfloat16: (1e-2,) * 4}[dtype]
    for name, a, b, t in zip(("forward", "grad input", "grad offset", "grad filter"), got, want, tol):
        if name == "grad offset" and dtype == torch.float32:
            o32 = _oracle((x, wt, rot, off, gout, cfg), np.float32)[2].astype(np.float64)
            err = np.minimum(np.abs(a.double().numpy() - b), np.abs(a.double().numpy() - o32))
            assert err.max() / np.abs(b).max() < t, name
        else:
            assert rel_err(a.float() if dtype == torch.bfloat16 else a, b) < t, name


def test_deform_conv_module_runs_without_a_rotation_tensor_and_is_a_depthwise_deformable_convolution():
    """DeformConv2d (scope = kernel, rotation = None, reference modules/deform_conv.py:15-42): with
    zero image-space offsets it is the plain depthwise convolution with its own weights."""
    from deformable_kernels.modules import DeformConv2d
    dev = torch.device("cuda:0")
    torch.manual_seed(11)
    m = DeformConv2d(12, 12, kernel_size=3, stride=1, padding=1, groups=12).to(dev)
    with torch.no_grad():                                # the module marks offset_conv for zero initialisation (:262)
        m.offset_conv.weight.zero_()
        m.offset_conv.bias.zero_()
    x = torch.randn(2, 12, 10, 9, device=dev, requires_grad=True)
    out = m(x)
    want = torch.nn.functional.conv2d(x.detach().double(), m.inner_conv.weight.detach().double(), padding=1, groups=12)
    assert rel_err(out.detach().cpu(), want.cpu()) < 1e-5
    out.sum().backward()
    assert x.grad is not None and m.inner_conv.weight.grad is not None and m.offset_conv.weight.grad is not None


@pytest.mark.parametrize("case", [CASES[0], CASES[8], CASES[13]])  # one kernel (small planes, several chunks); 56 x 56: the two kernels in turn
def test_both_coordinate_gradients_from_one_call_equal_the_separate_entry_points(case):
    """dk_deformable_sample_depthwise_backward_offset_rotation forms the same sums in the same order as
    the two separate entry points, whether it runs as one kernel or as the two in turn: equal bits."""
    from deformable_kernels.ops.deform_kernel import _lib
    N, C, H, W, k, S, s, p, d, G, rs, os_ = case
    x, wt, rot, off, gout, cfg = make_deform(N, C, H, W, k, S, s, p, d, G, rs, os_, seed=3, dtype=torch.float32)
    dev = torch.device("cuda:0")
    xg, wg, rg, og, gg = [t.to(dev) for t in (x, wt, rot, off, gout)]
    L, P = _lib.lib(), _lib.ptr
    desc = _lib.conv_desc(xg, wg, cfg["kernel_size"], cfg["stride"], cfg["padding"], cfg["dilation"], G)
    st = _lib.stream_ptr(xg)
    goff, grot, goff2, grot2 = [torch.empty_like(t) for t in (og, rg, og, rg)]
    ws, n = _lib.workspace(L.dk_deformable_sample_depthwise_backward_offset_workspace(desc), dev)
    _lib.check(L.dk_deformable_sample_depthwise_backward_offset(desc, P(gg), P(xg), P(og), P(rg), P(wg), P(goff), P(ws), n, st), "offset")
    ws, n = _lib.workspace(L.dk_deformable_sample_depthwise_backward_rotation_workspace(desc), dev)
    _lib.check(L.dk_deformable_sample_depthwise_backward_rotation(desc, P(gg), P(xg), P(og), P(rg), P(wg), P(grot), P(ws), n, st), "rotation")
    ws, n = _lib.workspace(L.dk_deformable_sample_depthwise_backward_offset_rotation_workspace(desc), dev)
    _lib.check(L.dk_deformable_sample_depthwise_backward_offset_rotation(
        desc, P(gg), P(xg), P(og), P(rg), P(wg), P(goff2), P(grot2), P(ws), n, st), "both")
    assert L.dk_deformable_sample_depthwise_backward_offset_rotation(
        desc, P(gg), P(xg), P(og), P(rg), P(wg), P(goff2), P(grot2), P(ws), max(n - 1, 0), st) == (-5 if n else 0)  # DK_ERR_WORKSPACE
    torch.cuda.synchronize()
    assert torch.equal(goff, goff2) and torch.equal(grot, grot2)
