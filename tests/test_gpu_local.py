"""GPU parity of the local deformable-kernel operator (forward, grad-input,
grad-rotation, grad-filter) against the CPU oracle, through the Python
Functions and therefore through the C ABI of libdk_hip.so.

Tolerances (relative to the largest magnitude of the expected tensor):
  fp32: forward and grad-input 1e-5 against the fp32 oracle; grad-rotation and
        grad-filter 1e-4 against the fp64 oracle (summation order differs);
  fp64: 1e-11 everywhere;
  fp16 / bf16: 1e-2 against the fp32 oracle evaluated on the rounded inputs.
"""
import numpy as np
import pytest
import torch

from _cases import clipped_rotation, elem_err, make_local, rel_err
from oracle import dk_oracle as orc

pytestmark = pytest.mark.gpu


def _lib_switches(*names):
    from deformable_kernels.ops.deform_kernel import _lib
    return _lib.test_switches(*names)

# N, C, H, W, k, S, stride, pad, dil, groups, rot_std
TUNED = [
    (2, 32, 28, 28, 3, (4, 4), 1, 1, 1, 1, 0.5),    # benchmark configuration 1
    (3, 20, 17, 23, 3, (4, 4), 1, 1, 1, 1, 1.0),    # ragged sizes, partial tiles
    (2, 24, 19, 19, 3, (4, 4), 2, 1, 1, 1, 1.0),    # stride 2
    (2, 12, 15, 14, 3, (4, 4), 1, 2, 2, 3, 1.0),    # dilation 2, rotation groups 3
    (2, 16, 13, 13, 3, (3, 3), 1, 1, 1, 1, 1.0),    # scope == kernel
    (1, 16, 13, 12, 3, (5, 5), 1, 0, 1, 2, 1.5),    # scope 5, no padding
    (1, 200, 9, 9, 3, (4, 4), 1, 1, 1, 1, 2.0),     # many channels, many samples outside the scope
    (3, 40, 21, 17, 3, (4, 4), 1, 1, 1, 2, 1.0),    # same-width geometry, 2 groups, 20 channels per group (1.25 MFMA blocks)
    (1, 272, 12, 12, 3, (3, 3), 1, 1, 1, 1, 1.0),   # more than 256 channels: two channel splits of the matrix-core grad filter
    (2, 10, 16, 18, 3, (4, 4), 2, 0, 1, 1, 1.0),    # stride 2 without padding, even sizes (tap parity of grad input)
    (2, 8, 70, 40, 3, (4, 4), 1, 1, 1, 1, 0.7),     # 2800-pixel planes: many tiles per image, partial last tile
    (1, 600, 40, 64, 3, (5, 5), 1, 1, 1, 1, 1.0),   # 600 channels x 36-block tables: more than one block's LDS, scope 5
    (2, 12, 15, 16, 3, (4, 4), 2, 1, 1, 2, 1.0),    # stride 2, padding 1, even width: pair-load kernels; odd height, 2 groups
    (1, 20, 40, 44, 3, (3, 3), 2, 1, 1, 1, 0.8),    # the same on 440-pixel output planes (two tiles), scope 3
    (4, 64, 28, 28, 3, (4, 4), 1, 1, 1, 1, 1.0),    # grad rotation in 4 channel splits, summed by the few-parts reduction
    (1, 5, 5, 64, 3, (4, 4), 1, 1, 1, 1, 1.0),      # planes 64 / 112 / 130 columns wide: the first element of the plane
    (1, 3, 4, 112, 3, (3, 3), 1, 1, 1, 1, 1.0),     # sits in the second or third 64-element chunk of the first tile's
    (1, 3, 3, 130, 3, (4, 4), 1, 1, 1, 1, 1.0),     # staged range, behind the (out-of-range) top halo row
    (1, 4, 6, 64, 3, (4, 4), 2, 1, 1, 1, 1.0),      # the same for the stride-2 geometry
    (1, 3, 5, 130, 3, (5, 5), 2, 1, 1, 1, 1.0),
    (2, 20, 14, 14, 3, (7, 7), 1, 1, 1, 1, 2.0),    # scope 7: four 16-cell slices of the matrix-core grad filter
    (2, 12, 15, 16, 3, (7, 7), 2, 1, 1, 2, 2.0),    # scope 7, stride 2: grad filter on the generic kernel
    (1, 24, 40, 44, 3, (5, 5), 2, 1, 1, 1, 1.5),    # scope 5, stride 2: two slices of the stride-2 matrix-core grad filter
    (1, 24, 41, 43, 3, (5, 5), 2, 1, 1, 1, 1.5),    # the same with an odd width: dense grad filter with two cells per lane
    (2, 80, 12, 18, 3, (4, 4), 1, 1, 1, 2, 1.0),    # same width, even: 40 channels per group (1.25 units of the 16-bit matrix-core forward), 2 groups
]
GENERIC = [
    (2, 6, 9, 8, (5, 3), (7, 4), (1, 2), (2, 0), 1, 3, 0.7),
    (1, 4, 10, 11, 3, (5, 3), 1, 2, 2, 1, 1.5),
    (2, 5, 6, 5, 1, (2, 2), 1, 0, 1, 1, 0.6),
    (1, 4, 8, 8, 2, (4, 4), 2, 0, 1, 2, 0.5),
]


def _run(case, dtype, seed=0):
    from deformable_kernels.ops.deform_kernel.functions import sample_depthwise
    N, C, H, W, k, S, s, p, d, G, rs = case
    x, wt, rot, gout, cfg = make_local(N, C, H, W, k, S, s, p, d, G, rs, seed=seed, dtype=dtype)
    dev = torch.device("cuda:0")
    xg, rg, wg = [t.to(dev).requires_grad_() for t in (x, rot, wt)]
    out = sample_depthwise(xg, rg, wg, cfg["kernel_size"], cfg["stride"], cfg["padding"], cfg["dilation"],
                           cfg["groups"])
    out.backward(gout.to(dev))
    torch.cuda.synchronize()
    got = [t.detach().cpu() for t in (out, xg.grad, rg.grad, wg.grad)]
    return (x, wt, rot, gout, cfg), got


def _oracle(inputs, np_dtype):
    x, wt, rot, gout, cfg = inputs
    a = [t.to(torch.float64).numpy().astype(np_dtype) for t in (x, rot, wt, gout)]
    out = orc.sample_depthwise_forward(a[0], a[1], a[2], **cfg)
    gin, grot, gw = orc.sample_depthwise_backward(a[3], a[0], a[1], a[2], **cfg)
    return out, gin, grot, gw


@pytest.mark.parametrize("case", TUNED + GENERIC)
def test_fp32_matches_oracle(case):
    inputs, got = _run(case, torch.float32)
    o32 = _oracle(inputs, np.float32)
    o64 = _oracle(inputs, np.float64)
    assert got[0].dtype == torch.float32
    assert rel_err(got[0], o32[0]) < 1e-5, "forward"
    assert rel_err(got[1], o32[1]) < 1e-5, "grad input"
    assert rel_err(got[2], o64[2]) < 1e-4, "grad rotation"
    assert rel_err(got[3], o64[3]) < 1e-4, "grad filter"
    # element by element: every element within the tolerance of its OWN magnitude, with an absolute floor of
    # tolerance * eps * (largest magnitude) for the elements that are small by cancellation (measured over these
    # cases: 2e-6, 1.7e-6, 1.7e-5 and 4.2e-5 with the eps below)
    assert elem_err(got[0], o32[0], 0.05) < 1e-5, "forward, element-wise"
    assert elem_err(got[1], o32[1], 0.05) < 1e-5, "grad input, element-wise"
    assert elem_err(got[2], o64[2], 0.01) < 1e-4, "grad rotation, element-wise"
    assert elem_err(got[3], o64[3], 0.1) < 1e-4, "grad filter, element-wise"


@pytest.mark.parametrize("case", [c for c in TUNED if c[6] == 1 and c[7] == 1 and c[8] == 1 and c[5] in ((4, 4), (3, 3))])
def test_matrix_core_forward_and_grad_input_on_every_same_width_shape(case, switch_off):
    """The dispatch takes the matrix-core forward / grad input only on large planes with many channels,
    where it is the faster kernel (the full-size configuration 2 test runs it); forced, it must serve
    every same-width shape: ragged tiles, few channels, planes smaller than a tile, several groups."""
    switch_off("DK_FORCE_GATHER_MFMA")
    inputs, got = _run(case, torch.float32, seed=6)
    o32 = _oracle(inputs, np.float32)
    assert rel_err(got[0], o32[0]) < 1e-5, "forward"
    assert rel_err(got[1], o32[1]) < 1e-5, "grad input"


@pytest.mark.parametrize("dtype,tol", [(torch.float16, 1e-3), (torch.bfloat16, 5e-3)])
@pytest.mark.parametrize("case", [c for c in TUNED if c[6] == 1 and c[7] == 1 and c[8] == 1 and c[5] in ((4, 4), (3, 3))])
def test_matrix_core_forward_and_grad_input_on_16_bit_tensors(case, dtype, tol, switch_off):
    """16-bit tensors take the same kernel with two elements per slot of its staged tiles and two channel
    blocks per unit (rows of an even number of elements; other widths stay on the row kernels, which this
    test then runs).  The products carry fp32 sums, so the error is the result's own rounding to the type."""
    switch_off("DK_FORCE_GATHER_MFMA")
    inputs, got = _run(case, dtype, seed=7)
    want = _oracle(inputs, np.float32)  # the inputs are already rounded to `dtype`
    assert rel_err(got[0].float(), want[0]) < tol, "forward"
    assert rel_err(got[1].float(), want[1]) < tol, "grad input"


SAME_WIDTH = [c for c in TUNED if c[6] == 1 and c[7] == 1 and c[8] == 1 and c[5] in ((4, 4), (3, 3))] + [
    (2, 144, 56, 56, 3, (4, 4), 1, 1, 1, 1, 1.0),  # the headline layer's geometry: three whole rounds of tiles per wave and a shared remainder
    (1, 272, 12, 12, 3, (3, 3), 1, 1, 1, 1, 1.0),  # 8.5 blocks of 32 channels; waves that change tile after a single block
    (2, 70, 9, 31, 3, (4, 4), 1, (2, 1), (2, 1), 2, 1.0),  # dilated rows (pad_h = dil_h = 2), 35 channels per group, a tile spans a row's end
]


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.float16, 1e-3), (torch.bfloat16, 5e-3)])
@pytest.mark.parametrize("case", SAME_WIDTH)
def test_forward_and_grad_input_with_the_pixels_on_the_matrix_lanes(case, dtype, tol, switch_off):
    """dk_local_lanes.hip: channels on the rows of the 32 x 32 matrix instruction, pixels on its columns, source
    rows loaded straight into the registers the multiply-adds read, with hand-counted waits.  The dispatch takes
    it on large planes with many channels (the full-size configuration 2 test runs it there); forced, it must
    serve every same-width shape: partial tiles, channel blocks that end beyond the group's last channel, several
    groups, tiles that wrap around a row's end, one block per tile."""
    switch_off("DK_FORCE_PIXEL_LANES")
    inputs, got = _run(case, dtype, seed=5)
    want = _oracle(inputs, np.float32)  # 16-bit inputs are already rounded to the type
    assert rel_err(got[0].float(), want[0]) < tol, "forward"
    assert rel_err(got[1].float(), want[1]) < tol, "grad input"


@pytest.mark.parametrize("case", [
    (2, 37, 28, 28, 3, (4, 4), 1, 1, 1, 1, 1.0),   # odd channel count: the last pair's second channel is a dummy
    (1, 74, 12, 18, 3, (5, 5), 1, 1, 1, 2, 1.5),   # 37 channels per group, two groups, scope 5
    (1, 73, 20, 22, 3, (3, 3), 1, 1, 1, 1, 1.0),   # passes of 36, 36 and 1 channels
    (4, 64, 28, 28, 3, (4, 4), 1, 1, 1, 1, 1.0),   # four channel splits of 16 channels, partial sums
])
def test_grad_rotation_by_channel_pairs_on_bfloat16_tensors(case):
    """bfloat16 tensors with at least 16 channels per group take grad rotation two channels per step, the
    products rounded to bfloat16 and summed in fp32 by dot-product instructions: the result stays within the
    1e-2 the 16-bit types are held to (about 6e-3 of the largest element at worst, of which 4e-3 is the
    result's own rounding)."""
    inputs, got = _run(case, torch.bfloat16, seed=11)
    want = _oracle(inputs, np.float32)  # the inputs are already rounded to bfloat16
    assert got[2].dtype == torch.bfloat16
    assert rel_err(got[2].float(), want[2]) < 1e-2, "grad rotation"


@pytest.mark.parametrize("case", TUNED[:4] + GENERIC[:2])
def test_fp64_matches_oracle(case):
    inputs, got = _run(case, torch.float64)
    want = _oracle(inputs, np.float64)
    for g, w, name in zip(got, want, ("forward", "grad input", "grad rotation", "grad filter")):
        assert g.dtype == torch.float64
        assert rel_err(g, w) < 1e-11, name


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
# the matrix-core grad filter multiplies 16-bit inputs with bfloat16 matrix instructions (hat products and
# x * gout products rounded to bfloat16, fp32 sums): same-width, wide-plane, stride-2, 5 x 5 and 7 x 7 geometries
@pytest.mark.parametrize("case", TUNED[:5] + [TUNED[7], TUNED[10], TUNED[15], TUNED[18], TUNED[20], TUNED[22]] + GENERIC[:2])
def test_half_precisions_match_fp32_oracle(case, dtype):
    inputs, got = _run(case, dtype)
    want = _oracle(inputs, np.float32)  # the inputs are already rounded to `dtype`
    for g, w, name in zip(got, want, ("forward", "grad input", "grad rotation", "grad filter")):
        assert g.dtype == dtype
        assert rel_err(g.float(), w) < 1e-2, name


def test_bf16_group_of_one_channel_keeps_fp32_matrix_instructions():
    """Nine results from one channel: their largest element can be small against the rounding noise of
    bfloat16 products (1.1e-2 was seen on this case), so groups of fewer than 16 channels multiply in fp32."""
    inputs, got = _run((1, 1, 33, 14, 3, (3, 3), 1, 1, 1, 1, 0.5), torch.bfloat16)
    want = _oracle(inputs, np.float32)
    assert rel_err(got[3].float(), want[3]) < 4e-3   # the result's own rounding to bfloat16: 2e-3


@pytest.mark.parametrize("clip", [(-0.4, 0.3), 'scope'])
@pytest.mark.parametrize("case", [TUNED[0], TUNED[2], TUNED[3], TUNED[5], GENERIC[0], GENERIC[1]])
def test_rotation_clip_inside_the_operator(case, clip):
    # the operator clamping the offsets itself == the reference's sequence (clamp the tensor,
    # then the plain operator); the rotation gradient is zero where the clamp was active
    from deformable_kernels.ops.deform_kernel.functions import sample_depthwise
    N, C, H, W, k, S, s, p, d, G, rs = case
    x, wt, rot, gout, cfg = make_local(N, C, H, W, k, S, s, p, d, G, 1.5 * rs, seed=5)
    dev = torch.device("cuda:0")
    xg, rg, wg = [t.to(dev).requires_grad_() for t in (x, rot, wt)]
    out = sample_depthwise(xg, rg, wg, cfg["kernel_size"], cfg["stride"], cfg["padding"], cfg["dilation"],
                           cfg["groups"], clip)
    out.backward(gout.to(dev))
    got = [t.detach().cpu() for t in (out, xg.grad, rg.grad, wg.grad)]
    rot_c, open_ = clipped_rotation(rot, clip, cfg["kernel_size"], S, G)
    assert 0.02 < 1.0 - open_.float().mean().item() < 0.9  # the clamp is active on a real share of the offsets
    o32 = _oracle((x, wt, rot_c, gout, cfg), np.float32)
    o64 = _oracle((x, wt, rot_c, gout, cfg), np.float64)
    assert rel_err(got[0], o32[0]) < 1e-5, "forward"
    assert rel_err(got[1], o32[1]) < 1e-5, "grad input"
    assert rel_err(got[2], torch.as_tensor(o64[2]) * open_) < 1e-4, "grad rotation"
    assert rel_err(got[3], o64[3]) < 1e-4, "grad filter"
    assert (got[2][~open_] == 0).all()


def test_taps_outside_the_scope_and_nan_free_borders():
    # rotations that push every tap outside (-1, S): all four results are exact zeros
    from deformable_kernels.ops.deform_kernel.functions import sample_depthwise
    x, wt, rot, gout, cfg = make_local(2, 8, 10, 10, 3, (4, 4), 1, 1, 1, 1, 0.0, seed=3)
    dev = torch.device("cuda:0")
    for shift in (-10.0, 10.0, -3.5, 4.0):
        xg, rg, wg = [t.to(dev).requires_grad_() for t in (x, rot + shift, wt)]
        out = sample_depthwise(xg, rg, wg, (3, 3), (1, 1), (1, 1), (1, 1), 1)
        out.backward(gout.to(dev))
        for t in (out, xg.grad, rg.grad, wg.grad):
            assert torch.count_nonzero(t).item() == 0


def test_non_contiguous_inputs_and_needs_input_grad_gating():
    from deformable_kernels.ops.deform_kernel.functions import sample_depthwise
    x, wt, rot, gout, cfg = make_local(2, 8, 12, 10, 3, (4, 4), 1, 1, 1, 1, 0.8, seed=4)
    dev = torch.device("cuda:0")
    xt = x.transpose(2, 3).contiguous().transpose(2, 3).to(dev)  # same values, strided layout
    assert not xt.is_contiguous()
    rg = rot.to(dev).requires_grad_()
    out = sample_depthwise(xt, rg, wt.to(dev), (3, 3), (1, 1), (1, 1), (1, 1), 1)
    out.backward(gout.to(dev))
    want = orc.sample_depthwise_forward(x.numpy(), rot.numpy(), wt.numpy(), **cfg)
    _, grot, _ = orc.sample_depthwise_backward(gout.double().numpy(), x.double().numpy(), rot.double().numpy(),
                                               wt.double().numpy(), **cfg)
    assert rel_err(out.detach().cpu(), want) < 1e-5
    assert rel_err(rg.grad.cpu(), grot) < 1e-4


def test_runs_on_a_side_stream_and_empty_batch():
    from deformable_kernels.ops.deform_kernel.functions import sample_depthwise
    x, wt, rot, gout, cfg = make_local(2, 8, 12, 10, 3, (4, 4), 1, 1, 1, 1, 0.8, seed=5)
    dev = torch.device("cuda:0")
    xg, rg, wg = x.to(dev), rot.to(dev), wt.to(dev)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        out = sample_depthwise(xg, rg, wg, (3, 3), (1, 1), (1, 1), (1, 1), 1)
    side.synchronize()
    want = orc.sample_depthwise_forward(x.numpy(), rot.numpy(), wt.numpy(), **cfg)
    assert rel_err(out.cpu(), want) < 1e-5
    # an empty batch is rejected by the output-size rule, as in the reference
    # (functions/filter_sample_depthwise.py:98-101 tests every output extent, batch included)
    with pytest.raises(ValueError):
        sample_depthwise(xg[:0], rg[:0], wg, (3, 3), (1, 1), (1, 1), (1, 1), 1)


def test_headline_shape_properties_at_full_size():
    """benchmark configuration 2 (N=64, C=144, 56x56, k=3, scope 4x4, fp32) at full size: the oracle is
    run on a slice of images; the rest is covered by size-independent properties -- batch
    independence, linearity in the input, and <gout, F(x)> = <grad_input, x>."""
    from deformable_kernels.ops.deform_kernel.functions import sample_depthwise
    N, C = 64, 144
    x, wt, rot, gout, cfg = make_local(N, C, 56, 56, 3, (4, 4), 1, 1, 1, 1, 1.0, seed=0)
    dev = torch.device("cuda:0")
    xg, rg, wg = [t.to(dev).requires_grad_() for t in (x, rot, wt)]
    args = ((3, 3), (1, 1), (1, 1), (1, 1), 1)
    out = sample_depthwise(xg, rg, wg, *args)
    out.backward(gout.to(dev))
    torch.cuda.synchronize()
    # oracle on images {0, 37, 63}
    for n in (0, 37, 63):
        sl = slice(n, n + 1)
        want = orc.sample_depthwise_forward(x[sl].numpy(), rot[sl].numpy(), wt.numpy(), **cfg)
        gin, grot, _ = orc.sample_depthwise_backward(
            gout[sl].double().numpy(), x[sl].double().numpy(), rot[sl].double().numpy(), wt.double().numpy(), **cfg)
        assert rel_err(out[sl].detach().cpu(), want) < 1e-5
        assert rel_err(xg.grad[sl].cpu(), gin) < 1e-5
        assert rel_err(rg.grad[sl].cpu(), grot) < 1e-4
    # grad filter: full batch against the fp64 oracle (a few seconds of CPU)
    _, _, gw = orc.sample_depthwise_backward(gout.double().numpy(), x.double().numpy(), rot.double().numpy(),
                                             wt.double().numpy(), **cfg)
    assert rel_err(wg.grad.cpu(), gw) < 1e-4
    # The float32 filter gradient multiplies bfloat16 PAIRS of its operands (three products, fp32 sums) instead
    # of float32 matrix instructions.  Its error is pinned here, well inside the tolerance, so that a drift
    # shows: measured 5.1e-6 of the largest element (element-wise with a 10 % floor: 3.3e-5), against 2.4e-7
    # (1.4e-6) for the float32 instructions, which the test switch DK_NO_FILTER_SPLIT brings back.
    assert rel_err(wg.grad.cpu(), gw) < 1.5e-5, "bfloat16-pair filter gradient drifted"
    assert elem_err(wg.grad.cpu(), gw, 0.1) < 1e-4
    with _lib_switches("DK_NO_FILTER_SPLIT"):
        xs, rs, ws_ = [t.detach().requires_grad_() for t in (xg, rg, wg)]
        gw32, = torch.autograd.grad(sample_depthwise(xs, rs, ws_, *args), ws_, gout.to(dev))
    assert rel_err(gw32.cpu(), gw) < 1e-6, "float32 matrix instructions"
    assert elem_err(gw32.cpu(), gw, 0.1) < 5e-6
    del xs, rs, ws_, gw32
    # linearity in the input
    with torch.no_grad():
        x2 = torch.randn_like(xg)
        lhs = sample_depthwise(2 * xg + 3 * x2, rg, wg, *args)
        rhs = 2 * out + 3 * sample_depthwise(x2, rg, wg, *args)
        assert rel_err(lhs.cpu(), rhs.cpu()) < 1e-5
        # adjoint identity in fp64 accumulation
        a = (gout.to(dev).double() * out.double()).sum().item()
        b = (xg.grad.double() * xg.double()).sum().item()
        assert abs(a - b) < 1e-6 * max(abs(a), 1.0)


@pytest.mark.parametrize("switch", ["DK_NO_MFMA", "DK_NO_ROWS", "DK_NO_GATHER_MFMA", "DK_NO_FILTER_SPLIT", "DK_NO_PIXEL_LANES"])
def test_more_general_kernels_on_a_same_width_shape(switch, switch_off):
    """The dispatch prefers the most specialised kernel; the library's test switches make it take
    the next more general family for the same shape (dense grad filter instead of the
    matrix-core one; per-tap loads instead of the row kernels; the row kernels instead of the
    matrix-core forward / grad input; float32 matrix instructions instead of bfloat16 pairs in the
    grad filter), which must give the same results."""
    switch_off(switch)
    case = (2, 40, 20, 24, 3, (4, 4), 1, 1, 1, 2, 1.0)
    inputs, got = _run(case, torch.float32)
    o32, o64 = _oracle(inputs, np.float32), _oracle(inputs, np.float64)
    assert rel_err(got[0], o32[0]) < 1e-5
    assert rel_err(got[1], o32[1]) < 1e-5
    assert rel_err(got[2], o64[2]) < 1e-4
    assert rel_err(got[3], o64[3]) < 1e-4


@pytest.mark.parametrize("switch", ["DK_NO_MFMA_S2", "DK_NO_S2_QUADS"])
def test_more_general_kernels_on_a_stride_2_shape(switch, switch_off):
    """Stride 2, padding 1, even width: the dense pair-load grad filter instead of the matrix-core one,
    the gather over input pixels instead of the one over 2 x 2 input quads."""
    switch_off(switch)
    case = (2, 24, 22, 20, 3, (4, 4), 2, 1, 1, 2, 1.0)
    inputs, got = _run(case, torch.float32)
    o32, o64 = _oracle(inputs, np.float32), _oracle(inputs, np.float64)
    assert rel_err(got[0], o32[0]) < 1e-5
    assert rel_err(got[1], o32[1]) < 1e-5
    assert rel_err(got[2], o64[2]) < 1e-4
    assert rel_err(got[3], o64[3]) < 1e-4


@pytest.mark.parametrize("deform", [False, True])
@pytest.mark.parametrize("shape", [(8, 4), (1200, 4)])  # channels, scope: both reduction kernels
def test_c_abi_filter_gradient_of_an_empty_batch_is_written_as_zeros(deform, shape):
    """batch == 0 through the raw C ABI (the Python Functions refuse empty batches as the reference's
    output-size rule does): the filter gradient is the one result that is not empty, and it is zeros."""
    from deformable_kernels.ops.deform_kernel import _lib
    L, P = _lib.lib(), _lib.ptr
    dev = torch.device("cuda:0")
    C, S = shape
    x = torch.empty(0, C, 12, 12, device=dev)
    wt = torch.empty(C, 1, S, S, device=dev)
    desc = _lib.conv_desc(x, wt, (3, 3), (1, 1), (1, 1), (1, 1), 1)
    gw = torch.full_like(wt, float("nan"))
    s = torch.cuda.current_stream().cuda_stream
    one = P(gw)  # never read: the batch is empty
    if deform:
        need = L.dk_deformable_sample_depthwise_backward_filter_workspace(desc)
        ws, nbytes = _lib.workspace(max(need, 16), dev)
        rc = L.dk_deformable_sample_depthwise_backward_filter(desc, one, one, one, one, P(gw), P(ws), nbytes, s)
    else:
        need = L.dk_sample_depthwise_backward_filter_workspace(desc)
        ws, nbytes = _lib.workspace(max(need, 16), dev)
        rc = L.dk_sample_depthwise_backward_filter(desc, one, one, one, P(gw), P(ws), nbytes, s)
    torch.cuda.synchronize()
    assert rc == 0
    assert torch.count_nonzero(gw).item() == 0 and torch.isfinite(gw).all()
