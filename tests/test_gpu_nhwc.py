"""The local deformable-kernel operator on channels-last tensors against the CPU oracle (which works on
the logical NCHW tensors: the layout changes where an element is stored, not its value), through the
Python Function and the C ABI's layout field.  Tolerances as for the planar operator: fp32 forward and
grad input 1e-5 (fp32 oracle), grad rotation and grad filter 1e-4 (fp64 oracle); fp64 1e-11; fp16 /
bf16 1e-2 against the fp32 oracle on the rounded inputs."""
import numpy as np
import pytest
import torch

from _cases import clipped_rotation, make_local, rel_err
from oracle import dk_oracle as orc

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")

# N, C, H, W, k, S, stride, pad, dil, groups, rot_std
CASES = [
    (2, 32, 28, 28, 3, (4, 4), 1, 1, 1, 1, 0.5),    # benchmark configuration 1: four channels per lane
    (3, 20, 17, 23, 3, (4, 4), 1, 1, 1, 1, 1.0),    # ragged sizes
    (2, 24, 19, 19, 3, (4, 4), 2, 1, 1, 1, 1.0),    # stride 2: grad input skips the taps off the stride's grid
    (2, 12, 15, 14, 3, (4, 4), 1, 2, 2, 3, 1.0),    # dilation 2, rotation groups 3: one channel per lane
    (2, 18, 13, 13, 3, (3, 3), 1, 1, 1, 1, 1.0),    # scope == kernel, channels not a multiple of 4
    (1, 16, 13, 12, 3, (5, 5), 1, 0, 1, 2, 1.5),    # scope 5, no padding, two groups
    (1, 300, 9, 9, 3, (4, 4), 1, 1, 1, 1, 2.0),     # more channels than a chunk (256): two channel chunks
    (2, 6, 9, 8, (5, 3), (7, 4), (1, 2), (2, 0), 1, 3, 0.7),   # general taps and scope: sums in LDS columns
    (1, 4, 8, 8, 2, (4, 4), 2, 0, 1, 2, 0.5),
    (2, 8, 40, 36, 3, (4, 4), 1, 1, 1, 1, 0.7),     # 2880 pixels: several partial sums of the grad filter
    (1, 36, 56, 56, 3, (4, 4), 1, 1, 1, 1, 1.0),    # a plane of the headline's size: six staged elements per lane
    (2, 20, 13, 13, 3, (3, 3), 1, 1, 1, 1, 1.0),    # scope == kernel on the staged kernels
    (1, 40, 13, 12, 3, (5, 5), 1, 1, 1, 1, 1.5),    # scope 5: two slices of sixteen cells
    (2, 16, 15, 14, 3, (4, 4), 1, 2, 2, 1, 1.0),    # dilation 2 with one group: the matrix-core kernels' general taps
    (1, 32, 12, 11, 3, (3, 3), 2, 0, 1, 1, 1.0),    # stride 2 without padding, scope == kernel
    (2, 128, 7, 7, 3, (4, 4), 1, 1, 1, 1, 1.0),     # few pixels, many channels: the grad rotation's channel steps split over two workgroups
    (1, 200, 6, 5, 3, (3, 3), 1, 1, 1, 1, 1.0),     # seven steps of 32 channels over three splits (3, 3, 1), the last step partial
    (1, 960, 7, 7, 3, (4, 4), 1, 1, 1, 1, 1.0),     # MobileNetV2's last stage: filter tables of more than 64 KB of LDS in the matrix-core kernels
]


def _run(case, dtype, seed=0, clip=None):
    from deformable_kernels.ops.deform_kernel.functions import sample_depthwise
    N, C, H, W, k, S, s, p, d, G, rs = case
    x, wt, rot, gout, cfg = make_local(N, C, H, W, k, S, s, p, d, G, rs, seed=seed, dtype=dtype)
    cl = torch.channels_last
    xg = x.to(DEV).contiguous(memory_format=cl).requires_grad_()
    rg = rot.to(DEV).contiguous(memory_format=cl).requires_grad_()
    wg = wt.to(DEV).requires_grad_()
    out = sample_depthwise(xg, rg, wg, cfg["kernel_size"], cfg["stride"], cfg["padding"], cfg["dilation"],
                           cfg["groups"], clip)
    assert out.is_contiguous(memory_format=cl)
    out.backward(gout.to(DEV).contiguous(memory_format=cl))
    torch.cuda.synchronize()
    if C > 1 and H * W > 1:
        assert xg.grad.is_contiguous(memory_format=cl) and rg.grad.is_contiguous(memory_format=cl)
    return (x, wt, rot, gout, cfg), [t.detach().cpu().contiguous() for t in (out, xg.grad, rg.grad, wg.grad)]


def _oracle(inputs, np_dtype):
    x, wt, rot, gout, cfg = inputs
    a = [t.to(torch.float64).numpy().astype(np_dtype) for t in (x, rot, wt, gout)]
    out = orc.sample_depthwise_forward(a[0], a[1], a[2], **cfg)
    return (out,) + tuple(orc.sample_depthwise_backward(a[3], a[0], a[1], a[2], **cfg))


@pytest.mark.parametrize("case", CASES)
def test_fp32_matches_oracle(case):
    inputs, got = _run(case, torch.float32)
    o32, o64 = _oracle(inputs, np.float32), _oracle(inputs, np.float64)
    assert rel_err(got[0], o32[0]) < 1e-5
    assert rel_err(got[1], o32[1]) < 1e-5
    assert rel_err(got[2], o64[2]) < 1e-4
    assert rel_err(got[3], o64[3]) < 1e-4


@pytest.mark.parametrize("case", CASES[:3] + CASES[4:7] + CASES[9:])
def test_fp32_without_the_matrix_core_kernels(case, switch_off):
    """Grad filter and grad rotation of one-group layers run on the matrix cores; with that family
    switched off the channel-per-thread and wave-per-pixel kernels serve the same shapes."""
    switch_off("DK_NO_NHWC_MFMA")
    inputs, got = _run(case, torch.float32, seed=2)
    o32, o64 = _oracle(inputs, np.float32), _oracle(inputs, np.float64)
    assert rel_err(got[0], o32[0]) < 1e-5
    assert rel_err(got[1], o32[1]) < 1e-5
    assert rel_err(got[2], o64[2]) < 1e-4
    assert rel_err(got[3], o64[3]) < 1e-4


@pytest.mark.parametrize("case", CASES[:2] + [CASES[6]] + CASES[9:])
def test_fp32_without_the_staged_kernels(case, switch_off):
    """Stride-1 layers of one group with a multiple of 4 channels take the kernels that stage planar tiles
    in LDS; switched off, the matrix-core kernels that read the channels-last rows directly serve them."""
    switch_off("DK_NO_NHWC_STAGED")
    inputs, got = _run(case, torch.float32, seed=4)
    o32, o64 = _oracle(inputs, np.float32), _oracle(inputs, np.float64)
    assert rel_err(got[0], o32[0]) < 1e-5
    assert rel_err(got[1], o32[1]) < 1e-5
    assert rel_err(got[2], o64[2]) < 1e-4
    assert rel_err(got[3], o64[3]) < 1e-4


# the shapes the matrix-core forward / grad input covers: one group, 3 x 3 taps, scope 3 x 3 or 4 x 4, at least 16 channels in fours
GATHER_CASES = [CASES[0], CASES[1], CASES[2], CASES[6], CASES[10], CASES[11], CASES[13], CASES[14], CASES[15], CASES[16], CASES[17]]


@pytest.mark.parametrize("case", GATHER_CASES)
def test_fp32_matrix_core_forward_and_grad_input_on_every_shape_they_cover(case, switch_off):
    """The library takes the matrix-core forward / grad input only on large layers with many channels, where they
    are the faster kernels; forced, they serve every shape they cover: ragged sizes, channel counts that are
    not a multiple of 16, stride 2 (where the transposed walk skips the taps off the stride's grid),
    dilation, nineteen channel blocks."""
    switch_off("DK_FORCE_NHWC_GATHER_MFMA")
    inputs, got = _run(case, torch.float32, seed=6)
    o32, o64 = _oracle(inputs, np.float32), _oracle(inputs, np.float64)
    assert rel_err(got[0], o32[0]) < 1e-5
    assert rel_err(got[1], o32[1]) < 1e-5
    assert rel_err(got[2], o64[2]) < 1e-4
    assert rel_err(got[3], o64[3]) < 1e-4


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", [CASES[0], CASES[2], CASES[11], CASES[13]])
def test_half_precision_matrix_core_forward_and_grad_input(case, dtype, switch_off):
    switch_off("DK_FORCE_NHWC_GATHER_MFMA")
    inputs, got = _run(case, dtype, seed=7)
    want = _oracle(inputs, np.float32)
    for g, w in zip(got, want):
        assert g.dtype == dtype
        assert rel_err(g.float(), w) < 1e-2


@pytest.mark.parametrize("case", CASES[:4] + CASES[7:8])
def test_fp64_matches_oracle(case):
    inputs, got = _run(case, torch.float64)
    want = _oracle(inputs, np.float64)
    for g, w in zip(got, want):
        assert rel_err(g, w) < 1e-11


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", CASES[:3] + CASES[5:7] + CASES[10:])   # (the last two: grad rotation partials reduced into a 16-bit tensor)
def test_half_precisions_match_fp32_oracle(case, dtype):
    inputs, got = _run(case, dtype, seed=3)
    want = _oracle(inputs, np.float32)
    for g, w in zip(got, want):
        assert g.dtype == dtype
        assert rel_err(g.float(), w) < 1e-2


def test_equals_the_planar_operator_on_the_same_tensors():
    """Same logical input, two layouts: the results agree to rounding (the sums run in another order)."""
    from deformable_kernels.ops.deform_kernel.functions import sample_depthwise
    case = (2, 48, 30, 26, 3, (4, 4), 1, 1, 1, 1, 1.0)
    N, C, H, W, k, S, s, p, d, G, rs = case
    x, wt, rot, gout, cfg = make_local(N, C, H, W, k, S, s, p, d, G, rs, seed=9)
    res = []
    for fmt in (torch.contiguous_format, torch.channels_last):
        xg = x.to(DEV).contiguous(memory_format=fmt).requires_grad_()
        rg = rot.to(DEV).contiguous(memory_format=fmt).requires_grad_()
        wg = wt.to(DEV).requires_grad_()
        out = sample_depthwise(xg, rg, wg, cfg["kernel_size"], cfg["stride"], cfg["padding"], cfg["dilation"], G)
        out.backward(gout.to(DEV))  # a planar out_grad for both: the Function brings it into its layout
        res.append([t.detach().cpu().contiguous() for t in (out, xg.grad, rg.grad, wg.grad)])
    for a, b, tol in zip(res[1], res[0], (1e-5, 1e-5, 1e-4, 1e-4)):
        assert rel_err(a, b) < tol


@pytest.mark.parametrize("groups", [2, 1])   # one group: the matrix-core kernels
@pytest.mark.parametrize("clip", ['scope', (-0.3, 0.2)])
def test_rotation_clip_inside_the_channels_last_operator(clip, groups, switch_off):
    switch_off("DK_FORCE_NHWC_GATHER_MFMA")
    case = (2, 12 if groups == 2 else 24, 11, 10, 3, (4, 4), 1, 1, 1, groups, 1.5)
    inputs, got = _run(case, torch.float32, seed=5, clip=clip)
    x, wt, rot, gout, cfg = inputs
    clamped, open_ = clipped_rotation(rot, clip, cfg["kernel_size"], (4, 4), groups)
    o64 = _oracle((x, wt, clamped, gout, cfg), np.float64)
    assert rel_err(got[0], o64[0]) < 1e-5
    assert rel_err(got[1], o64[1]) < 1e-5
    assert rel_err(got[2], torch.as_tensor(o64[2]) * open_.double()) < 1e-4
    assert rel_err(got[3], o64[3]) < 1e-4


def test_c_abi_layout_field():
    from deformable_kernels.ops.deform_kernel import _lib
    L = _lib.lib()
    x = torch.zeros(1, 4, 6, 6, device=DEV)
    d = _lib.ConvDesc(1, 4, 6, 6, 3, 3, 1, 1, 1, 1, 1, 1, 4, 4, 1, _lib.DK_F32, 0, 0.0, 0.0, 7)
    assert L.dk_sample_depthwise_forward(d, _lib.ptr(x), _lib.ptr(x), _lib.ptr(x), _lib.ptr(x), None) == -2  # bad layout
    d.layout = _lib.LAYOUT_NHWC
    off = torch.zeros(1, 18, 6, 6, device=DEV)
    assert L.dk_deformable_sample_depthwise_forward(d, _lib.ptr(x), _lib.ptr(off), _lib.ptr(off), _lib.ptr(x),
                                                    _lib.ptr(x), None) == -7  # DK_ERR_UNSUPPORTED
    assert L.dk_image_depthwise_supported(d) == 0
    assert L.dk_sample_depthwise_backward_filter_workspace(d) > 0
    assert L.dk_sample_depthwise_backward_rotation_workspace(d) == 0


def test_channels_last_input_of_a_geometry_the_channels_last_kernels_do_not_cover():
    """64 rotation groups with 3 x 3 taps and a 4 x 4 scope need 41472 bytes of tap tables, more than the
    channels-last kernels have (dk_sample_depthwise_layout_supported says 0, the C entry point DK_ERR_UNSUPPORTED).
    The Function then runs the planar kernels on a planar copy and hands the result back channels-last:
    same values as the planar call."""
    from deformable_kernels.ops.deform_kernel import _lib
    from deformable_kernels.ops.deform_kernel.functions import sample_depthwise
    case = (2, 64, 9, 10, 3, (4, 4), 1, 1, 1, 64, 1.0)
    N, C, H, W, k, S, s, p, d, G, rs = case
    x, wt, rot, gout, cfg = make_local(N, C, H, W, k, S, s, p, d, G, rs, seed=13)
    cl = torch.channels_last
    xg = x.to(DEV).contiguous(memory_format=cl)
    desc = _lib.conv_desc(xg, wt.to(DEV), cfg["kernel_size"], cfg["stride"], cfg["padding"], cfg["dilation"], G,
                          None, _lib.LAYOUT_NHWC)
    assert _lib.lib().dk_sample_depthwise_layout_supported(desc) == 0
    desc.layout = _lib.LAYOUT_NCHW
    assert _lib.lib().dk_sample_depthwise_layout_supported(desc) == 1
    res = []
    for fmt in (torch.contiguous_format, cl):
        xg = x.to(DEV).contiguous(memory_format=fmt).requires_grad_()
        rg = rot.to(DEV).contiguous(memory_format=fmt).requires_grad_()
        wg = wt.to(DEV).requires_grad_()
        out = sample_depthwise(xg, rg, wg, cfg["kernel_size"], cfg["stride"], cfg["padding"], cfg["dilation"], G)
        if fmt is cl:
            assert out.is_contiguous(memory_format=cl)
        out.backward(gout.to(DEV).contiguous(memory_format=fmt))
        res.append([t.detach().cpu().contiguous() for t in (out, xg.grad, rg.grad, wg.grad)])
    for a, b in zip(res[1], res[0]):
        assert torch.equal(a, b)  # the same kernels ran on the same values
    o64 = _oracle((x, wt, rot, gout, cfg), np.float64)
    assert rel_err(res[1][0], o64[0]) < 1e-5 and rel_err(res[1][3], o64[3]) < 1e-4
