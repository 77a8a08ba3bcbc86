"""The user-facing modules: constructor surface, state-dict keys and initialisation (CPU), and
on the GPU the module outputs against independent compositions."""
import math

import pytest
import torch
import torch.nn.functional as F

import _composite as comp
from _cases import rel_err


def test_public_names_and_state_dict_keys():
    from deformable_kernels.modules import (DeformConv2d, DeformKernel2d, DeformKernelConv2d,
                                            GlobalDeformKernel2d, LocalDeformKernel2d)
    assert DeformKernel2d is LocalDeformKernel2d
    m = DeformKernel2d((4, 4), 8, 8, 3, 1, 1, groups=8)
    assert sorted(m.state_dict()) == ["inner_conv.weight", "rotation_conv.bias", "rotation_conv.weight"]
    assert m.inner_conv.weight.shape == (8, 1, 4, 4)
    assert m.rotation_conv.weight.shape == (18, 8, 3, 3)
    g = GlobalDeformKernel2d((2, 2), 8, 8, groups=8)
    assert sorted(g.state_dict()) == ["fc.bias", "fc.weight", "weight"]
    assert g.fc.out_features == 2 and g.weight.shape == (8, 1, 2, 2)
    c = DeformKernelConv2d((4, 4), 8, 8, 3, 1, 1, groups=8)
    assert sorted(c.state_dict()) == ["inner_conv.weight", "offset_conv.bias", "offset_conv.weight"]
    d = DeformConv2d(8, 8, 3, 1, 1, groups=8)
    assert d.inner_conv.weight.shape == (8, 1, 3, 3)
    for mod in (m.rotation_conv, g.fc, c.offset_conv):
        assert mod.zero_init is True


def test_scope_weight_init_bound_and_depthwise_assertion():
    from deformable_kernels.ops.deform_kernel.modules import DeformableSampleDepthwise, SampleDepthwise
    torch.manual_seed(0)
    m = SampleDepthwise((4, 4), 64, 64, kernel_size=3, groups=64)
    bound = 1.0 / math.sqrt(9)
    assert m.weight.abs().max().item() <= bound and m.weight.abs().max().item() > 0.8 * bound
    assert m.bias is None
    b = DeformableSampleDepthwise((4, 4), 8, 8, groups=8, bias=True)
    assert torch.count_nonzero(b.bias).item() == 0 and "bias" in b.state_dict()
    with pytest.raises(AssertionError):
        SampleDepthwise((4, 4), 8, 16, groups=8)
    with pytest.raises(AssertionError):
        SampleDepthwise((4, 4), 8, 8, groups=1)


def test_global_fc_bias_is_the_centred_tap_grid():
    from deformable_kernels.modules import GlobalDeformKernel2d
    g = GlobalDeformKernel2d((5, 5), 4, 4, kernel_size=3, padding=1, groups=4)
    want = []
    for h in range(3):
        for w in range(3):
            want += [1.0 + h, 1.0 + w]   # (S - k) / 2 + tap index, the local operator's centring
    assert g.fc_bias == want


def test_cpu_tensors_are_rejected_like_the_reference():
    from deformable_kernels.modules import DeformKernel2d
    m = DeformKernel2d((4, 4), 4, 4, 3, 1, 1, groups=4)
    with pytest.raises(NotImplementedError):
        m(torch.randn(1, 4, 6, 6))


def test_hooks_on_the_offset_branch_convolution_fire():
    """A forward hook on rotation_conv / offset_conv (weight norm, profilers, quantisation observers)
    relies on the convolution being called as a module: the library's own offset-branch kernels,
    which take the parameters directly, are only used on a convolution without hooks."""
    from deformable_kernels.modules import DeformKernel2d, DeformKernelConv2d
    for m, conv in ((lambda m: (m, m.rotation_conv))(DeformKernel2d((4, 4), 4, 4, 3, 1, 1, groups=4)),
                    (lambda m: (m, m.offset_conv))(DeformKernelConv2d((4, 4), 4, 4, 3, 1, 1, groups=4))):
        seen = []
        conv.register_forward_hook(lambda mod, i, o: seen.append(tuple(o.shape)))
        with pytest.raises(NotImplementedError):   # the operator itself exists on the GPU only
            m(torch.randn(1, 4, 6, 6))
        assert seen == [(1, 18, 6, 6)]


def test_descriptor_structs_have_the_library_s_size():
    """The descriptor structs are declared three times: in include/dk_hip.h (what the library is compiled
    from), in the ctypes loader, and in the binding that the integration guide shows a maintainer of the reference.  The
    library reports its sizeof() for each; the loader's and the documented declaration must agree with it
    (a struct that is shorter than the library's is read past its end)."""
    import ctypes
    import os
    import re
    from deformable_kernels.ops.deform_kernel import _lib
    L = _lib.lib()  # the loader itself compares the three sizes and raises on a mismatch
    assert L.dk_version() >= 3  # 0.3: dk_conv_desc has `layout`, the size queries exist
    assert ctypes.sizeof(_lib.ConvDesc) == L.dk_conv_desc_size() == 19 * 4 + 4
    assert ctypes.sizeof(_lib.NdDesc) == L.dk_nd_desc_size()
    assert ctypes.sizeof(_lib.OffsetConvDesc) == L.dk_offset_conv_desc_size()
    # the struct as the integration guide declares it: take the class statement out of the document and build it
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    doc = open(os.path.join(root, "INTEGRATION.md")).read()
    m = re.search(r"^class ConvDesc\(ctypes\.Structure\):.*?\n(?=\nlib = )", doc, re.S | re.M)
    assert m, "the integration guide no longer shows the ConvDesc declaration"
    scope = {"ctypes": ctypes}
    exec(m.group(0), scope)
    documented = scope["ConvDesc"]
    assert ctypes.sizeof(documented) == L.dk_conv_desc_size()
    assert [f[0] for f in documented._fields_] == [f[0] for f in _lib.ConvDesc._fields_]


def test_c_abi_exports_every_declared_symbol():
    import ctypes
    import os
    import re
    from deformable_kernels.ops.deform_kernel import _lib
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    header = open(os.path.join(root, "include", "dk_hip.h")).read()
    declared = set(re.findall(r"\b(dk_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(handle, name), name
    assert _lib.lib().dk_version() >= 1


def test_c_abi_rejects_bad_arguments_before_any_launch():
    import ctypes
    from deformable_kernels.ops.deform_kernel import _lib
    L = _lib.lib()
    ok = _lib.ConvDesc(1, 4, 8, 8, 3, 3, 1, 1, 1, 1, 1, 1, 4, 4, 1, _lib.DK_F32)
    oh, ow = ctypes.c_int32(), ctypes.c_int32()
    assert L.dk_conv_out_size(ctypes.byref(ok), ctypes.byref(oh), ctypes.byref(ow)) == 0
    assert (oh.value, ow.value) == (8, 8)
    null = ctypes.c_void_p(0)
    assert L.dk_sample_depthwise_forward(None, null, null, null, null, null) == -1
    assert L.dk_sample_depthwise_forward(ctypes.byref(ok), null, null, null, null, null) == -1
    bad_groups = _lib.ConvDesc(1, 4, 8, 8, 3, 3, 1, 1, 1, 1, 1, 1, 4, 4, 3, _lib.DK_F32)
    assert L.dk_conv_out_size(ctypes.byref(bad_groups), None, None) == -2
    too_small = _lib.ConvDesc(1, 4, 2, 2, 5, 5, 1, 1, 0, 0, 1, 1, 4, 4, 1, _lib.DK_F32)
    assert L.dk_conv_out_size(ctypes.byref(too_small), None, None) == -2
    bad_dtype = _lib.ConvDesc(1, 4, 8, 8, 3, 3, 1, 1, 1, 1, 1, 1, 4, 4, 1, 9)
    assert L.dk_conv_out_size(ctypes.byref(bad_dtype), None, None) == -3
    bad_clip = _lib.ConvDesc(1, 4, 8, 8, 3, 3, 1, 1, 1, 1, 1, 1, 4, 4, 1, _lib.DK_F32, 3, 0.0, 1.0)
    assert L.dk_conv_out_size(ctypes.byref(bad_clip), None, None) == -2
    empty_range = _lib.ConvDesc(1, 4, 8, 8, 3, 3, 1, 1, 1, 1, 1, 1, 4, 4, 1, _lib.DK_F32, 1, 1.0, 0.0)
    assert L.dk_conv_out_size(ctypes.byref(empty_range), None, None) == -2
    huge = _lib.ConvDesc(4096, 4096, 512, 512, 3, 3, 1, 1, 1, 1, 1, 1, 4, 4, 1, _lib.DK_F32)
    assert L.dk_conv_out_size(ctypes.byref(huge), None, None) == -4
    # a workspace that is too small is refused
    one = ctypes.c_void_p(16)  # never dereferenced: the call is rejected first
    need = L.dk_sample_depthwise_backward_filter_workspace(ctypes.byref(ok))
    assert need > 0
    assert L.dk_sample_depthwise_backward_filter(ctypes.byref(ok), one, one, one, one, one, need - 1, null) == -5
    nd = _lib.NdDesc(4, 2, 9, (ctypes.c_int32 * 8)(*([2] * 8)), _lib.DK_F32)
    assert L.dk_nd_linear_sample_forward(ctypes.byref(nd), one, one, null, one, null, 0, null) == -7
    assert b"workspace" in L.dk_status_string(-5)


def test_native_self_tests_of_the_c_abi_and_the_oracle():
    """The C driver of the C ABI's argument handling (every rejection path and the workspace arithmetic
    over a sweep of geometries; all answered on the host) against the library as built, and the oracle's
    own driver under AddressSanitizer + UndefinedBehaviorSanitizer.  (`make -C deformable-kernels_amd/csrc
    sanitize` runs the first one with the library's host code under the sanitizers as well: a build of
    minutes, not part of this suite.)"""
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run(["make", "-s", "-C", os.path.join(root, "deformable-kernels_amd", "csrc"), "selftest"],
                       capture_output=True, text=True)
    assert r.returncode == 0 and "abi selftest ok" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]
    r = subprocess.run(["make", "-s", "-C", os.path.join(root, "oracle"), "sanitize"], capture_output=True, text=True)
    assert r.returncode == 0 and "oracle selftest ok" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]


@pytest.mark.gpu
def test_local_module_matches_composite_and_backpropagates():
    from deformable_kernels.modules import DeformKernel2d
    torch.manual_seed(1)
    dev = torch.device("cuda:0")
    m = DeformKernel2d((4, 4), 12, 12, 3, 1, 1, groups=12).to(dev)
    torch.nn.init.normal_(m.rotation_conv.weight, std=0.05)
    x = torch.randn(2, 12, 10, 9, device=dev, requires_grad=True)
    out = m(x)
    out.square().sum().backward()
    assert x.grad is not None and m.inner_conv.weight.grad is not None and m.rotation_conv.weight.grad is not None
    rot = m.rotation_conv(x).detach().double().cpu()
    want = comp.local_dk(x.detach().double().cpu(), rot, m.inner_conv.weight.detach().double().cpu())
    assert rel_err(out.detach().cpu(), want) < 1e-5


@pytest.mark.gpu
def test_rotation_clip_scope_keeps_coordinates_inside_the_tile():
    from deformable_kernels.modules import DeformKernel2d
    torch.manual_seed(2)
    dev = torch.device("cuda:0")
    m = DeformKernel2d((4, 4), 6, 6, 3, 1, 1, groups=6, rotation_clip='scope').to(dev)
    torch.nn.init.normal_(m.rotation_conv.weight, std=1.0)
    x = torch.randn(1, 6, 8, 8, device=dev)
    rot = m._clip_rotation(m.rotation_conv(x))
    centre = torch.tensor([0.5, 0.5, 0.5, 1.5, 0.5, 2.5, 1.5, 0.5, 1.5, 1.5, 1.5, 2.5, 2.5, 0.5, 2.5, 1.5, 2.5, 2.5],
                          device=dev).view(1, 18, 1, 1)
    coord = rot + centre
    assert coord.min().item() >= -1e-6 and coord.max().item() <= 3 + 1e-6
    assert m(x).shape == (1, 6, 8, 8)
    m2 = DeformKernel2d((4, 4), 6, 6, 3, 1, 1, groups=6, rotation_clip=(-0.25, 0.25)).to(dev)
    torch.nn.init.normal_(m2.rotation_conv.weight, std=1.0)
    assert m2._clip_rotation(m2.rotation_conv(x)).abs().max().item() <= 0.25


@pytest.mark.gpu
def test_deform_conv_module_is_depthwise_conv_at_zero_offsets():
    from deformable_kernels.modules import DeformConv2d, DeformKernelConv2d
    torch.manual_seed(3)
    dev = torch.device("cuda:0")
    m = DeformConv2d(8, 8, 3, 2, 1, groups=8).to(dev)
    torch.nn.init.zeros_(m.offset_conv.weight)
    torch.nn.init.zeros_(m.offset_conv.bias)
    x = torch.randn(2, 8, 11, 11, device=dev)
    want = F.conv2d(x, m.inner_conv.weight, None, 2, 1, 1, groups=8)
    assert rel_err(m(x).cpu(), want.cpu()) < 1e-5
    k = DeformKernelConv2d((4, 4), 8, 8, 3, 1, 1, groups=8).to(dev)
    torch.nn.init.normal_(k.offset_conv.weight, std=0.1)
    xr = x.clone().requires_grad_()
    k(xr).sum().backward()
    assert xr.grad is not None and k.offset_conv.weight.grad is not None


@pytest.mark.gpu
def test_global_module_equals_local_operator_with_constant_rotation():
    """GlobalDeformKernel2d (nd_linear_sample + one grouped conv) computes what the local operator
    computes when every pixel of an image shares the rotation fc(avg(x)): the cross-check that
    ties the N-d sampler to the fused operator (centring term, tap order, clamp)."""
    from deformable_kernels.modules import GlobalDeformKernel2d
    from deformable_kernels.ops.deform_kernel.functions import sample_depthwise
    torch.manual_seed(4)
    dev = torch.device("cuda:0")
    N, C, S, k = 3, 10, 5, 3
    m = GlobalDeformKernel2d((S, S), C, C, kernel_size=k, padding=1, groups=C).to(dev)
    m.fused = False  # the reference's route: nd_linear_sample + grouped convolution
    torch.nn.init.normal_(m.fc.weight, std=0.3)
    x = torch.randn(N, C, 9, 8, device=dev)
    out = m(x)
    with torch.no_grad():
        centre = torch.tensor(m.fc_bias, device=dev).unsqueeze(0)
        coord = (m.fc(x.mean((2, 3))) + centre).clamp(0, S - 1)
        rot = (coord - centre).view(N, 18, 1, 1).expand(N, 18, 9, 8).contiguous()
        want = sample_depthwise(x, rot, m.weight, (k, k), (1, 1), (1, 1), (1, 1), 1)
    assert rel_err(out.detach().cpu(), want.cpu()) < 1e-5
    out.sum().backward()
    assert m.weight.grad is not None and m.fc.weight.grad is not None
    # the fused route of the module (one call of the local operator): same output, same gradients
    g_ref = [p.grad.clone() for p in (m.weight, m.fc.weight, m.fc.bias)]
    m.zero_grad()
    m.fused = True
    x2 = x.clone().requires_grad_()
    out2 = m(x2)
    assert rel_err(out2.detach().cpu(), out.detach().cpu()) < 1e-5
    out2.sum().backward()
    for got, ref in zip((m.weight.grad, m.fc.weight.grad, m.fc.bias.grad), g_ref):
        assert rel_err(got.cpu(), ref.cpu()) < 1e-4


@pytest.mark.gpu
def test_global_module_under_autocast_returns_what_the_framework_convolution_returns():
    """Inside an autocast region the reference's F.conv2d (modules/deform_kernel.py:103-111) returns the autocast
    dtype.  The library's per-image convolution computes in the tensors' own type, so the module only takes it
    outside such regions: with and without `native_conv` the output dtype is the same."""
    from deformable_kernels.modules import GlobalDeformKernel2d
    dev = torch.device("cuda:0")
    torch.manual_seed(3)
    m = GlobalDeformKernel2d((5, 5), 16, 16, kernel_size=3, padding=1, groups=16).to(dev)
    x = torch.randn(2, 16, 12, 12, device=dev)
    outs = []
    for native in (True, False):
        m.native_conv = native
        with torch.autocast(device_type="cuda", dtype=torch.float16):
            outs.append(m(x))
    assert outs[0].dtype == outs[1].dtype == torch.float16
    assert rel_err(outs[0].float().cpu(), outs[1].float().cpu()) < 1e-6
    m.native_conv = True
    assert m(x).dtype == torch.float32  # outside the region: the library's convolution, in the tensors' type


@pytest.mark.gpu
@pytest.mark.parametrize("clip", ['scope', (-0.3, 0.2)])
def test_local_module_clamps_inside_the_operator_as_the_reference_sequence_does(clip):
    """LocalDeformKernel2d with rotation_clip: clamping inside the operator (fused_clip, the
    default) against the reference's sequence of clamping the rotation tensor first
    (modules/deform_kernel.py:185-221) -- same output, same gradients down to rotation_conv."""
    from deformable_kernels.modules import LocalDeformKernel2d
    torch.manual_seed(11)
    dev = torch.device("cuda:0")
    C = 12
    m = LocalDeformKernel2d((4, 4), C, C, 3, 1, 1, 1, C, 2, False, clip).to(dev)
    torch.nn.init.normal_(m.rotation_conv.weight, std=0.2)
    x = torch.randn(2, C, 11, 10, device=dev)
    gout = torch.randn(2, C, 11, 10, device=dev)
    results = []
    for fused in (False, True):
        m.fused_clip = fused
        m.zero_grad()
        xi = x.clone().requires_grad_()
        out = m(xi)
        out.backward(gout)
        results.append([t.detach().cpu().clone() for t in (
            out, xi.grad, m.inner_conv.weight.grad, m.rotation_conv.weight.grad, m.rotation_conv.bias.grad)])
    assert rel_err(results[1][0], results[0][0]) < 1e-5
    for got, ref in zip(results[1][1:], results[0][1:]):
        assert rel_err(got, ref) < 1e-4
