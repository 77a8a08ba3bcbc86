"""Seeded random geometries through the tuned kernels against the CPU oracle: plane sizes from one
pixel to 260 columns, channel counts that fill no tile, every scope and stride of the tuned
families, rotation groups.  The fixed cases of test_gpu_local.py / test_gpu_deform.py name the
situations they cover; this sweep is for the ones nobody thought of (it found planes 64 and 112
columns wide losing their first three elements in the matrix-core grad filter)."""
import random

import numpy as np
import pytest
import torch

import test_gpu_deform as td
import test_gpu_local as tl
from _cases import rel_err

pytestmark = pytest.mark.gpu


def _local_cases():
    rnd = random.Random(5)
    cases = []
    for _ in range(24):   # stride 2, padding 1: pair-load forward, quad grad input, matrix-core or dense grad filter
        cases.append((rnd.choice([1, 2, 3]), rnd.choice([1, 2, 3, 5, 16, 17, 33, 48]),
                      rnd.choice([2, 3, 4, 5, 6, 7, 9, 12, 14, 17, 28, 33]),
                      rnd.choice([2, 4, 6, 8, 10, 14, 18, 26, 30, 56, 64, 112, 130, 260]), 3,
                      rnd.choice([(3, 3), (4, 4), (5, 5), (7, 7)]), 2, 1, 1, 1, 1.0))
    for _ in range(12):   # stride 1, padding 1: row kernels, matrix-core grad filter
        cases.append((rnd.choice([1, 2]), rnd.choice([1, 3, 16, 20, 40]), rnd.choice([1, 2, 3, 5, 8, 13]),
                      rnd.choice([1, 2, 3, 5, 9, 31, 63, 64, 112, 130]), 3,
                      rnd.choice([(3, 3), (4, 4), (5, 5), (7, 7)]), 1, 1, 1, 1, 1.0))
    out = []
    for c in cases:   # rotation groups that divide the channel count
        groups = [g for g in (1, 2, 3) if c[1] % g == 0]
        out.append(c[:9] + (rnd.choice(groups), c[10]))
    return out


def _deform_cases():
    rnd = random.Random(11)
    cases = []
    while len(cases) < 20:
        H = rnd.choice([1, 2, 3, 5, 7, 8, 14, 16, 17, 28, 31, 32, 33, 36])
        W = rnd.choice([1, 2, 3, 7, 8, 14, 16, 28, 31, 32, 33, 36, 40, 64])
        C = rnd.choice([1, 2, 3, 4, 5, 8, 9, 16, 17, 33, 48])
        G = rnd.choice([g for g in (1, 2, 3) if C % g == 0])
        s, p, d = rnd.choice([1, 2]), rnd.choice([0, 1]), rnd.choice([1, 1, 2])
        if (H + 2 * p - 2 * d - 1) // s + 1 < 1 or (W + 2 * p - 2 * d - 1) // s + 1 < 1:
            continue
        cases.append((rnd.choice([1, 2]), C, H, W, 3, rnd.choice([(3, 3), (4, 4), (5, 5)]), s, p, d, G, 0.7,
                      rnd.choice([0.5, 2.0, 6.0])))
    return cases


@pytest.mark.parametrize("case", _local_cases())
def test_local_operator_on_random_geometries(case):
    inputs, got = tl._run(case, torch.float32)
    o32, o64 = tl._oracle(inputs, np.float32), tl._oracle(inputs, np.float64)
    assert rel_err(got[0], o32[0]) < 1e-5
    assert rel_err(got[1], o32[1]) < 1e-5
    assert rel_err(got[2], o64[2]) < 1e-4
    assert rel_err(got[3], o64[3]) < 1e-4


def _deform_large_cases():
    """Planes of 30 to 64 rows and columns: the 1024-thread channel-interleaved kernels, tiled grad input."""
    rnd = random.Random(13)
    cases = []
    for _ in range(10):
        C = rnd.choice([1, 3, 4, 6, 9, 13])
        cases.append((rnd.choice([1, 2]), C, rnd.randint(30, 64), rnd.randint(30, 64), 3,
                      rnd.choice([(3, 3), (4, 4), (5, 5)]), rnd.choice([1, 2]), rnd.choice([0, 1]), rnd.choice([1, 1, 2]),
                      rnd.choice([g for g in (1, 3) if C % g == 0]), 0.7, rnd.choice([0.5, 2.0, 6.0])))
    return cases


def _deform_huge_cases():
    """Planes that fit LDS once or not at all (100 to 260 rows and columns): row windows, the rows-and-columns window
    of the grad filter, the band form of the grad input."""
    rnd = random.Random(17)
    cases = []
    for _ in range(6):
        C = rnd.choice([2, 3, 6, 10])
        cases.append((1, C, rnd.randint(100, 260), rnd.randint(100, 260), 3, rnd.choice([(3, 3), (4, 4), (5, 5)]),
                      rnd.choice([1, 1, 2]), rnd.choice([0, 1]), rnd.choice([1, 1, 2]),
                      rnd.choice([g for g in (1, 2, 3) if C % g == 0]), 0.7, rnd.choice([0.5, 2.0, 9.0])))
    return cases


@pytest.mark.parametrize("case", _deform_cases() + _deform_large_cases() + _deform_huge_cases())
def test_deformable_operator_on_random_geometries(case):
    inputs, got = td._run(case, torch.float32)
    td.assert_fp32_parity(got, td._oracle(inputs, np.float32), td._oracle(inputs, np.float64))


@pytest.mark.parametrize("k,case", list(enumerate(_local_cases()))[::2])
def test_local_operator_on_random_geometries_in_16_bits(k, case):
    """bf16 and fp16 in turn; the matrix-core grad filter multiplies them with bfloat16 instructions."""
    dtype = torch.bfloat16 if k % 4 == 0 else torch.float16
    inputs, got = tl._run(case, dtype)
    want = tl._oracle(inputs, np.float32)   # on the inputs as rounded to dtype
    for g, w, name in zip(got, want, ("forward", "grad input", "grad rotation", "grad filter")):
        assert g.dtype == dtype
        assert rel_err(g.float(), w) < 1e-2, name


def _nhwc_cases():
    """One rotation group, 3 x 3 taps, channel counts in fours and eights: the shapes the channels-last
    matrix-core kernels cover, with every stride / padding / dilation and both of their scopes."""
    rnd = random.Random(31)
    cases = []
    while len(cases) < 28:
        H, W = rnd.choice([1, 2, 3, 5, 7, 8, 13, 14, 16, 17, 28, 33]), rnd.choice([1, 2, 3, 4, 7, 9, 15, 16, 17, 31, 40])
        C = rnd.choice([16, 20, 24, 36, 40, 64, 72, 100, 136])
        s, p, d = rnd.choice([1, 1, 2]), rnd.choice([0, 1, 2]), rnd.choice([1, 1, 2])
        if (H + 2 * p - 2 * d - 1) // s + 1 < 1 or (W + 2 * p - 2 * d - 1) // s + 1 < 1:
            continue
        cases.append((rnd.choice([1, 2, 3]), C, H, W, 3, rnd.choice([(3, 3), (4, 4), (4, 4), (5, 5)]), s, p, d, 1, 1.0))
    return cases


@pytest.mark.parametrize("k,case", list(enumerate(_nhwc_cases())))
def test_channels_last_matrix_core_kernels_on_random_geometries(k, case, switch_off):
    """float32, and every fourth case bfloat16 / float16; the matrix-core forward / grad input forced on every
    shape it covers (scope 5 x 5 keeps the table kernel for them; grad rotation and grad filter take their
    matrix-core kernels)."""
    import test_gpu_nhwc as tn
    switch_off("DK_FORCE_NHWC_GATHER_MFMA")
    if k % 4 == 3:
        dtype = torch.bfloat16 if k % 8 == 3 else torch.float16
        inputs, got = tn._run(case, dtype, seed=k)
        want = tn._oracle(inputs, np.float32)
        for g, w, name in zip(got, want, ("forward", "grad input", "grad rotation", "grad filter")):
            assert g.dtype == dtype
            assert rel_err(g.float(), w) < 1e-2, name
        return
    inputs, got = tn._run(case, torch.float32, seed=k)
    o32, o64 = tn._oracle(inputs, np.float32), tn._oracle(inputs, np.float64)
    assert rel_err(got[0], o32[0]) < 1e-5
    assert rel_err(got[1], o32[1]) < 1e-5
    assert rel_err(got[2], o64[2]) < 1e-4
    assert rel_err(got[3], o64[3]) < 1e-4


def _offset_conv_cases():
    rnd = random.Random(23)
    cases = []
    for _ in range(36):
        stride = rnd.choice([1, 1, 2])
        W = rnd.choice([7, 14, 28, 56, 112] if stride == 1 else [14, 28, 56, 112])
        cases.append((rnd.choice([1, 2, 3, 5]), rnd.choice([16, 32, 48, 80, 144]), rnd.choice([1, 2, 3, 5, 7, 8, 9, 14, 17, 23, 33]),
                      W, rnd.choice([1, 2, 7, 15, 16, 18, 20]), stride, rnd.choice(["float32", "float16", "bfloat16"])))
    return cases


@pytest.mark.parametrize("case", _offset_conv_cases())
def test_offset_branch_convolution_on_random_shapes(case):
    """Every pass of the layers' 3 x 3 offset convolution (forward, input, weight and bias gradient; stride 1 and
    2; 1 to 20 outputs; tiles of one row, partial last tiles, planes lower than a tile) against the float64
    convolution on the CPU."""
    import test_gpu_offset_conv as toc
    from deformable_kernels.ops.deform_kernel.functions import offset_conv, offset_conv_supported
    N, C, H, W, O, stride, dtype_name = case
    dtype = getattr(torch, dtype_name)
    tol = {"float32": 1e-5, "float16": 2e-3, "bfloat16": 1e-2}[dtype_name]
    g = torch.Generator().manual_seed(hash(case[:6]) % 1000)
    dev = torch.device("cuda:0")
    x = torch.randn(N, C, H, W, generator=g).to(dtype).to(dev).requires_grad_()
    w = (torch.randn(O, C, 3, 3, generator=g) * 0.05).to(dtype).to(dev).requires_grad_()
    b = torch.randn(O, generator=g).to(dtype).to(dev).requires_grad_()
    assert offset_conv_supported(x, w, b, stride, 1, 1)
    out = offset_conv(x, w, b, stride=stride, force=True)
    gout = torch.randn(out.shape, generator=g).to(dtype).to(dev)
    want, gx, gw, gb = toc.reference(x, w, b, gout, stride=stride)
    assert out.shape == want.shape and out.dtype == dtype
    out.backward(gout)
    assert rel_err(out.detach().double().cpu(), want) < tol, "forward"
    assert rel_err(x.grad.double().cpu(), gx) < tol, "input gradient"
    assert rel_err(w.grad.double().cpu(), gw) < tol, "weight gradient"
    assert rel_err(b.grad.double().cpu(), gb) < tol, "bias gradient"
