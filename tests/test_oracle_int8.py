"""Pins the oracle's int8 arithmetic: exact-rational brute force and invariants
for the quantiser, integer identities against torch._int_mm for the GEMM, numpy
float32 for the epilogue and F.linear (the reference's real path,
astrai/model/components/linear.py:20-21) end to end."""
from fractions import Fraction

import numpy as np
import pytest
import torch


def _fl32(q: Fraction) -> Fraction:
    """Correctly rounded (nearest-even) fp32 value of a rational."""
    if q == 0:
        return Fraction(0)
    sign = -1 if q < 0 else 1
    a = abs(q)
    e = 0
    while a / Fraction(2) ** e >= 2 ** 24:
        e += 1
    while a / Fraction(2) ** e < 2 ** 23 and e > -149:
        e -= 1
    n = round(a / Fraction(2) ** e)  # Fraction.__round__ is half-to-even
    return sign * n * Fraction(2) ** e


def _quant_row_exact(row):
    """The frozen definition evaluated in exact rationals."""
    fr = [Fraction(float(v)) for v in row]
    amax = max((abs(v) for v in fr), default=Fraction(0))
    s = _fl32(amax / 127) if amax != 0 else Fraction(1)
    q = []
    for v in fr:
        r = round(_fl32(v / s))  # rint, half-to-even
        q.append(max(-127, min(127, r)))
    return q, float(s)


def _both(oracle, x):
    qn, sn = oracle.np_quant_rowwise_i8(x)
    qc, sc = oracle.c_quant_rowwise_i8(x)
    assert np.array_equal(qn, qc) and np.array_equal(sn.view(np.uint32), sc.view(np.uint32))
    return qc, sc


def test_quant_rowwise_brute_force_exact_rationals(oracle):
    rng = np.random.default_rng(3)
    x = np.concatenate([
        rng.standard_normal((12, 48)),
        rng.standard_normal((4, 48)) * 1e-30,   # tiny magnitudes, scale near subnormal
        rng.standard_normal((4, 48)) * 1e30,
        rng.integers(-5, 6, (4, 48)),           # many exact ratios and ties
    ]).astype(np.float32)
    q, s = _both(oracle, x)
    for r in range(x.shape[0]):
        qe, se = _quant_row_exact(x[r])
        assert s[r] == np.float32(se)
        assert list(q[r]) == qe, f"row {r}"


def test_quant_rowwise_half_to_even_ties(oracle):
    # amax = 127 -> s = 1 exactly, so a = n + 0.5 are exact ties.
    row = np.array([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, 64.5, 126.5, -126.5, 0.49999997], np.float32)
    q, s = _both(oracle, row[None, :])
    assert s[0] == 1.0
    assert list(q[0]) == [127, 0, 2, 2, 0, -2, -2, 64, 64, 126, -126, 0]
    # s = 2: a = 2n + 1 are ties
    row2 = np.array([254.0, 1.0, 3.0, 5.0, -7.0, 253.0], np.float32)
    q2, s2 = _both(oracle, row2[None, :])
    assert s2[0] == 2.0 and list(q2[0]) == [127, 0, 2, 2, -4, 126]


def test_quant_rowwise_invariants(oracle):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((64, 256)).astype(np.float32)
    x[:, 7] *= 20
    x[5] = 0
    x[9, :] = 0
    x[9, 3] = -2.5
    q, s = _both(oracle, x)
    nz = np.abs(x).max(1) > 0
    assert np.all(np.abs(q[nz]).max(1) == 127)
    assert np.all(q[5] == 0) and s[5] == 1.0
    assert q[9, 3] == -127 and np.count_nonzero(q[9]) == 1
    qn, sn = _both(oracle, -x)
    assert np.array_equal(qn, -q) and np.array_equal(sn, s)
    err = np.abs(x.astype(np.float64) - q.astype(np.float64) * s[:, None].astype(np.float64))
    assert np.all(err <= s[:, None].astype(np.float64) * 0.5 * (1 + 1e-6))
    # the scale is invariant to the order of the row
    perm = rng.permutation(256)
    qp, sp = _both(oracle, x[:, perm])
    assert np.array_equal(qp, q[:, perm]) and np.array_equal(sp, s)


def test_quant_rowwise_bf16_input_equals_widened_f32(oracle):
    rng = np.random.default_rng(5)
    bits = oracle.np_f32_to_bf16_bits(rng.standard_normal((16, 128)).astype(np.float32))
    q1, s1 = oracle.c_quant_rowwise_i8(bits, bf16_bits=True)
    q2, s2 = oracle.c_quant_rowwise_i8(oracle.np_bf16_bits_to_f32(bits))
    assert np.array_equal(q1, q2) and np.array_equal(s1, s2)


@pytest.mark.parametrize("M,N,K", [(1, 1, 16), (7, 13, 48), (64, 96, 2048), (3, 5, 8192)])
def test_gemm_i8_i32_matches_torch_int_mm_and_numpy(oracle, M, N, K):
    rng = np.random.default_rng(6)
    xq = rng.integers(-127, 128, (M, K), dtype=np.int8)
    wq = rng.integers(-127, 128, (N, K), dtype=np.int8)
    want = xq.astype(np.int64) @ wq.astype(np.int64).T
    assert np.array_equal(oracle.c_gemm_i8_i32(xq, wq), want)
    assert np.array_equal(oracle.np_gemm_i8_i32(xq, wq), want)
    t = torch.matmul(torch.from_numpy(xq).int(), torch.from_numpy(wq).int().T).numpy()
    assert np.array_equal(t, want)


def test_gemm_int_mm_library_routine(oracle):
    # torch._int_mm wants M > 16 and multiples of 8
    rng = np.random.default_rng(7)
    xq = rng.integers(-127, 128, (32, 256), dtype=np.int8)
    wq = rng.integers(-127, 128, (64, 256), dtype=np.int8)
    want = torch._int_mm(torch.from_numpy(xq), torch.from_numpy(wq).T.contiguous()).numpy()
    assert np.array_equal(oracle.c_gemm_i8_i32(xq, wq), want)


def test_gemm_extremes_do_not_overflow(oracle):
    K = 8192
    xq = np.full((2, K), 127, np.int8)
    wq = np.stack([np.full(K, 127, np.int8), np.full(K, -127, np.int8)])
    acc = oracle.c_gemm_i8_i32(xq, wq)
    assert acc[0, 0] == K * 127 * 127 and acc[1, 1] == -K * 127 * 127


def test_epilogue_c_equals_numpy_f32_and_bf16(oracle):
    rng = np.random.default_rng(8)
    acc = rng.integers(-(2 ** 27), 2 ** 27, (33, 65)).astype(np.int32)
    sx = rng.uniform(1e-3, 1e-1, 33).astype(np.float32)
    sw = rng.uniform(1e-4, 1e-2, 65).astype(np.float32)
    b = rng.standard_normal(65).astype(np.float32) * 0.01
    for bias in (None, b):
        y = oracle.np_dequant_epilogue(acc, sx, sw, bias)
        yc = oracle.c_dequant_epilogue(acc, sx, sw, bias)
        assert np.array_equal(y.view(np.uint32), yc.view(np.uint32))
        yb = oracle.c_dequant_epilogue(acc, sx, sw, bias, bf16_out=True)
        assert np.array_equal(yb, oracle.np_f32_to_bf16_bits(y))
    # hand-checked values: acc=3, sx=0.5, sw=0.25, bias=1 -> 1.375
    one = oracle.c_dequant_epilogue(np.array([[3]], np.int32), np.array([0.5], np.float32),
                                    np.array([0.25], np.float32), np.array([1.0], np.float32))
    assert one[0, 0] == 1.375


def _config1(seed=0):
    """benchmark configuration 1: X 64x2048 N(0,1) with 4 seeded outlier columns x20,
    W 2048x2048 N(0, 0.02)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(64, 2048, generator=g)
    cols = torch.randperm(2048, generator=g)[:4]
    x[:, cols] *= 20
    w = torch.randn(2048, 2048, generator=g) * 0.02
    return x, w


def _predicted_rel_error(x, w, sx, sw):
    """Uniform-noise model of symmetric rounding: each operand element carries
    an independent error of variance scale^2/12."""
    e2 = (sx.astype(np.float64) ** 2 / 12).sum() * (w.astype(np.float64) ** 2).sum()
    e2 += (sw.astype(np.float64) ** 2 / 12).sum() * (x.astype(np.float64) ** 2).sum()
    ref = x.astype(np.float64) @ w.astype(np.float64).T
    return np.sqrt(e2) / np.linalg.norm(ref)


def test_config1_linear_w8a8_vs_reference_float_linear(oracle):
    x, w = _config1()
    wq, sw = oracle.c_quant_rowwise_i8(w.numpy())
    _, sx = oracle.c_quant_rowwise_i8(x.numpy())
    y = oracle.c_linear_w8a8(x.numpy(), wq, sw)
    y2 = oracle.np_linear_w8a8(x.numpy(), wq, sw)
    assert np.array_equal(y.view(np.uint32), y2.view(np.uint32))
    ref = torch.nn.functional.linear(x, w).numpy()  # linear.py:21
    rel = np.linalg.norm(y - ref) / np.linalg.norm(ref)
    pred = _predicted_rel_error(x.numpy(), w.numpy(), sx, sw)
    # two-sided: a wrong scale, a dropped term or a transposed operand lands
    # far outside the rounding-noise prediction
    assert 0.8 * pred < rel < 1.25 * pred, (rel, pred)
    assert rel < 8e-2
    # without the outlier columns the same scheme does markedly better
    g = torch.Generator().manual_seed(0)
    x0 = torch.randn(64, 2048, generator=g)
    _, sx0 = oracle.c_quant_rowwise_i8(x0.numpy())
    y0 = oracle.c_linear_w8a8(x0.numpy(), wq, sw)
    ref0 = torch.nn.functional.linear(x0, w).numpy()
    rel0 = np.linalg.norm(y0 - ref0) / np.linalg.norm(ref0)
    pred0 = _predicted_rel_error(x0.numpy(), w.numpy(), sx0, sw)
    assert 0.8 * pred0 < rel0 < 1.25 * pred0, (rel0, pred0)
    assert rel0 < 0.4 * rel and rel0 < 1.5e-2, (rel0, rel)
    # the oracle's own fp32 Linear agrees with torch's
    assert np.allclose(oracle.c_linear_f32(x.numpy(), w.numpy()), ref, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("divisor", [127.0, 448.0])
def test_one_correction_divide_gives_the_code_of_the_divide_for_every_pair_of_bf16_numbers(oracle, divisor):
    """The HIP quantisers round rows of bf16 numbers with one correction step on a correctly rounded
    reciprocal instead of the divide of the definition.  Every pair (row maximum, value) of bf16 numbers the
    shortcut can meet, 5.6e8 of them per code format, evaluated one by one with the same IEEE operations:
    no pair's code differs.  The product with the reciprocal alone (no correction) does differ, so the
    evaluation can tell."""
    bad, pairs = oracle.c_one_step_divide_mismatches(divisor)
    assert pairs > 5.5e8 and bad == 0
    bad0, _ = oracle.c_one_step_divide_mismatches(divisor, am_lo=0x3F80, am_hi=0x4000, steps=0)
    assert bad0 > 0


def test_adjusted_reciprocal_product_gives_the_code_of_the_divide_for_every_pair_of_bf16_numbers(oracle):
    """The int8 quantisers round rows of bf16 numbers with ONE product, value times a reciprocal of the scale
    that is moved by one unit in the last place where the row maximum's mantissa asks for it.  Every pair
    (row maximum, value), 5.6e8 of them: no code differs from the divide's.  The same product with the plain
    reciprocal does differ (steps=0 above), and so does a table that moves nothing or moves the wrong way --
    one binade of maxima under the plain reciprocal shows mismatches exactly where the table holds a move."""
    bad, pairs = oracle.c_one_step_divide_mismatches(127.0, steps=-1)
    assert pairs > 5.5e8 and bad == 0
    # per mantissa: the plain reciprocal fails for the 24 mantissas whose entry is not 0, and only there
    table = [0x00000000, 0x05015A02, 0x80000000, 0x10004480, 0x00000000, 0x40014442, 0x40000004, 0x00000105]
    moved = {m for m in range(128) if (table[m >> 4] >> (2 * (m & 15))) & 3}
    assert len(moved) == 24
    failing = {m for m in range(128)
               if oracle.c_one_step_divide_mismatches(127.0, am_lo=0x3F80 + m, am_hi=0x3F80 + m + 1, steps=0)[0]}
    assert failing == moved
