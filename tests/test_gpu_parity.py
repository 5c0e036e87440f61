"""GPU parity: the HIP kernels, called through the C ABI (ctypes, via
khaosz_amd.ops), against the CPU oracle on the same seeded inputs.

Bar: bit-exact for int8 codes, scales, int32 accumulators and (stronger than
required) the dequantised int8-path outputs; FP8 codes bit-exact, FP8 GEMM
outputs within rtol 1e-2 (the stated tolerance for bf16/FP8 outputs)."""
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from khaosz_amd import _abi, ops  # noqa: E402
from khaosz_amd.linear import Fp8Linear, Linear, QuantLinear, quantize_model  # noqa: E402

DEV = "cuda:0"


def _say(*a):
    print(*a, file=sys.stderr, flush=True)


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def to_np(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().numpy()


def make_x(M, K, seed, outlier_cols=0, outlier_gain=20.0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g)
    if outlier_cols:
        cols = torch.randperm(K, generator=g)[:outlier_cols]
        x[:, cols] *= outlier_gain
    return x


# ------------------------------------------------------------------ quantise

ROW_SHAPES = [(1, 16), (7, 48), (5, 1040), (64, 2048), (9, 5632), (3, 8192 + 48), (130, 16384)]


@pytest.mark.parametrize("M,K", ROW_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_quant_rowwise_bit_exact(oracle, M, K, dtype):
    _say("quant_rowwise", M, K, dtype)
    x = make_x(M, K, seed=M * 7 + K, outlier_cols=min(4, K // 8))
    if M > 4:
        x[1] = 0                      # all-zero row -> scale 1, codes 0
        x[2] *= 1e-30                 # scale near the subnormal range
        x[3] *= 1e30
        x[4, :] = torch.arange(K) % 7 - 3  # small integers: many exact ratios / ties
    xd = x.to(DEV, dtype)
    q, s = ops.quant_rowwise_i8(xd)
    if dtype == torch.bfloat16:
        qo, so = oracle.c_quant_rowwise_i8(bf16_bits(xd), bf16_bits=True)
    else:
        qo, so = oracle.c_quant_rowwise_i8(to_np(xd))
    assert np.array_equal(to_np(s).view(np.uint32), so.view(np.uint32))
    assert np.array_equal(to_np(q), qo)


def test_quant_rowwise_ties_and_strided_rows(oracle):
    # amax 127 -> scale exactly 1: n + 0.5 inputs are exact ties (half-to-even)
    row = torch.tensor([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, 64.5, 126.5, -126.5, 0.49999997,
                        3.5, -3.5, 100.5, 101.5])
    q, s = ops.quant_rowwise_i8(row[None].to(DEV))
    assert s.item() == 1.0
    assert to_np(q)[0].tolist() == [127, 0, 2, 2, 0, -2, -2, 64, 64, 126, -126, 0, 4, -4, 100, 102]
    # rows taken out of a wider matrix: ldx > K
    big = make_x(20, 96, seed=3).to(DEV)
    view = big[:, :64]
    from khaosz_amd import _abi
    q2 = torch.empty((20, 64), dtype=torch.int8, device=DEV)
    s2 = torch.empty((20,), dtype=torch.float32, device=DEV)
    rc = _abi.load().aq_quant_rowwise_i8(view.data_ptr(), 0, 20, 64, 96, q2.data_ptr(), s2.data_ptr(),
                                         torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    qo, so = oracle.c_quant_rowwise_i8(to_np(view.contiguous()))
    assert np.array_equal(to_np(q2), qo) and np.array_equal(to_np(s2), so)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_quant_rowwise_scale_range_and_dense_ties(oracle, dtype):
    """Rows whose scale sweeps the whole fp32 exponent range (the kernels switch to a full
    divide outside [2^-64, 2^64]: both sides and both borders are hit), each row dense in exact
    and near ties: multiples of amax/254 are half-integers after division by amax/127."""
    K = 2048
    exps = list(range(-140, 121, 4)) + [-64, -63, -65, 64, 63, 65, -71, -57, 57, 71]
    g = torch.Generator().manual_seed(11)
    rows = []
    for e in exps:
        amax = 127.0 * 2.0 ** e * (1.0 + 0.37 * torch.rand(1, generator=g).item())
        k = torch.randint(-254, 255, (K,), generator=g).double()
        r = (k * (amax / 254.0)).float()          # ties and integers in equal parts
        r[::3] = (torch.randn(K, generator=g).double()[::3] * (amax / 3.0)).clamp(-amax, amax).float()
        r[5] = amax
        rows.append(r)
    x = torch.stack(rows)
    x = x[torch.isfinite(x).all(dim=1)]
    xd = x.to(DEV, dtype)
    q, s_ = ops.quant_rowwise_i8(xd)
    if dtype == torch.bfloat16:
        qo, so = oracle.c_quant_rowwise_i8(bf16_bits(xd), bf16_bits=True)
    else:
        qo, so = oracle.c_quant_rowwise_i8(to_np(xd))
    assert np.array_equal(to_np(s_).view(np.uint32), so.view(np.uint32))
    bad = np.argwhere(to_np(q) != qo)
    assert bad.size == 0, f"first mismatches (row, col): {bad[:5].tolist()}"
    # the same rows through the decode kernel that quantises in-kernel (bf16, up to 8 rows a call)
    if dtype == torch.bfloat16:
        wq = torch.zeros((64, K), dtype=torch.int8)
        wq[torch.arange(64), torch.arange(64) * 31 % K] = 1      # y[m, n] = code of column 31n % K times sx
        sw = torch.ones(64)
        for r0 in range(0, xd.shape[0], 8):
            xs = xd[r0:r0 + 8].contiguous()
            y = ops.gemv_w8a8_decode(xs, wq.to(DEV), sw.to(DEV), None, out_dtype=torch.float32)
            want = qo[r0:r0 + 8][:, (np.arange(64) * 31) % K].astype(np.float32) * so[r0:r0 + 8, None]
            assert np.array_equal(to_np(y), want), f"rows {r0}.."


def _rows_of_every_value_up_to(amax_bits: int, K: int) -> np.ndarray:
    """bf16 bit patterns: rows of K values that begin with the maximum and together hold every bf16 number of
    magnitude up to it, both signs (the last row is filled up with zeros)."""
    mags = np.arange(amax_bits + 1, dtype=np.uint16)
    vals = np.concatenate([mags, mags | np.uint16(0x8000)])
    per = K - 1
    n_rows = (vals.size + per - 1) // per
    rows = np.zeros((n_rows, K), np.uint16)
    rows[:, 0] = amax_bits
    flat = np.zeros(n_rows * per, np.uint16)
    flat[:vals.size] = vals
    rows[:, 1:] = flat.reshape(n_rows, per)
    return rows


def test_bf16_rows_one_product_rounding_for_every_mantissa_of_the_maximum(oracle):
    """Rows of bf16 numbers are rounded with one product, value times a reciprocal of the scale that is moved
    by one unit in the last place for 24 of the 128 mantissas a row maximum can have.  Here: every mantissa, at
    three exponents (the choice must not depend on it), rows that hold EVERY bf16 value up to the maximum --
    through the row quantiser (rows of 8192 and of 2048 values: two kernels) against the oracle's divide."""
    for K in (8192, 2048):
        blocks = []
        for exp_field in ([127, 90, 170] if K == 8192 else [127]):
            for m in range(128):
                blocks.append(_rows_of_every_value_up_to((exp_field << 7) | m, K))
        bits = np.concatenate(blocks)
        _say("every value of bf16 rows", K, bits.shape)
        xd = torch.from_numpy(bits.view(np.int16)).to(DEV).view(torch.bfloat16)
        q, s_ = ops.quant_rowwise_i8(xd)
        qo, so = oracle.c_quant_rowwise_i8(bits, bf16_bits=True)
        assert np.array_equal(to_np(s_).view(np.uint32), so.view(np.uint32))
        bad = np.argwhere(to_np(q) != qo)
        assert bad.size == 0, f"K={K}: first mismatches (row, col): {bad[:5].tolist()}"
        del xd, q


def test_bf16_rows_one_product_rounding_inside_the_decode_kernels(oracle):
    """The same rows (every mantissa of the maximum, every value up to it) through the kernels that quantise
    their rows themselves: 16 rows a call through the matrix-core GEMV, 8 and 3 through the dot-product one.
    The weight is the identity, so the output is the codes times the row's scale, exactly."""
    K = 2048
    wq = torch.eye(K, dtype=torch.int8, device=DEV)
    sw = torch.ones(K, device=DEV)
    for m in range(128):
        bits = _rows_of_every_value_up_to((127 << 7) | m, K)
        qo, so = oracle.c_quant_rowwise_i8(bits, bf16_bits=True)
        want = qo.astype(np.float32) * so[:, None]
        xd = torch.from_numpy(bits.view(np.int16)).to(DEV).view(torch.bfloat16)
        for rows in (16, 8, 3):
            for r0 in range(0, xd.shape[0], rows):
                y = ops.gemv_w8a8_decode(xd[r0:r0 + rows].contiguous(), wq, sw, None, out_dtype=torch.float32)
                assert np.array_equal(to_np(y), want[r0:r0 + rows]), f"mantissa {m}, rows {r0}.. ({rows} a call)"


@pytest.mark.parametrize("M,K", [(1, 16), (7, 48), (5, 1040), (64, 2048), (8, 5632), (130, 4096), (3, 12288)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_quant_bit_exact(oracle, M, K, dtype):
    if dtype == torch.float32 and K > 6144:
        pytest.skip("fp32 rows longer than 6144 are outside the kernel's register budget")
    _say("rmsnorm_quant", M, K, dtype)
    g = torch.Generator().manual_seed(M * 13 + K)
    x = torch.randn(M, K, generator=g) * (0.05 + 5 * torch.rand(M, 1, generator=g))
    if M > 4:
        x[1] = 0                                   # zero row: eps keeps the root finite, codes 0
        x[2] *= 1e-18
        x[3] *= 1e12
    gamma = 1 + 0.2 * torch.randn(K, generator=g)
    xd, gd = x.to(DEV, dtype), gamma.to(DEV, dtype)
    q, s = ops.rmsnorm_quant_rowwise_i8(xd, gd, 1e-5)
    if dtype == torch.bfloat16:
        qo, so = oracle.c_rmsnorm_quant_i8(bf16_bits(xd), bf16_bits(gd), 1e-5, bf16_bits=True)
    else:
        qo, so = oracle.c_rmsnorm_quant_i8(to_np(xd), to_np(gd), 1e-5)
    assert np.array_equal(to_np(s).view(np.uint32), so.view(np.uint32))
    bad = np.argwhere(to_np(q) != qo)
    assert bad.size == 0, f"first mismatches (row, col): {bad[:5].tolist()}"


def test_rmsnorm_quant_tracks_torch_rms_norm_then_quantise():
    """Against the unfused flow (F.rms_norm, norm.py:14-15, then the row quantiser): the fused kernel
    skips the bf16 rounding of the normalised activations, so codes may differ by one step."""
    x = make_x(64, 2048, seed=9).to(DEV, torch.bfloat16)
    gamma = (1 + 0.1 * make_x(1, 2048, seed=10)[0]).to(DEV, torch.bfloat16)
    q, s = ops.rmsnorm_quant_rowwise_i8(x, gamma, 1e-5)
    q2, s2 = ops.quant_rowwise_i8(torch.nn.functional.rms_norm(x, (2048,), gamma, 1e-5))
    assert torch.allclose(s, s2, rtol=1e-2)
    d = (q.int() - q2.int()).abs()
    assert d.max().item() <= 1 and (d != 0).float().mean().item() < 0.2
    with pytest.raises(ValueError):
        ops.rmsnorm_quant_rowwise_i8(x, gamma.float(), 1e-5)       # gain in another dtype
    with pytest.raises(ValueError):
        ops.rmsnorm_quant_rowwise_i8(torch.zeros(2, 32768, device=DEV), torch.ones(32768, device=DEV), 1e-5)


@pytest.mark.parametrize("M,F", [(1, 16), (7, 48), (5, 1040), (64, 2048), (8, 5632), (130, 704), (1100, 1040), (4, 6912),
                                 (1030, 6912), (3, 8192),
                                 # many long rows (the workgroup-per-row kernel at prefill sizes; ragged row ends,
                                 # odd row counts)
                                 (1031, 8192), (1101, 6160), (4099, 6912), (1029, 3600), (1500, 3344)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu_quant_bit_exact(oracle, M, F, dtype):
    if dtype == torch.float32 and F > 4096:
        pytest.skip("fp32 rows longer than 4096 are outside the kernel's limit")
    _say("swiglu_quant", M, F, dtype)
    g = torch.Generator().manual_seed(M * 17 + F)
    ug = torch.randn(M, 2 * F, generator=g) * (0.05 + 6 * torch.rand(M, 1, generator=g))
    if M > 4:
        ug[1] = 0
        ug[2, F:] = -120.0           # gates below the exponential's clamp
        ug[3, F:] = 95.0             # and above it
        ug[4] *= 1e-20
    ud = ug.to(DEV, dtype)
    q, s = ops.swiglu_quant_rowwise_i8(ud)
    if dtype == torch.bfloat16:
        qo, so = oracle.c_swiglu_quant_i8(bf16_bits(ud), bf16_bits=True)
    else:
        qo, so = oracle.c_swiglu_quant_i8(to_np(ud))
    assert np.array_equal(to_np(s).view(np.uint32), so.view(np.uint32))
    bad = np.argwhere(to_np(q) != qo)
    assert bad.size == 0, f"first mismatches (row, col): {bad[:5].tolist()}"


@pytest.mark.parametrize("M,F", [(40, 5632), (40, 1040), (1100, 704), (1100, 6912), (1100, 3600)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu_quant_divide_range_edges(oracle, M, F, dtype):
    """The kernels take a short divide for rows whose gates are zero or in 2^-62 .. 80 and the general one for the
    rest: one special gate per row on either side of each bound (and zeros of both signs, a denormal, gates past
    the exponential's clamp), among ordinary values, must give the oracle's bits on both paths."""
    if dtype == torch.float32 and F > 4096:
        pytest.skip("fp32 rows longer than 4096 are outside the kernel's limit")
    _say("swiglu_quant edges", M, F, dtype)
    g = torch.Generator().manual_seed(M + F)
    ug = torch.randn(M, 2 * F, generator=g) * 1.5
    specials = [0.0, -0.0, 2.0 ** -62, -(2.0 ** -62), 2.0 ** -63, -(2.0 ** -63), 2.0 ** -100, 1e-39, -1e-39, 80.0, -80.0,
                80.5, -80.5, 31.9, 32.0, 88.0, -88.0, 1e30, -1e30, 2.0 ** -126, 3.0 * 2.0 ** -64]
    cols = torch.randint(0, F, (len(specials),), generator=g)
    for r, (v, c) in enumerate(zip(specials, cols.tolist())):
        ug[r, F + c] = v
    ug[len(specials), F:F + 64] = 0.0          # a run of zero gates
    ug[len(specials) + 1, :F] = 0.0            # up all zero: h = 0 whatever the gates
    ud = ug.to(DEV, dtype)
    q, s = ops.swiglu_quant_rowwise_i8(ud)
    if dtype == torch.bfloat16:
        qo, so = oracle.c_swiglu_quant_i8(bf16_bits(ud), bf16_bits=True)
    else:
        qo, so = oracle.c_swiglu_quant_i8(to_np(ud))
    assert np.array_equal(to_np(s).view(np.uint32), so.view(np.uint32))
    bad = np.argwhere(to_np(q) != qo)
    assert bad.size == 0, f"first mismatches (row, col): {bad[:5].tolist()}"


def _all_bf16_gates():
    """every bf16 pattern that is a finite number, as uint16"""
    pats = np.arange(65536, dtype=np.uint32)
    finite = ((pats >> 7) & 0xff) != 0xff
    return pats[finite].astype(np.uint16)


def test_swiglu_short_divide_is_the_oracles_divide_for_every_bf16_gate(oracle):
    """The row kernel's bf16 path divides g by 1 + exp(-g) with a sequence that is correctly rounded for this family
    of operands only.  The family has one member per gate: every finite bf16 gate pattern goes through the same
    arithmetic (lab probe: the header's functions, no clamp, short divide) against the oracle's product, which
    uses the true divide -- all gates the kernel's range test admits must agree bit for bit, with up = 1 (the
    quotient itself) and with other multipliers."""
    from khaosz_amd import _abi
    lab = _abi.load_lab()
    gates = _all_bf16_gates()
    n = gates.size
    gd = torch.from_numpy(gates.view(np.int16)).to(DEV)
    admitted = None
    for up_val in (1.0, -1.0, 0.9921875, 3.140625, 2.0 ** -20):
        up = torch.full((n,), up_val, dtype=torch.bfloat16)
        ub = bf16_bits(up)
        ud = torch.from_numpy(ub.view(np.int16)).to(DEV)
        h = torch.empty(n, dtype=torch.float32, device=DEV)
        ok = torch.empty(n, dtype=torch.uint8, device=DEV)
        rc = lab.aq_lab_probe_swiglu_bf16(ud.data_ptr(), gd.data_ptr(), n, h.data_ptr(), ok.data_ptr(),
                                          torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        torch.cuda.synchronize()
        ug = np.stack([ub, gates], axis=1).reshape(n, 2)          # rows of one product each: [up | gate]
        _, _, want = oracle.c_swiglu_quant_i8(ug, bf16_bits=True, want_h=True)
        got = to_np(h).view(np.uint32)
        okn = to_np(ok).astype(bool)
        admitted = okn
        gf = (gates.astype(np.uint32) << 16).view(np.float32)
        # the range test admits zero and 2^-62 <= |g| <= 80, nothing else
        assert np.array_equal(okn, (gf == 0) | ((np.abs(gf) >= 2.0 ** -62) & (np.abs(gf) <= 80.0)))
        w = want.reshape(n).view(np.uint32)
        zero = gf == 0                                           # 0 / d: the sign of a zero is free
        bad = np.flatnonzero(okn & ~zero & (got != w))
        assert bad.size == 0, [(hex(int(gates[i])), hex(int(got[i])), hex(int(w[i]))) for i in bad[:5]]
        assert np.all((got[zero] & 0x7fffffff) == 0)
    assert admitted.sum() > 17000                                # two signs x 68 binades x 128 mantissas, and the zeros


def test_swiglu_quant_kernel_scales_reveal_every_bf16_gates_quotient(oracle):
    """The same certification through the SHIPPED kernel: a row whose only non-zero product is 1 * silu(g) has
    amax = |silu(g)|, so its scale amax / 127 carries the quotient's bits (the map is one-to-one except where the
    quotient's mantissa is above 1.984; a second row with up = 127/128 covers those).  Every admitted gate, both
    multipliers, 5632-wide rows through the wavefront-per-row kernel."""
    gates = _all_bf16_gates()
    gf = (gates.astype(np.uint32) << 16).view(np.float32)
    gates = gates[(np.abs(gf) >= 2.0 ** -62) & (np.abs(gf) <= 80.0)]
    F = 5632
    for up_val in (1.0, 0.9921875):
        M = gates.size
        ug = np.zeros((M, 2 * F), np.uint16)
        col = (np.arange(M) * 37) % F
        ug[np.arange(M), col] = bf16_bits(torch.tensor([up_val], dtype=torch.bfloat16))[0]
        ug[np.arange(M), F + col] = gates
        for lo in range(0, M, 4096):                             # (the oracle's turn takes most of the time)
            part = np.ascontiguousarray(ug[lo:lo + 4096])
            d = torch.from_numpy(part.view(np.int16)).to(DEV).view(torch.bfloat16)
            q, s = ops.swiglu_quant_rowwise_i8(d)
            qo, so = oracle.c_swiglu_quant_i8(part, bf16_bits=True)
            assert np.array_equal(to_np(s).view(np.uint32), so.view(np.uint32)), (up_val, lo)
            assert np.array_equal(to_np(q), qo), (up_val, lo)


def test_swiglu_quant_tracks_the_unfused_flow():
    """Against silu, product and row quantiser as three launches (mlp.py:25-26 in bf16): the fused
    kernel keeps the product in fp32, so codes may differ by one step."""
    ug = make_x(64, 2 * 2048, seed=12).to(DEV, torch.bfloat16)
    q, s = ops.swiglu_quant_rowwise_i8(ug)
    up, gate = ug.chunk(2, dim=-1)
    q2, s2 = ops.quant_rowwise_i8(up * torch.nn.functional.silu(gate))
    assert torch.allclose(s, s2, rtol=2e-2)
    d = (q.int() - q2.int()).abs()
    assert d.max().item() <= 2 and (d != 0).float().mean().item() < 0.2


def test_quant_rowwise_empty():
    q, s = ops.quant_rowwise_i8(torch.empty((0, 32), device=DEV))
    assert q.shape == (0, 32) and s.shape == (0,)


# ---------------------------------------------------------------- int8 GEMM

GEMM_SHAPES = [(1, 1, 16), (37, 91, 48), (17, 5, 2048), (256, 128, 128), (257, 129, 144), (300, 200, 2064),
               (512, 384, 5632), (1000, 520, 1024)]


@pytest.fixture(params=[32, 33, 64, 65, 128, 129, 256])
def tile(request):
    """Run a GEMM test once per workgroup tile shape (the library would pick one by shape)."""
    with _abi.lab_library() as lab:  # the lab build of the same sources: its tile can be forced
        assert lab.aq_lab_set_gemm_tile(request.param) == 0
        yield request.param


def rand_codes(M, K, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8)


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
def test_gemm_i8_i32_bit_exact(oracle, tile, M, N, K):
    _say("gemm_i8_i32", M, N, K, tile)
    xq, wq = rand_codes(M, K, 1), rand_codes(N, K, 2)
    acc = ops.gemm_i8_i32(xq.to(DEV), wq.to(DEV))
    want = oracle.c_gemm_i8_i32(xq.numpy(), wq.numpy())
    assert np.array_equal(to_np(acc), want)


def test_gemm_with_more_tiles_than_compute_units(oracle, tile):
    """Beyond 256 tiles a workgroup walks several of them, reusing its LDS stages: 8200 x 1300 is 363
    tiles of 256 rows (two passes, the second partial) or 715 of 128 (three).  int32 sums, the fused
    epilogue with bias and residual, and the FP8 product, each against the oracle."""
    M, N, K = 8200, 1300, 144
    _say("gemm many tiles", M, N, K, tile)
    xq, wq = rand_codes(M, K, 11), rand_codes(N, K, 12)
    want = oracle.c_gemm_i8_i32(xq.numpy(), wq.numpy())
    assert np.array_equal(to_np(ops.gemm_i8_i32(xq.to(DEV), wq.to(DEV))), want)
    g = torch.Generator().manual_seed(13)
    sx, sw = torch.rand(M, generator=g) + 0.01, torch.rand(N, generator=g) * 0.01 + 1e-4
    bias = torch.randn(N, generator=g) * 0.01
    res = (torch.randn(M, N, generator=g) * 2).to(torch.bfloat16)
    y = ops.linear_w8a8(xq.to(DEV), sx.to(DEV), wq.to(DEV), sw.to(DEV), bias.to(DEV), out_dtype=torch.bfloat16)
    assert np.array_equal(bf16_bits(y), oracle.c_dequant_epilogue(want, sx.numpy(), sw.numpy(), bias.numpy(), bf16_out=True))
    y2 = ops.linear_w8a8(xq.to(DEV), sx.to(DEV), wq.to(DEV), sw.to(DEV), bias.to(DEV), out_dtype=torch.bfloat16,
                         residual=res.to(DEV))
    assert torch.equal(y2, y + res.to(DEV))
    # FP8 codes from two binades: every product and partial sum is exact in fp32, so the result does not
    # depend on the summation order or on the tile walk
    a8 = torch.randint(0x30, 0x40, (M, K), generator=g, dtype=torch.uint8)     # e4m3 values 0.5 .. 1.875
    b8 = torch.randint(0x30, 0x40, (N, K), generator=g, dtype=torch.uint8)
    one = torch.ones(1, device=DEV)
    y8 = ops.linear_fp8(a8.to(DEV), one, b8.to(DEV), one, out_dtype=torch.float32)
    ref = a8.view(torch.float8_e4m3fn).float() @ b8.view(torch.float8_e4m3fn).float().T
    assert torch.equal(y8.cpu(), ref)


PRODUCT_TILES = {256: "256 x 128", 128: "128 x 128", 64: "128 x 64", 32: "128 x 32", 65: "64 x 64", 33: "64 x 32"}


def _smallest_shape_for_tile(kind, cus):
    """The (M, N) of fewest outputs for which the library's own rule (a pure function, asked of the lab library;
    no GEMM runs there) picks tile `kind` on a device of `cus` compute units."""
    lab = _abi.load_lab()
    best = None
    for M in range(33, 2100, 7):
        for N in list(range(32, 2100, 32)) + [3072, 4096, 8192]:
            if lab.aq_lab_choose_gemm_tile(M, N, cus) == kind and (best is None or M * N < best[0] * best[1]):
                best = (M, N)
    return best


@pytest.mark.parametrize("kind", sorted(PRODUCT_TILES))
def test_every_product_tile_on_the_shipped_library(oracle, kind):
    """Each of the six tile shapes of libastrai_q.so (the tests above force tiles in the lab library, a separate
    compile of the same source): a shape for which the shipped library's rule picks that tile, run through the
    shipped library, int32 sums, fused epilogue and FP8 product against the oracle."""
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    shape = _smallest_shape_for_tile(kind, cus)
    assert shape is not None, f"no shape found for which the rule picks the {PRODUCT_TILES[kind]} tile"
    M, N = shape
    lib = _abi.load()
    assert lib is not _abi.load_lab() and not hasattr(lib, "aq_lab_set_gemm_tile")  # the product object does the work
    for K in (144, 256):  # ragged K steps, whole K steps
        _say("product tile", PRODUCT_TILES[kind], M, N, K)
        xq, wq = rand_codes(M, K, 301).numpy(), rand_codes(N, K, 302).numpy()
        want = oracle.c_gemm_i8_i32(xq, wq)
        acc = ops.gemm_i8_i32(torch.from_numpy(xq).to(DEV), torch.from_numpy(wq).to(DEV))
        assert np.array_equal(to_np(acc), want)
        g = np.random.default_rng(303)
        sx = (g.random(M) * 0.02 + 0.001).astype(np.float32)
        sw = (g.random(N) * 0.002 + 0.0001).astype(np.float32)
        b = (g.standard_normal(N) * 0.01).astype(np.float32)
        y = ops.linear_w8a8(torch.from_numpy(xq).to(DEV), torch.from_numpy(sx).to(DEV), torch.from_numpy(wq).to(DEV),
                            torch.from_numpy(sw).to(DEV), torch.from_numpy(b).to(DEV), out_dtype=torch.bfloat16)
        assert np.array_equal(bf16_bits(y), oracle.c_dequant_epilogue(want, sx, sw, b, bf16_out=True))
        yf = ops.linear_w8a8(torch.from_numpy(xq).to(DEV), torch.from_numpy(sx).to(DEV), torch.from_numpy(wq).to(DEV),
                             torch.from_numpy(sw).to(DEV), None, out_dtype=torch.float32)
        assert np.array_equal(to_np(yf).view(np.uint32),
                              oracle.c_dequant_epilogue(want, sx, sw, None, bf16_out=False).view(np.uint32))
        # FP8 codes from two binades: every product and partial sum is exact in fp32 (no order dependence)
        gt = torch.Generator().manual_seed(304)
        a8 = torch.randint(0x30, 0x40, (M, K), generator=gt, dtype=torch.uint8)
        b8 = torch.randint(0x30, 0x40, (N, K), generator=gt, dtype=torch.uint8)
        one = torch.ones(1, device=DEV)
        y8 = ops.linear_fp8(a8.to(DEV), one, b8.to(DEV), one, out_dtype=torch.float32)
        ref = a8.view(torch.float8_e4m3fn).float() @ b8.view(torch.float8_e4m3fn).float().T
        assert torch.equal(y8.cpu(), ref)


def test_product_fp8_256x256_tile(oracle):
    """FP8 launches of two rounds or more of 256 x 256 tiles take that tile in the shipped library (whole 256-row
    multiples, even N, whole 64-byte K steps, no residual).  Exact-in-fp32 operands against a float product, a
    random-data slab against the oracle within the FP8 tolerance, and the neighbouring shapes that must NOT take it
    (ragged M, a residual) against the same references."""
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    N, K = 2048 + 130, 192                      # ragged N (even), three K steps
    M = 256 * ((2 * cus + (N + 255) // 256 - 1) // ((N + 255) // 256))
    assert (M // 256) * ((N + 255) // 256) >= 2 * cus
    _say("product fp8 256x256", M, N, K)
    gt = torch.Generator().manual_seed(305)
    b8 = torch.randint(0x30, 0x40, (N, K), generator=gt, dtype=torch.uint8)
    one = torch.ones(1, device=DEV)
    for rows in (M, M + 3):                     # the 256 x 256 tile, and a ragged M that goes to another tile
        a8 = torch.randint(0x30, 0x40, (rows, K), generator=gt, dtype=torch.uint8)
        y8 = ops.linear_fp8(a8.to(DEV), one, b8.to(DEV), one, out_dtype=torch.float32)
        ref = a8.view(torch.float8_e4m3fn).float() @ b8.view(torch.float8_e4m3fn).float().T
        assert torch.equal(y8.cpu(), ref)
        yb = ops.linear_fp8(a8.to(DEV), one, b8.to(DEV), one, out_dtype=torch.bfloat16)
        assert torch.equal(yb.cpu(), ref.to(torch.bfloat16))
    # random data with real scales, a bias and bf16 output: a slab of rows against the oracle
    x = make_x(M, K, 306)
    w = make_x(N, K, 307) * 0.02
    xq, sx = ops.quant_tensor_fp8(x.to(DEV))
    wq, sw = ops.quant_tensor_fp8(w.to(DEV))
    bias = (torch.randn(N, generator=gt) * 0.01)
    y = ops.linear_fp8(xq, sx, wq, sw, out_dtype=torch.bfloat16, bias=bias.to(DEV))
    rows = slice(M - 40, M)
    want = oracle.c_linear_fp8(to_np(xq)[rows], float(to_np(sx)[0]), to_np(wq), float(to_np(sw)[0]), bf16_out=False,
                               bias=bias.numpy())
    got = y[rows].float().cpu().numpy()
    assert np.allclose(got, want, rtol=1e-2, atol=1e-2 * float(np.sqrt((want ** 2).mean())))


def test_lab_tile_256x256_on_shapes_it_takes(oracle):
    """The lab build's 256 x 256 tile (four wavefronts of 128 x 128, accumulators in AGPRs, per-row scales through
    LDS) takes whole 256-row multiples, even N and whole 64-byte K steps without a residual; anything else falls
    back to the 256 x 128 tile.  Same bits as the oracle on both routes, int8 sums, fused epilogue and FP8."""
    with _abi.lab_library() as lab:
        assert lab.aq_lab_set_gemm_tile(512) == 0
        for (M, N, K) in ((512, 768, 320), (256, 130, 64), (300, 256, 128), (512, 256, 80)):
            _say("tile 256x256", M, N, K)
            xq, wq = rand_codes(M, K, 91).numpy(), rand_codes(N, K, 92).numpy()
            acc = ops.gemm_i8_i32(torch.from_numpy(xq).to(DEV), torch.from_numpy(wq).to(DEV))
            assert np.array_equal(to_np(acc), oracle.c_gemm_i8_i32(xq, wq))
            g = np.random.default_rng(93)
            sx = (g.random(M) * 0.02 + 0.001).astype(np.float32)
            sw = (g.random(N) * 0.002 + 0.0001).astype(np.float32)
            b = (g.standard_normal(N) * 0.01).astype(np.float32)
            y = ops.linear_w8a8(torch.from_numpy(xq).to(DEV), torch.from_numpy(sx).to(DEV), torch.from_numpy(wq).to(DEV),
                                torch.from_numpy(sw).to(DEV), torch.from_numpy(b).to(DEV), out_dtype=torch.bfloat16)
            want = oracle.c_dequant_epilogue(oracle.c_gemm_i8_i32(xq, wq), sx, sw, b, bf16_out=True)
            assert np.array_equal(bf16_bits(y), want)
            x8, s8 = oracle.c_quant_tensor_fp8(make_x(M, K, 94).numpy())
            w8, t8 = oracle.c_quant_tensor_fp8((make_x(N, K, 95) * 0.02).numpy())
            y8 = ops.linear_fp8(torch.from_numpy(x8).to(DEV), torch.tensor([s8], device=DEV), torch.from_numpy(w8).to(DEV),
                                torch.tensor([t8], device=DEV), torch.from_numpy(b).to(DEV), out_dtype=torch.float32)
            exact = oracle.np_linear_fp8(x8, s8, w8, t8, bias=b)
            assert np.max(np.abs(to_np(y8) - exact)) <= 1e-3 * float(np.sqrt(np.mean(exact.astype(np.float64) ** 2)))


def test_gemm_i8_extremes(oracle, tile):
    K = 8192
    xq = torch.full((40, K), 127, dtype=torch.int8)
    wq = torch.full((33, K), -127, dtype=torch.int8)
    wq[::2] = 127
    acc = to_np(ops.gemm_i8_i32(xq.to(DEV), wq.to(DEV)))
    assert np.all(acc[:, ::2] == K * 127 * 127) and np.all(acc[:, 1::2] == -K * 127 * 127)


def test_gemm_i8_one_hot_pins_operand_order(tile):
    # xq has a single 1 at (m, k=m*3 % K); wq[n, k] = n*K + k small codes -> acc[m, n] = wq[n, k_m]
    M, N, K = 70, 45, 64
    xq = torch.zeros((M, K), dtype=torch.int8)
    ks = (torch.arange(M) * 3) % K
    xq[torch.arange(M), ks] = 1
    wq = ((torch.arange(N)[:, None] * 5 + torch.arange(K)[None, :] * 3) % 251 - 125).to(torch.int8)
    acc = to_np(ops.gemm_i8_i32(xq.to(DEV), wq.to(DEV)))
    want = wq.numpy().astype(np.int32)[:, ks.numpy()].T
    assert np.array_equal(acc, want)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("bias_kind", ["none", "f32", "bf16"])
@pytest.mark.parametrize("M,N,K", [(150, 200, 512), (77, 91, 144)])  # the second: odd N, rows not a multiple of 4
def test_linear_w8a8_epilogue_bit_exact(oracle, tile, M, N, K, out_dtype, bias_kind):
    _say("linear_w8a8", M, N, K, out_dtype, bias_kind, tile)
    x = make_x(M, K, 5, outlier_cols=3)
    w = make_x(N, K, 6) * 0.02
    xq, sx = oracle.c_quant_rowwise_i8(x.numpy())
    wq, sw = oracle.c_quant_rowwise_i8(w.numpy())
    bias = None
    bias_np = None
    if bias_kind != "none":
        b = torch.randn(N, generator=torch.Generator().manual_seed(7)) * 0.01
        bias = b.to(DEV, torch.float32 if bias_kind == "f32" else torch.bfloat16)
        bias_np = to_np(bias.float())
    y = ops.linear_w8a8(torch.from_numpy(xq).to(DEV), torch.from_numpy(sx).to(DEV), torch.from_numpy(wq).to(DEV),
                        torch.from_numpy(sw).to(DEV), bias, out_dtype=out_dtype)
    acc = oracle.c_gemm_i8_i32(xq, wq)
    if out_dtype == torch.float32:
        want = oracle.c_dequant_epilogue(acc, sx, sw, bias_np)
        assert np.array_equal(to_np(y).view(np.uint32), want.view(np.uint32))
    else:
        want = oracle.c_dequant_epilogue(acc, sx, sw, bias_np, bf16_out=True)
        assert np.array_equal(bf16_bits(y), want)
    # with a residual: the bits of the reference's separate add of the two tensors (decoder_block.py:56-57)
    r = (torch.randn(M, N, generator=torch.Generator().manual_seed(8)) * 2).to(DEV, out_dtype)
    y2 = ops.linear_w8a8(torch.from_numpy(xq).to(DEV), torch.from_numpy(sx).to(DEV), torch.from_numpy(wq).to(DEV),
                         torch.from_numpy(sw).to(DEV), bias, out_dtype=out_dtype, residual=r)
    assert torch.equal(y2, y + r)


def test_linear_residual_may_alias_the_output(tile):
    """x += linear(h): the residual pointer is the output pointer (GEMM and GEMV entry points)."""
    from khaosz_amd import _abi
    lib = _abi.load()
    for M in (200, 7):
        N, K = 384, 256
        g = torch.Generator().manual_seed(M)
        xq = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8).to(DEV)
        wq = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8).to(DEV)
        sx = (torch.rand(M, generator=g) * 1e-2 + 1e-3).to(DEV)
        sw = (torch.rand(N, generator=g) * 1e-2 + 1e-3).to(DEV)
        r = torch.randn(M, N, generator=g).to(DEV, torch.bfloat16)
        fn = ops.linear_w8a8 if M > 16 else ops.gemv_w8a8_codes
        want = fn(xq, sx, wq, sw, residual=r)
        assert torch.equal(want, fn(xq, sx, wq, sw) + r)
        y = r.clone()
        entry = lib.aq_linear_w8a8_residual if M > 16 else lib.aq_gemv_w8a8_codes_residual
        rc = entry(xq.data_ptr(), sx.data_ptr(), wq.data_ptr(), sw.data_ptr(), None, 0, y.data_ptr(), y.data_ptr(), 1,
                   M, N, K, None)
        torch.cuda.synchronize()
        assert rc == 0 and torch.equal(y, want)


# ------------------------------------------------------------------- decode

@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 8, 11, 16])
@pytest.mark.parametrize("N,K", [(8192, 2048), (50, 16), (130, 1040), (2048, 5632), (1536, 6912), (11264, 2048), (8200, 512), (77, 1536)])
def test_gemv_decode_bit_exact(oracle, M, N, K):
    """(11264, 2048), (8200, 512) and 9+ rows of (77, 1536) take the matrix-core kernel that quantises its rows
    itself: 64-row workgroups on the first (more 32-row blocks than compute units), a ragged last block on the
    second, a single partly filled workgroup on the third."""
    _say("gemv", M, N, K)
    x = make_x(M, K, 11 + M).to(torch.bfloat16)
    w = make_x(N, K, 12) * 0.02
    wq, sw = oracle.c_quant_rowwise_i8(w.numpy())
    b = (torch.randn(N, generator=torch.Generator().manual_seed(13)) * 0.01)
    for bias in (None, b):
        y = ops.gemv_w8a8_decode(x.to(DEV), torch.from_numpy(wq).to(DEV), torch.from_numpy(sw).to(DEV),
                                 None if bias is None else bias.to(DEV), out_dtype=torch.bfloat16)
        want = oracle.c_linear_w8a8(bf16_bits(x), wq, sw, None if bias is None else bias.numpy(),
                                    x_bf16_bits=True, bf16_out=True)
        assert np.array_equal(bf16_bits(y), want)
        r = (torch.randn(M, N, generator=torch.Generator().manual_seed(14)) * 2).to(DEV, torch.bfloat16)
        y2 = ops.gemv_w8a8_decode(x.to(DEV), torch.from_numpy(wq).to(DEV), torch.from_numpy(sw).to(DEV),
                                  None if bias is None else bias.to(DEV), out_dtype=torch.bfloat16, residual=r)
        assert torch.equal(y2, y + r)


@pytest.mark.parametrize("M", [1, 3, 4, 8, 12, 16])
@pytest.mark.parametrize("N,K", [(3072, 2048), (130, 1536), (2048, 4096), (50, 16), (11264, 2048), (8192, 1024)])
def test_gemv_with_the_norm_folded_in_equals_norm_quantise_then_gemv(oracle, M, N, K):
    """RMSNorm inside the decode GEMV (one launch for M <= 8, K <= 2048; two launches through the
    workspace otherwise): the codes are those of the stand-alone norm-and-quantise kernel, which is
    bit-exact against the oracle, so outputs must equal that kernel followed by the GEMV on codes."""
    _say("gemv+rmsnorm", M, N, K)
    g = torch.Generator().manual_seed(M * 31 + K)
    x = (torch.randn(M, K, generator=g) * (0.1 + 4 * torch.rand(M, 1, generator=g))).to(torch.bfloat16).to(DEV)
    gamma = (1 + 0.2 * torch.randn(K, generator=g)).to(torch.bfloat16).to(DEV)
    w = make_x(N, K, 12) * 0.02
    wq, sw = oracle.c_quant_rowwise_i8(w.numpy())
    wqd, swd = torch.from_numpy(wq).to(DEV), torch.from_numpy(sw).to(DEV)
    r = torch.randn(M, N, generator=g).to(torch.bfloat16).to(DEV)
    xq, sx = ops.rmsnorm_quant_rowwise_i8(x, gamma, 1e-5)
    qo, so = oracle.c_rmsnorm_quant_i8(bf16_bits(x), bf16_bits(gamma), 1e-5, bf16_bits=True)
    assert np.array_equal(to_np(xq), qo) and np.array_equal(to_np(sx).view(np.uint32), so.view(np.uint32))
    for res in (None, r):
        want = ops.gemv_w8a8_codes(xq, sx, wqd, swd, out_dtype=torch.bfloat16, residual=res)
        got = ops.gemv_w8a8_decode(x, wqd, swd, out_dtype=torch.bfloat16, residual=res, norm=(gamma, 1e-5))
        assert torch.equal(got, want)


@pytest.mark.parametrize("M,F,K,norm", [(8, 5632, 2048, True), (4, 6912, 1536, True), (16, 5632, 2048, False),
                                          (1, 48, 512, False), (11, 8208, 1024, True), (3, 2048, 2048, False)])
def test_up_gate_gemv_with_the_activation_in_its_epilogue_against_an_oracle_composition(oracle, M, F, K, norm):
    """up(x) * silu(gate(x)) as one launch at decode.  Composed on the CPU from the oracle's own functions: the
    row quantiser (with the RMSNorm in front when folded in), the int8 GEMM and its epilogue rounded to bf16 for
    both projections, the SwiGLU arithmetic on those bf16 values, one rounding to bf16.  Bit for bit, with and
    without a bias, for F below and above the device's count of 16-row blocks (both workgroup shapes) and F not a
    multiple of the workgroup's columns; and the same codes for `down` as the separate activation kernel would
    give when h is quantised afterwards."""
    _say("gemv+swiglu", M, F, K)
    g = torch.Generator().manual_seed(M * 131 + F)
    x = (torch.randn(M, K, generator=g) * (0.2 + 2 * torch.rand(M, 1, generator=g))).to(torch.bfloat16).to(DEV)
    gamma = (1 + 0.2 * torch.randn(K, generator=g)).to(torch.bfloat16).to(DEV)
    w = make_x(2 * F, K, 15) * 0.03
    wq, sw = oracle.c_quant_rowwise_i8(w.numpy())
    wqd, swd = torch.from_numpy(wq).to(DEV), torch.from_numpy(sw).to(DEV)
    bias = (torch.randn(2 * F, generator=g) * 0.05)
    if norm:
        xq, sx = oracle.c_rmsnorm_quant_i8(bf16_bits(x), bf16_bits(gamma), 1e-5, bf16_bits=True)
    else:
        xq, sx = oracle.c_quant_rowwise_i8(bf16_bits(x), bf16_bits=True)
    acc = oracle.c_gemm_i8_i32(xq, wq)
    assert ops.gemv_swiglu_ok(x, F)
    for b in (None, bias):
        ug = oracle.c_dequant_epilogue(acc, sx, sw, None if b is None else b.numpy(), bf16_out=True)  # bf16 bits [M, 2F]
        _, _, h = oracle.c_swiglu_quant_i8(ug, bf16_bits=True, want_h=True)
        want = oracle.np_f32_to_bf16_bits(h)
        got = ops.gemv_w8a8_decode_swiglu(x, wqd, swd, None if b is None else b.to(DEV), out_dtype=torch.bfloat16,
                                          norm=(gamma, 1e-5) if norm else None)
        assert got.shape == (M, F)
        assert np.array_equal(bf16_bits(got), want), int((bf16_bits(got) != want).sum())
    # fp32 output: the projections are not rounded in between
    ugf = oracle.c_dequant_epilogue(acc, sx, sw, None, bf16_out=False)
    _, _, hf = oracle.c_swiglu_quant_i8(ugf, want_h=True)
    gotf = ops.gemv_w8a8_decode_swiglu(x, wqd, swd, None, out_dtype=torch.float32, norm=(gamma, 1e-5) if norm else None)
    assert np.array_equal(to_np(gotf).view(np.uint32), hf.view(np.uint32))


def test_up_gate_gemv_with_the_activation_refuses_what_it_does_not_serve():
    x = torch.zeros(4, 4096, dtype=torch.bfloat16, device=DEV)  # rows too long for the in-kernel quantiser
    assert not ops.gemv_swiglu_ok(x, 1024)
    assert not ops.gemv_swiglu_ok(torch.zeros(4, 2048, dtype=torch.float32, device=DEV), 1024)  # fp32 rows
    assert not ops.gemv_swiglu_ok(torch.zeros(17, 2048, dtype=torch.bfloat16, device=DEV), 1024)
    assert not ops.gemv_swiglu_ok(torch.zeros(4, 2048, dtype=torch.bfloat16, device=DEV), 1000)  # F not a multiple of 16
    with pytest.raises(ValueError):
        ops.gemv_w8a8_decode_swiglu(x, torch.zeros(2048, 4096, dtype=torch.int8, device=DEV),
                                    torch.ones(2048, device=DEV))


@pytest.mark.parametrize("M", [17, 31, 32, 33, 48, 50, 64])
@pytest.mark.parametrize("N,K", [(8192, 2048), (200, 256), (77, 1536), (2048, 2304), (3072, 4096), (130, 9984),
                                 (2048, 5632), (8200, 6912), (77, 11008), (40, 128), (12000, 4224), (8400, 1024),
                                 (4200, 4224)])
def test_a_few_dozen_rows_same_bits_as_the_oracle(oracle, M, N, K):
    """17..32 rows: the Linear on codes hands them to the weight-streaming matrix-core kernel with 2 groups of
    16 tokens, which walks rows of any length (whole 128-byte lines) in chunks: 1024-byte chunks for short rows,
    2048 otherwise, 4096 for K >= 4096; 16, 32 or 64 rows per workgroup by the number of row blocks against the
    compute units; ragged last chunks, rows shorter than a chunk.  33..64 rows: the tiled GEMM, whose tile
    narrows to 128 x 64 or 128 x 32 for so few rows.  int32 sums and the frozen epilogue: bit for bit against the
    oracle, bf16 and fp32 outputs, with bias and residual, odd N."""
    _say("linear, few dozen rows", M, N, K)
    x = make_x(M, K, 50 + M).to(torch.bfloat16)
    w = make_x(N, K, 51) * 0.02
    wq, sw = oracle.c_quant_rowwise_i8(w.numpy())
    xq, sx = oracle.c_quant_rowwise_i8(bf16_bits(x), bf16_bits=True)
    g = torch.Generator().manual_seed(52)
    b = torch.randn(N, generator=g) * 0.01
    wqd, swd = torch.from_numpy(wq).to(DEV), torch.from_numpy(sw).to(DEV)
    xqd, sxd = torch.from_numpy(xq).to(DEV), torch.from_numpy(sx).to(DEV)
    acc = oracle.c_gemm_i8_i32(xq, wq)
    for bias in (None, b):
        want = oracle.c_dequant_epilogue(acc, sx, sw, None if bias is None else bias.numpy(), bf16_out=True)
        y = ops.linear_w8a8(xqd, sxd, wqd, swd, None if bias is None else bias.to(DEV), out_dtype=torch.bfloat16)
        assert np.array_equal(bf16_bits(y), want)
        r = torch.randn(M, N, generator=g).to(torch.bfloat16).to(DEV)
        yr = ops.linear_w8a8(xqd, sxd, wqd, swd, None if bias is None else bias.to(DEV), out_dtype=torch.bfloat16, residual=r)
        assert torch.equal(yr, y + r)
    wantf = oracle.c_dequant_epilogue(acc, sx, sw, b.numpy(), bf16_out=False)
    yf = ops.linear_w8a8(xqd, sxd, wqd, swd, b.to(DEV), out_dtype=torch.float32)
    assert np.array_equal(to_np(yf).view(np.uint32), wantf.view(np.uint32))
    rf = torch.randn(M, N, generator=g).to(DEV)
    assert torch.equal(ops.linear_w8a8(xqd, sxd, wqd, swd, b.to(DEV), out_dtype=torch.float32, residual=rf), yf + rf)


@pytest.mark.parametrize("M,K", [(12, 11008), (16, 14336), (7, 22016), (9, 10160)])
def test_decode_rows_too_long_for_the_gemv_take_the_kernel_that_walks_k_in_chunks(oracle, M, K):
    """Activation codes of 9..16 tokens fit a compute unit's LDS up to K = 10 096 (5..8 tokens: 20 208).
    Longer rows (FFN down projections of 11 008 or 14 336) must still work at decode batch sizes:
    the decode entry points hand them on to the Linear on codes, whose weight-streaming kernel walks such
    rows in chunks (rows that are not whole 128-byte lines would take the tiles).  Same bits as the oracle,
    with bias and residual, through the drop-in module as well."""
    N = 200
    _say("gemv long K", M, N, K)
    x = make_x(M, K, 41 + M).to(torch.bfloat16)
    w = make_x(N, K, 42) * 0.02
    wq, sw = oracle.c_quant_rowwise_i8(w.numpy())
    b = torch.randn(N, generator=torch.Generator().manual_seed(43)) * 0.01
    wqd, swd = torch.from_numpy(wq).to(DEV), torch.from_numpy(sw).to(DEV)
    want = oracle.c_linear_w8a8(bf16_bits(x), wq, sw, b.numpy(), x_bf16_bits=True, bf16_out=True)
    y = ops.gemv_w8a8_decode(x.to(DEV), wqd, swd, b.to(DEV), out_dtype=torch.bfloat16)
    assert np.array_equal(bf16_bits(y), want)
    r = torch.randn(M, N, generator=torch.Generator().manual_seed(44)).to(DEV, torch.bfloat16)
    assert torch.equal(ops.gemv_w8a8_decode(x.to(DEV), wqd, swd, b.to(DEV), out_dtype=torch.bfloat16, residual=r), y + r)
    xq, sx = ops.quant_rowwise_i8(x.to(DEV))
    assert torch.equal(ops.gemv_w8a8_codes(xq, sx, wqd, swd, b.to(DEV), out_dtype=torch.bfloat16), y)
    lin = Linear(K, N, bias=True)
    with torch.no_grad():
        lin.weight.copy_(w)
        lin.bias.copy_(b)
    q = QuantLinear.from_linear(lin.to(DEV))
    with torch.inference_mode():
        assert np.array_equal(bf16_bits(q(x.to(DEV))), want)


def test_gemv_f32_in_out_and_agrees_with_gemm_path(oracle):
    M, N, K = 16, 1000, 2048
    x = make_x(M, K, 21, outlier_cols=4)
    w = make_x(N, K, 22) * 0.02
    wq, sw = oracle.c_quant_rowwise_i8(w.numpy())
    wqd, swd = torch.from_numpy(wq).to(DEV), torch.from_numpy(sw).to(DEV)
    y = ops.gemv_w8a8_decode(x.to(DEV), wqd, swd, out_dtype=torch.float32)
    want = oracle.c_linear_w8a8(x.numpy(), wq, sw)
    assert np.array_equal(to_np(y).view(np.uint32), want.view(np.uint32))
    xq, sx = ops.quant_rowwise_i8(x.to(DEV))
    y2 = ops.linear_w8a8(xq, sx, wqd, swd, out_dtype=torch.float32)
    assert torch.equal(y, y2)
    r = torch.randn(M, N, generator=torch.Generator().manual_seed(23)).to(DEV)
    assert torch.equal(ops.gemv_w8a8_decode(x.to(DEV), wqd, swd, out_dtype=torch.float32, residual=r), y + r)
    assert torch.equal(ops.gemv_w8a8_codes(xq, sx, wqd, swd, out_dtype=torch.float32, residual=r), y + r)


# ---------------------------------------------------------------------- FP8

def test_quant_tensor_fp8_codes_bit_exact(oracle):
    tab = oracle.np_e4m3fn_table()[:127].astype(np.float64)
    mids = (tab[:-1] + tab[1:]) / 2
    rng = np.random.default_rng(31)
    base = np.concatenate([tab, -tab, mids, -mids, rng.uniform(-448, 448, 4096 - 506)]).astype(np.float32)
    assert base.size == 4096
    base[0] = 448.0  # amax == 448 -> scale exactly 1: inputs are cast as they are
    x = torch.from_numpy(base)
    q, s = ops.quant_tensor_fp8(x.to(DEV))
    qo, so = oracle.c_quant_tensor_fp8(base)
    assert s.item() == 1.0 == so
    assert np.array_equal(to_np(q), qo)
    # general scale, both input dtypes
    for dtype in (torch.float32, torch.bfloat16):
        xr = make_x(96, 512, 32).to(DEV, dtype)
        q, s = ops.quant_tensor_fp8(xr)
        if dtype == torch.bfloat16:
            qo, so = oracle.c_quant_tensor_fp8(bf16_bits(xr), bf16_bits=True)
        else:
            qo, so = oracle.c_quant_tensor_fp8(to_np(xr))
        assert np.float32(s.item()) == so
        assert np.array_equal(to_np(q), qo)
    q0, s0 = ops.quant_tensor_fp8(torch.zeros(4, 16, device=DEV))
    assert s0.item() == 1.0 and not to_np(q0).any()


@pytest.mark.parametrize("scale", [1.0, 0.37, 3.3e-3, 7.7e5, 1e-21, 1e-30, 3e25, 1e36])
def test_quant_tensor_fp8_scale_range_and_dense_midpoints(oracle, scale):
    """The cast kernel divides by the scale with a refined-reciprocal sequence that must equal the correctly
    rounded divide: inputs placed on and next to every e4m3 rounding midpoint (times the scale, one ulp either
    side), scales across the fp32 range (those outside [2^-64, 2^64] take the full divide), small and subnormal
    inputs.  Codes bit for bit against the oracle, fp32 and bf16 inputs; the GEMV's own cast gives the same codes."""
    tab = oracle.np_e4m3fn_table()[:127].astype(np.float64)
    mids = (tab[:-1] + tab[1:]) / 2
    pts = np.concatenate([tab, mids, -tab, -mids])
    s32 = np.float32(scale / 448.0) * np.float32(448.0)  # amax; the kernel's scale is amax / 448
    base = (pts * float(s32) / 448.0).astype(np.float32)
    near = np.concatenate([base, np.nextafter(base, np.float32(np.inf)), np.nextafter(base, np.float32(-np.inf))])
    rng = np.random.default_rng(61)
    rest = 4096 - near.size - 8
    tiny = np.array([1e-45, -1e-45, 1e-39, -3e-39, 0.0, -0.0, 1e-38, -1e-38], np.float32)
    x = np.concatenate([near, (rng.uniform(-1, 1, rest) * float(s32)).astype(np.float32), tiny]).astype(np.float32)
    x[0] = s32  # pins amax
    x = np.clip(x, -s32, s32)
    xd = torch.from_numpy(x).to(DEV)
    q, s = ops.quant_tensor_fp8(xd)
    qo, so = oracle.c_quant_tensor_fp8(x)
    assert np.float32(s.item()) == so
    assert np.array_equal(to_np(q), qo), int((to_np(q) != qo).sum())
    xb = xd.to(torch.bfloat16)
    qb, sb = ops.quant_tensor_fp8(xb)
    qbo, sbo = oracle.c_quant_tensor_fp8(bf16_bits(xb), bf16_bits=True)
    assert np.float32(sb.item()) == sbo and np.array_equal(to_np(qb), qbo)
    # the same rows through the GEMV that casts them itself: against the GEMV on the quantiser's codes
    if 1e-15 < scale < 1e15:
        rows = xb.view(2, 2048)
        w8, t8 = ops.quant_tensor_fp8(torch.randn(96, 2048, device=DEV) * 0.02)
        fused = ops.gemv_fp8_decode(rows, w8, t8, out_dtype=torch.float32)
        codes = ops.gemv_fp8_codes(qb.view(2, 2048), sb, w8, t8, out_dtype=torch.float32)
        ref = float(codes.abs().mean())
        assert float((fused - codes).abs().max()) <= 2e-5 * max(ref, 1e-30)


def test_quant_tensor_fp8_one_launch_form_same_codes_and_scale(oracle):
    """The one-launch per-tensor quantiser (partial maxima exchanged between the workgroups while the kernel runs,
    the tensor held in registers in between) against the oracle and the two-launch form, bit for bit: sizes from
    one vector to more than the registers hold (the rest is read again), both input types, calls in a row on ONE
    state tensor with sizes going up and down (the state a call leaves is what the next one starts from), the
    scale-setting element in the first, the last and a middle workgroup's share, a zero tensor."""
    state = ops.fp8_onepass_state(DEV)
    g = torch.Generator(device=DEV).manual_seed(77)
    cases = [(16, torch.float32), (4096, torch.bfloat16), (1 << 20, torch.bfloat16), (48, torch.float32),
             ((5 << 20) + 16 * 7, torch.float32), (20 << 20, torch.bfloat16), (256 * 1024 * 8 - 16, torch.bfloat16), (16, torch.bfloat16)]
    for n, dt in cases:
        x = (torch.randn(n, generator=g, device=DEV) * 0.3).to(dt)
        for where in (0, n // 2 + 3, n - 1):
            xx = x.clone()
            xx[where] = -7.25  # the element that sets the scale: first, middle or last share
            q, s = ops.quant_tensor_fp8(xx, state=state, onepass=True)
            q2, s2 = ops.quant_tensor_fp8(xx)
            assert s.item() == s2.item() == np.float32(7.25) / np.float32(448.0), (n, dt, where)
            assert torch.equal(q, q2), (n, dt, where)
        if n <= (1 << 20):
            if dt == torch.bfloat16:
                qo, so = oracle.c_quant_tensor_fp8(bf16_bits(xx), bf16_bits=True)
            else:
                qo, so = oracle.c_quant_tensor_fp8(to_np(xx))
            assert np.float32(s.item()) == so and np.array_equal(to_np(q), qo)
    q0, s0 = ops.quant_tensor_fp8(torch.zeros(64, 16, device=DEV), state=state, onepass=True)
    assert s0.item() == 1.0 and not to_np(q0).any()
    # the register-resident limit of this device: a tensor of 40 MiB takes the second-read path for its tail
    big = (torch.randn(20 << 20, generator=g, device=DEV) * 2).to(torch.bfloat16)
    q, s = ops.quant_tensor_fp8(big, state=state, onepass=True)
    q2, s2 = ops.quant_tensor_fp8(big)
    assert s.item() == s2.item() and torch.equal(q, q2)
    with pytest.raises(ValueError):
        ops.quant_tensor_fp8(big, onepass=True)  # no state
    with pytest.raises(ValueError):
        ops.quant_tensor_fp8(big, state=torch.zeros(8, dtype=torch.int64, device=DEV), onepass=True)  # too small


def test_quant_tensor_fp8_one_launch_form_when_the_workgroups_do_not_wait(oracle):
    """A device that cannot run all workgroups at once would leave them waiting for each other: the wait is bounded
    and a workgroup that gives up takes the whole tensor's maximum itself.  Forced here from the host by a bound of
    zero polls (lab build): same codes and scale, and the state it leaves is good for an ordinary call."""
    from khaosz_amd import _abi
    lab = _abi.load_lab()
    state = ops.fp8_onepass_state(DEV)
    g = torch.Generator(device=DEV).manual_seed(78)
    st = torch.cuda.current_stream().cuda_stream
    for n, dt, code in ((1 << 18, torch.bfloat16, _abi.AQ_BF16), (3 * 4096 + 16, torch.float32, _abi.AQ_F32)):
        x = (torch.randn(n, generator=g, device=DEV) * 0.1).to(dt)
        q = torch.empty(n, dtype=torch.uint8, device=DEV)
        s = torch.empty(1, dtype=torch.float32, device=DEV)
        for spin in (0, 1):
            rc = lab.aq_lab_quant_tensor_fp8_onepass_spin(x.data_ptr(), code, n, q.data_ptr(), s.data_ptr(),
                                                          state.data_ptr(), state.numel() * 8, spin, st)
            assert rc == 0
            q2, s2 = ops.quant_tensor_fp8(x)
            assert s.item() == s2.item() and torch.equal(q, q2), (n, dt, spin)
        q3, s3 = ops.quant_tensor_fp8(x, state=state, onepass=True)
        assert s3.item() == s2.item() and torch.equal(q3, q2)


def test_quant_tensor_fp8_one_launch_form_in_a_replayed_graph():
    """Its state lives in device memory and moves on by itself, so a captured call can be replayed: three calls on
    different inputs captured once, replayed five times with eager calls on the same state in between, every
    replay's codes and scales equal to the two-launch form's."""
    state = ops.fp8_onepass_state(DEV)
    g = torch.Generator(device=DEV).manual_seed(79)
    xs = [(torch.randn(512, 2048, generator=g, device=DEV) * (i + 1)).to(torch.bfloat16) for i in range(3)]
    want = [ops.quant_tensor_fp8(x) for x in xs]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for x in xs:
            ops.quant_tensor_fp8(x, state=state, onepass=True)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            outs = [ops.quant_tensor_fp8(x, state=state, onepass=True) for x in xs]
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for r in range(5):
        for q, s in outs:
            q.zero_()
            s.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for (q, s), (qw, sw) in zip(outs, want):
            assert s.item() == sw.item() and torch.equal(q, qw), r
        qe, se = ops.quant_tensor_fp8(xs[r % 3], state=state, onepass=True)  # eager work on the same state in between
        assert se.item() == want[r % 3][1].item() and torch.equal(qe, want[r % 3][0])


@pytest.mark.parametrize("M,N,K", [(1, 1, 16), (33, 70, 144), (256, 128, 1024), (300, 260, 2048), (64, 96, 8192)])
def test_linear_fp8_within_tolerance(oracle, tile, M, N, K):
    _say("linear_fp8", M, N, K)
    x = make_x(M, K, 41)
    w = make_x(N, K, 42) * 0.02
    xq, sx = oracle.c_quant_tensor_fp8(x.numpy())
    wq, sw = oracle.c_quant_tensor_fp8(w.numpy())
    args = (torch.from_numpy(xq).to(DEV), torch.tensor([sx], device=DEV), torch.from_numpy(wq).to(DEV),
            torch.tensor([sw], device=DEV))
    exact = oracle.np_linear_fp8(xq, sx, wq, sw)  # float64 accumulation of the decoded codes
    rms = float(np.sqrt(np.mean(exact.astype(np.float64) ** 2)))
    y32 = to_np(ops.linear_fp8(*args, out_dtype=torch.float32))
    # fp32 accumulation inside the matrix core (products aligned to the largest exponent before they are
    # summed) lands within ~1e-4 of the exact sum: ten times inside the stated 1e-2, while a wrong code
    # table or a dropped k-slice is far outside
    assert np.max(np.abs(y32 - exact)) <= 1e-3 * max(rms, 1e-30)
    yb = to_np(ops.linear_fp8(*args, out_dtype=torch.bfloat16).float())
    np.testing.assert_allclose(yb, exact, rtol=1e-2, atol=1e-2 * rms)  # stated tolerance: 1e-2 relative in bf16
    yc = oracle.c_linear_fp8(xq, sx, wq, sw)
    np.testing.assert_allclose(y32, yc, rtol=1e-2, atol=1e-3 * rms)
    # bias (fp32 and bf16) and residual in the epilogue: the bias inside the stated tolerance of the oracle
    # with a bias, the residual the bits of a separate add
    g = torch.Generator().manual_seed(43)
    for bias in (torch.randn(N, generator=g) * 0.5, (torch.randn(N, generator=g) * 0.5).to(torch.bfloat16)):
        want = oracle.np_linear_fp8(xq, sx, wq, sw, bias=bias.float().numpy())
        got32 = ops.linear_fp8(*args, bias.to(DEV), out_dtype=torch.float32)
        assert np.max(np.abs(to_np(got32) - want)) <= 1e-3 * max(rms, 0.5)
        np.testing.assert_allclose(to_np(got32), oracle.c_linear_fp8(xq, sx, wq, sw, bias=bias.float().numpy()),
                                   rtol=1e-2, atol=1e-3 * max(rms, 0.5))
        for dt in (torch.float32, torch.bfloat16):
            plain = ops.linear_fp8(*args, bias.to(DEV), out_dtype=dt)
            r = torch.randn(M, N, generator=g).to(dt).to(DEV)
            assert torch.equal(ops.linear_fp8(*args, bias.to(DEV), out_dtype=dt, residual=r), plain + r)
            y_in_place = r.clone()   # the residual may be the output buffer itself
            rc = _abi.load().aq_linear_fp8_residual(args[0].data_ptr(), args[1].data_ptr(), args[2].data_ptr(),
                                                    args[3].data_ptr(), None, 0, y_in_place.data_ptr(),
                                                    y_in_place.data_ptr(), 1 if dt == torch.bfloat16 else 0, M, N, K,
                                                    torch.cuda.current_stream().cuda_stream)
            assert rc == 0 and torch.equal(y_in_place, ops.linear_fp8(*args, out_dtype=dt) + r)


@pytest.mark.parametrize("M", [17, 32, 33, 50, 64])
@pytest.mark.parametrize("N,K", [(8192, 2048), (77, 512), (3072, 1536), (200, 256), (8400, 2304), (130, 4096),
                                 (8400, 1024), (300, 5632), (4200, 4224)])
def test_linear_fp8_a_few_dozen_rows(oracle, M, N, K):
    """17..32 rows of FP8 codes (whole 128-byte lines) go to the weight-streaming kernel (one 16x16x128 product
    per 128-byte line and token group, fp32 sums, chunks and K parts added in a fixed order), in every chunk and
    workgroup shape of its dispatch; 33..64 rows to the narrow tiles.  Against the float64 sum of the oracle's codes inside the stated
    tolerance, against the tiled GEMM on the same codes (a forced tile shape keeps it on the tiles) within the
    change of summation order, with bias and residual, and the same bits on a second call."""
    _say("linear_fp8, few dozen rows", M, N, K)
    x = make_x(M, K, 61 + M).to(torch.bfloat16)
    w = make_x(N, K, 62) * 0.02
    xq, sx = oracle.c_quant_tensor_fp8(bf16_bits(x), bf16_bits=True)
    wq, sw = oracle.c_quant_tensor_fp8(w.numpy())
    g = torch.Generator().manual_seed(63)
    bias = torch.randn(N, generator=g) * 0.3
    args = (torch.from_numpy(xq).to(DEV), torch.tensor([sx], device=DEV), torch.from_numpy(wq).to(DEV),
            torch.tensor([sw], device=DEV))
    exact = oracle.np_linear_fp8(xq, sx, wq, sw, bias=bias.numpy())
    rms = float(np.sqrt(np.mean(exact.astype(np.float64) ** 2)))
    y32 = ops.linear_fp8(*args, bias.to(DEV), out_dtype=torch.float32)
    assert np.max(np.abs(to_np(y32) - exact)) <= 1e-3 * rms
    assert torch.equal(ops.linear_fp8(*args, bias.to(DEV), out_dtype=torch.float32), y32)
    yb = ops.linear_fp8(*args, bias.to(DEV), out_dtype=torch.bfloat16)
    np.testing.assert_allclose(to_np(yb.float()), exact, rtol=1e-2, atol=1e-2 * rms)   # stated tolerance
    np.testing.assert_allclose(to_np(y32), oracle.c_linear_fp8(xq, sx, wq, sw, bias=bias.numpy()), rtol=1e-2,
                               atol=1e-3 * rms)
    nb = ops.linear_fp8(*args, out_dtype=torch.float32)
    assert np.max(np.abs(to_np(nb) - oracle.np_linear_fp8(xq, sx, wq, sw))) <= 1e-3 * rms
    for dt, plain in ((torch.float32, y32), (torch.bfloat16, yb)):
        r = torch.randn(M, N, generator=g).to(dt).to(DEV)
        assert torch.equal(ops.linear_fp8(*args, bias.to(DEV), out_dtype=dt, residual=r), plain + r)
    with _abi.lab_library() as lab:
        assert lab.aq_lab_set_gemm_tile(128) == 0
        yt = ops.linear_fp8(*args, bias.to(DEV), out_dtype=torch.float32)
    assert np.max(np.abs(to_np(yt) - to_np(y32))) <= 2e-5 * rms


@pytest.mark.parametrize("M", [1, 3, 8, 9, 16])
@pytest.mark.parametrize("N,K", [(8192, 2048), (77, 512), (11264, 1024), (300, 4096), (130, 1040), (200, 11008)])
def test_gemv_fp8_decode_within_tolerance(oracle, M, N, K):
    """The FP8 Linear at decode sizes: (8192, 2048), (77, 512) and (11264, 1024) cast their bf16 rows inside the
    GEMV kernel (32- and 64-row workgroups, a ragged single workgroup); (300, 4096) goes through the workspace
    (quantiser + GEMV on codes); (130, 1040) is handed to the tiled GEMM; rows of 11008 codes are too long for the
    GEMV's LDS and go to the Linear on codes (its weight-streaming kernel from 9 rows on).  All against the float64 sum of the
    oracle's codes, and the fused cast against the codes path (a wrong code would move an output by far more
    than a change of summation order)."""
    _say("gemv_fp8", M, N, K)
    g = torch.Generator().manual_seed(M * 13 + N)
    x = (torch.randn(M, K, generator=g) * (0.2 + 3 * torch.rand(M, 1, generator=g))).to(torch.bfloat16)
    w = make_x(N, K, 52) * 0.02
    xq, sx = oracle.c_quant_tensor_fp8(bf16_bits(x), bf16_bits=True)
    wq, sw = oracle.c_quant_tensor_fp8(w.numpy())
    bias = torch.randn(N, generator=g) * 0.3
    wqd, swd = torch.from_numpy(wq).to(DEV), torch.tensor([sw], device=DEV)
    exact = oracle.np_linear_fp8(xq, sx, wq, sw, bias=bias.numpy())
    rms = float(np.sqrt(np.mean(exact.astype(np.float64) ** 2)))
    y32 = ops.gemv_fp8_decode(x.to(DEV), wqd, swd, bias.to(DEV), out_dtype=torch.float32)
    assert np.max(np.abs(to_np(y32) - exact)) <= 1e-3 * rms
    yb = ops.gemv_fp8_decode(x.to(DEV), wqd, swd, bias.to(DEV), out_dtype=torch.bfloat16)
    np.testing.assert_allclose(to_np(yb.float()), exact, rtol=1e-2, atol=1e-2 * rms)   # stated tolerance
    # the library's own quantiser gives the oracle's codes; the GEMV on them agrees with the fused launch
    xqd, sxd = ops.quant_tensor_fp8(x.to(DEV))
    assert np.array_equal(to_np(xqd), xq) and float(sxd.item()) == float(sx)
    yc = ops.gemv_fp8_codes(xqd, sxd, wqd, swd, bias.to(DEV), out_dtype=torch.float32)
    assert np.max(np.abs(to_np(yc) - to_np(y32))) <= 2e-5 * rms
    # and with the tiled GEMM on the same codes
    yg = ops.linear_fp8(xqd, sxd, wqd, swd, bias.to(DEV), out_dtype=torch.float32)
    assert np.max(np.abs(to_np(yg) - to_np(y32))) <= 2e-5 * rms
    r = torch.randn(M, N, generator=g).to(torch.bfloat16).to(DEV)
    assert torch.equal(ops.gemv_fp8_decode(x.to(DEV), wqd, swd, bias.to(DEV), out_dtype=torch.bfloat16, residual=r), yb + r)


def test_fp8_linear_module_decode_rows_take_the_gemv_and_match_the_prefill_path():
    torch.manual_seed(9)
    lin = Linear(2048, 512)
    lin.reset_parameters()
    f = Fp8Linear.from_linear(lin.to(DEV))
    x = torch.randn(40, 2048, device=DEV, dtype=torch.bfloat16)
    with torch.inference_mode():
        big = f(x)                                   # 40 rows: quantiser + tiled GEMM, one scale for all 40
        small = f(x[:16])                            # 16 rows: the GEMV, one scale for these 16
    ref = torch.nn.functional.linear(x.float(), lin.weight)
    assert ((big.float() - ref).norm() / ref.norm()).item() < 0.08
    assert ((small.float() - ref[:16]).norm() / ref[:16].norm()).item() < 0.08


def test_fp8_linear_module_large_input_takes_the_one_launch_quantiser_same_bits():
    """From 16 MiB of activations Fp8Linear quantises them in one launch (its per-stream state is created on first
    use and carried from call to call): the output must be the bits of the two-launch quantiser + the same GEMM,
    call after call, and on a second stream with a state of its own."""
    torch.manual_seed(10)
    lin = Linear(2048, 256)
    lin.reset_parameters()
    f = Fp8Linear.from_linear(lin.to(DEV))
    xs = [torch.randn(4096, 2048, device=DEV, dtype=torch.bfloat16) * (i + 1) for i in range(2)]  # 16 MiB each
    assert xs[0].numel() * 2 >= ops.FP8_ONEPASS_MIN_BYTES
    with torch.inference_mode():
        want = []
        for x in xs:
            xq, sx = ops.quant_tensor_fp8(x)
            want.append(ops.linear_fp8(xq, sx, f.qweight, f.w_scale, None, out_dtype=torch.bfloat16))
        for rep in range(3):
            for x, w in zip(xs, want):
                assert torch.equal(f(x), w), rep
        assert len(f._quant_states) == 1
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            got = f(xs[1])
        side.synchronize()
        assert torch.equal(got, want[1]) and len(f._quant_states) == 2


def test_fp8_linear_module_with_a_bias_and_a_residual(oracle):
    """Fp8Linear keeps the reference's optional bias (linear.py:11) and takes the residual stream like QuantLinear."""
    torch.manual_seed(8)
    lin = Linear(256, 96, bias=True)
    lin.reset_parameters()
    lin = lin.to(DEV)
    f = Fp8Linear.from_linear(lin)
    assert torch.equal(f.bias, lin.bias) and set(f.state_dict()) == {"qweight", "w_scale", "bias"}
    x = torch.randn(3, 20, 256, device=DEV, dtype=torch.bfloat16)
    r = torch.randn(3, 20, 96, device=DEV, dtype=torch.bfloat16)
    with torch.inference_mode():
        y = f(x)
        assert torch.equal(f(x, residual=r), y + r)
    xq, sx = oracle.c_quant_tensor_fp8(bf16_bits(x.reshape(60, 256)), bf16_bits=True)
    want = oracle.np_linear_fp8(xq, sx, to_np(f.qweight), float(f.w_scale.item()), bias=to_np(lin.bias.detach()))
    np.testing.assert_allclose(to_np(y.float()).reshape(60, 96), want, rtol=1e-2, atol=1e-2 * float(np.abs(want).mean()))
    ref = torch.nn.functional.linear(x.float(), lin.weight, lin.bias)
    assert ((y.float() - ref).norm() / ref.norm()).item() < 0.08
    g = Fp8Linear(256, 96, bias=True, device=DEV)
    g.load_state_dict(f.state_dict())
    with torch.inference_mode():
        assert torch.equal(g(x), y)


def test_linear_fp8_one_hot_pins_operand_order(oracle, tile):
    M, N, K = 40, 35, 128
    tab = oracle.np_e4m3fn_table()
    xq = np.zeros((M, K), np.uint8)
    ks = (np.arange(M) * 5) % K
    xq[np.arange(M), ks] = 0x38  # 1.0
    wq = ((np.arange(N)[:, None] * 7 + np.arange(K)[None, :] * 3) % 120).astype(np.uint8)
    y = to_np(ops.linear_fp8(torch.from_numpy(xq).to(DEV), torch.tensor([1.0], device=DEV),
                             torch.from_numpy(wq).to(DEV), torch.tensor([1.0], device=DEV), out_dtype=torch.float32))
    assert np.array_equal(y, tab[wq][:, ks].T)


# -------------------------------------------------------------- module level

def test_config1_quant_linear_matches_oracle_and_float_reference(oracle):
    """benchmark configuration 1: X 64x2048 fp32 with 4 outlier columns x20, W 2048x2048 N(0, 0.02)."""
    g = torch.Generator().manual_seed(0)
    x = torch.randn(64, 2048, generator=g)
    cols = torch.randperm(2048, generator=g)[:4]
    x[:, cols] *= 20
    w = torch.randn(2048, 2048, generator=g) * 0.02
    lin = Linear(2048, 2048)
    with torch.no_grad():
        lin.weight.copy_(w)
    lin = lin.to(DEV)
    q = QuantLinear.from_linear(lin)
    wq, sw = oracle.c_quant_rowwise_i8(w.numpy())
    assert np.array_equal(to_np(q.qweight), wq) and np.array_equal(to_np(q.w_scale), sw)
    with torch.inference_mode():
        y = q(x.to(DEV))
    want = oracle.c_linear_w8a8(x.numpy(), wq, sw)
    assert np.array_equal(to_np(y).view(np.uint32), want.view(np.uint32))
    ref = torch.nn.functional.linear(x, w).numpy()  # the reference's real path, linear.py:21
    rel = np.linalg.norm(to_np(y) - ref) / np.linalg.norm(ref)
    assert rel < 8e-2, rel


def test_quant_linear_module_shapes_dispatch_and_state_dict(oracle):
    torch.manual_seed(1)
    lin = Linear(256, 192, bias=True)
    lin.reset_parameters()
    lin = lin.to(DEV)
    q = QuantLinear.from_linear(lin)
    assert isinstance(q, Linear)
    x3 = torch.randn(2, 20, 256, device=DEV, dtype=torch.bfloat16)   # M = 40 -> MFMA path
    xd = x3[:, :8].contiguous()                                       # M = 16 -> decode path
    with torch.inference_mode():
        y3 = q(x3)
        yd = q(xd)
    assert y3.shape == (2, 20, 192) and y3.dtype == torch.bfloat16
    assert torch.equal(yd, y3[:, :8])  # per-token quantisation: both paths give identical rows
    ref = torch.nn.functional.linear(x3.float(), lin.weight, lin.bias)
    assert (y3.float() - ref).norm() / ref.norm() < 3e-2
    # float checkpoints with the reference's key names load into the quantized module
    q2 = QuantLinear(256, 192, bias=True, device=DEV)
    q2.load_state_dict({"weight": lin.weight.detach(), "bias": lin.bias.detach()})
    assert torch.equal(q2.qweight, q.qweight) and torch.equal(q2.w_scale, q.w_scale)
    q3 = QuantLinear(256, 192, bias=True, device=DEV)
    q3.load_state_dict(q.state_dict())
    with torch.inference_mode():
        assert torch.equal(q3(x3), y3)
    with pytest.raises(RuntimeError, match="forward-only"):
        q(torch.randn(4, 256, device=DEV, requires_grad=True))


def test_called_from_a_daemon_thread_on_a_side_stream():
    """How the reference's serving loop calls Linear (a daemon thread under inference_mode,
    scheduler.py:191-196, executor.py:48,81): the work must go to that thread's current stream and
    give the bits of a main-thread call; two threads on two streams share one module."""
    import threading

    torch.manual_seed(2)
    lin = Linear(512, 320, bias=True)
    lin.reset_parameters()
    q = QuantLinear.from_linear(lin.to(DEV))
    xs = [torch.randn(m, 512, device=DEV, dtype=torch.bfloat16) for m in (4, 100)]   # decode and prefill paths
    with torch.inference_mode():
        want = [q(x) for x in xs]
    torch.cuda.synchronize()
    got, errs = {}, []

    def worker(name):
        try:
            s = torch.cuda.Stream()
            with torch.inference_mode(), torch.cuda.stream(s):
                for _ in range(20):
                    ys = [q(x) for x in xs]
                s.synchronize()  # the launches went to this thread's stream: waiting for it alone is enough
                got[name] = [y.clone() for y in ys]
        except Exception as e:  # surfaced in the main thread
            errs.append(e)

    ts = [threading.Thread(target=worker, args=(i,), daemon=True) for i in range(2)]
    [t.start() for t in ts]
    [t.join(60) for t in ts]
    assert not errs, errs
    for i in range(2):
        assert torch.equal(got[i][0], want[0]) and torch.equal(got[i][1], want[1])


def test_quantize_model_on_gpu_preserves_outputs_within_quantisation_error():
    import torch.nn as nn

    class MLP(nn.Module):  # the reference's MLP shape: down(up(x) * silu(gate(x))), mlp.py:24-27
        def __init__(self):
            super().__init__()
            self.up, self.gate, self.down = Linear(128, 352), Linear(128, 352), Linear(352, 128)

        def forward(self, x):
            return self.down(self.up(x) * torch.nn.functional.silu(self.gate(x)))

    torch.manual_seed(2)
    m = MLP()
    for l in (m.up, m.gate, m.down):
        l.reset_parameters()
    m = m.to(DEV)
    x = torch.randn(4, 33, 128, device=DEV)
    with torch.inference_mode():
        ref = m(x)
        assert quantize_model(m) == 3
        y = m(x)
        assert (y - ref).norm() / ref.norm() < 5e-2
        f = MLP().to(DEV)
        f.load_state_dict({k: v for k, v in zip(["up.weight", "gate.weight", "down.weight"],
                                                [m.up.weight, m.gate.weight, m.down.weight])})
        assert quantize_model(f, mode="fp8") == 3 and isinstance(f.up, Fp8Linear)
        yf = f(x)
        assert (yf - ref).norm() / ref.norm() < 0.12


# ------------------------------------------- full-size, size-independent checks

def test_full_size_prefill_checksum_of_checksums(oracle):
    """benchmark configuration 3 at full size (M=4096, K=N=2048, 1 % outlier channels x10)."""
    M, N, K = 4096, 2048, 2048
    x = make_x(M, K, 51, outlier_cols=20, outlier_gain=10.0).to(torch.bfloat16).to(DEV)
    w = (make_x(N, K, 52) * 0.02).to(DEV)
    xq, sx = ops.quant_rowwise_i8(x)
    wq, sw = ops.quant_rowwise_i8(w)
    assert int(xq.abs().amax(1).min()) == 127 and int(wq.abs().amax(1).min()) == 127
    acc = ops.gemm_i8_i32(xq, wq)
    # sum over all outputs == dot of the column sums (exact in int64)
    lhs = int(acc.sum(dtype=torch.int64))
    rhs = int((xq.sum(0, dtype=torch.int64) * wq.sum(0, dtype=torch.int64)).sum())
    assert lhs == rhs
    # row / column checksums against int64 matvecs
    ones_n = wq.sum(0, dtype=torch.int64).double()
    assert torch.equal(acc.sum(1, dtype=torch.int64), (xq.double() @ ones_n).long())
    ones_m = xq.sum(0, dtype=torch.int64).double()
    assert torch.equal(acc.sum(0, dtype=torch.int64), (wq.double() @ ones_m).long())
    # a slab of rows against the oracle, bit for bit, through the fused epilogue
    bias = (torch.randn(N, generator=torch.Generator().manual_seed(53)) * 0.01).to(DEV)
    y = ops.linear_w8a8(xq, sx, wq, sw, bias, out_dtype=torch.bfloat16)
    rows = slice(1900, 2200)
    want = oracle.c_dequant_epilogue(oracle.c_gemm_i8_i32(to_np(xq[rows]), to_np(wq)), to_np(sx[rows]), to_np(sw),
                                     to_np(bias), bf16_out=True)
    assert np.array_equal(bf16_bits(y[rows]), want)
    # permuting the tokens permutes the output rows
    perm = torch.randperm(M, generator=torch.Generator().manual_seed(54)).to(DEV)
    y2 = ops.linear_w8a8(xq[perm].contiguous(), sx[perm].contiguous(), wq, sw, bias, out_dtype=torch.bfloat16)
    assert torch.equal(y2, y[perm])


def test_full_size_fp8_linearity_in_scales(oracle):
    """benchmark configuration 4 at full size (M=2048, K=8192, N=2048)."""
    M, N, K = 2048, 2048, 8192
    x = make_x(M, K, 61).to(torch.bfloat16).to(DEV)
    w = (make_x(N, K, 62) * 0.02).to(DEV)
    xq, sx = ops.quant_tensor_fp8(x)
    wq, sw = ops.quant_tensor_fp8(w)
    assert int(xq.max()) >= 0x7E or int((xq & 0x7F).max()) == 0x7E  # amax lands on 448
    y = ops.linear_fp8(xq, sx, wq, sw, out_dtype=torch.float32)
    y2 = ops.linear_fp8(xq, sx * 2, wq, sw * 4, out_dtype=torch.float32)
    assert torch.equal(y2, y * 8)  # power-of-two scales commute with rounding
    rows = slice(700, 740)
    exact = oracle.np_linear_fp8(to_np(xq[rows]), sx.item(), to_np(wq), sw.item())
    rms = float(np.sqrt(np.mean(exact.astype(np.float64) ** 2)))
    assert np.max(np.abs(to_np(y[rows]) - exact)) <= 1e-3 * rms
    ref = torch.nn.functional.linear(x[rows].float(), w)
    assert ((y[rows] - ref).norm() / ref.norm()).item() < 0.06
