"""CPU oracle of the quantized-Linear path -- TEST INFRASTRUCTURE ONLY.

Only tests/, the smoke check and the benchmark's cpu_baseline leg may import
this module; the product (khaosz_amd) never does.

Two independent restatements of the same frozen arithmetic live here so that
each can check the other:

* ``np_*``  -- numpy, vectorised, float32 everywhere it matters;
* ``c_*``   -- the C file ``aq_oracle.c`` through ctypes (fast enough for the
  benchmark-size parity cases and the timed CPU baseline).

The float Linear that both are measured against is the reference's
``F.linear(x, weight, bias)`` (astrai/model/components/linear.py:20-21) with
``weight`` laid out ``[out_dim, in_dim]`` (linear.py:10).  The reference has no
quantized arithmetic; the closed forms are documented at the top of
``aq_oracle.c`` together with what pins each function.
"""
from __future__ import annotations

import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libaq_oracle.so")
_lib = None

F32 = np.float32


# --------------------------------------------------------------------------
# bf16 / e4m3fn scalar formats (numpy)
# --------------------------------------------------------------------------

def np_f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit pattern (uint16), round to nearest even."""
    u = np.ascontiguousarray(x, dtype=F32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def np_bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(F32)


def np_e4m3fn_table() -> np.ndarray:
    """All 256 e4m3fn codes decoded to fp32 (0x7f / 0xff are NaN)."""
    codes = np.arange(256, dtype=np.int64)
    sign = np.where(codes >= 128, -1.0, 1.0)
    e = (codes >> 3) & 0xF
    m = codes & 7
    sub = m * 2.0 ** -9
    nor = (8 + m) * 2.0 ** (e - 10.0)
    v = np.where(e == 0, sub, nor) * sign
    v[(e == 15) & (m == 7)] = np.nan
    return v.astype(F32)


def np_f32_to_e4m3fn(x: np.ndarray) -> np.ndarray:
    """fp32 -> e4m3fn code, round to nearest even, saturating at +-448.

    Implemented as a nearest-code search on the sorted table of the 127
    non-negative finite values, so it shares no logic with the C version's
    frexp-based rounding.
    """
    x = np.ascontiguousarray(x, dtype=F32)
    a = np.abs(x).astype(np.float64)
    pos = np_e4m3fn_table()[:127].astype(np.float64)  # codes 0x00..0x7e ascending
    hi = np.searchsorted(pos, a, side="left")  # first code with value >= a
    hi = np.clip(hi, 0, 126)
    lo = np.clip(hi - 1, 0, 126)
    d_hi = np.abs(pos[hi] - a)
    d_lo = np.abs(a - pos[lo])
    pick_lo = (d_lo < d_hi) | ((d_lo == d_hi) & (lo % 2 == 0))
    code = np.where(pick_lo, lo, hi).astype(np.uint8)
    code = np.where(np.isnan(x), np.uint8(0x7F), code)
    sign = (x.view(np.uint32) >> 24).astype(np.uint8) & np.uint8(0x80)
    return (code | sign).astype(np.uint8)


# --------------------------------------------------------------------------
# numpy restatement of the path
# --------------------------------------------------------------------------

def np_quant_rowwise_i8(x: np.ndarray):
    """Symmetric absmax int8 per row of a 2-D fp32 array -> (codes int8, scale f32)."""
    x = np.ascontiguousarray(x, dtype=F32)
    amax = np.max(np.abs(x), axis=1).astype(F32) if x.shape[1] else np.zeros(x.shape[0], F32)
    s = (amax / F32(127.0)).astype(F32)
    s = np.where(amax == 0, F32(1.0), s).astype(F32)
    q = np.rint((x / s[:, None]).astype(F32))
    q = np.clip(q, -127, 127).astype(np.int8)
    return q, s


def np_rmsnorm(x: np.ndarray, gamma: np.ndarray, eps: float, epv: int) -> np.ndarray:
    """y = x * (1 / sqrt(mean(x^2) + eps)) * gamma in fp32 with the fixed summation order of
    the C oracle: 64 stripes of ``epv``-element vectors, then an xor butterfly."""
    x = np.ascontiguousarray(x, dtype=F32)
    gamma = np.ascontiguousarray(gamma, dtype=F32)
    M, K = x.shape
    nvec = K // epv
    pad = (-nvec) % 64
    sq = (x * x).astype(F32).reshape(M, nvec, epv)
    if pad:
        sq = np.concatenate([sq, np.zeros((M, pad, epv), F32)], axis=1)
    sq = sq.reshape(M, -1, 64, epv)            # [M, round, stripe, element]
    p = np.zeros((M, 64), F32)
    for rnd in range(sq.shape[1]):
        for e in range(epv):
            p = (p + sq[:, rnd, :, e]).astype(F32)
    idx = np.arange(64)
    off = 1
    while off < 64:
        p = (p + p[:, idx ^ off]).astype(F32)
        off <<= 1
    mean = (p[:, 0] / F32(K)).astype(F32)
    r = (F32(1.0) / np.sqrt((mean + F32(eps)).astype(F32)).astype(F32)).astype(F32)
    return ((x * r[:, None]).astype(F32) * gamma[None, :]).astype(F32)


def np_rmsnorm_quant_i8(x: np.ndarray, gamma: np.ndarray, eps: float, epv: int):
    return np_quant_rowwise_i8(np_rmsnorm(x, gamma, eps, epv))


def _fma32(a, b, c):
    """fp32 fused multiply-add on arrays: the product of two fp32 values is exact in float64, and
    the float64 sum is rounded once more to fp32; the double rounding can only matter when the
    float64 sum lands exactly on an fp32 midpoint, which the callers' tests would show."""
    return (a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64)).astype(F32)


def np_exp_repro(x: np.ndarray) -> np.ndarray:
    x = np.clip(np.asarray(x, F32), F32(-87.0), F32(87.0)).astype(F32)
    n = np.rint((x * F32(1.44269504088896341)).astype(F32)).astype(F32)
    r = _fma32(n, np.full_like(n, F32(-0.693359375)), x)
    r = _fma32(n, np.full_like(n, F32(2.12194440e-4)), r)
    p = np.full_like(r, F32(1.9875691500e-4))
    for c in (1.3981999507e-3, 8.3334519073e-3, 4.1665795894e-2, 1.6666665459e-1, 5.0000001201e-1):
        p = _fma32(p, r, np.full_like(r, F32(c)))
    y = (_fma32(p, (r * r).astype(F32), r) + F32(1.0)).astype(F32)
    return (y.view(np.int32) + (n.astype(np.int32) << 23)).view(F32)


def np_swiglu(u: np.ndarray, g: np.ndarray) -> np.ndarray:
    u, g = np.asarray(u, F32), np.asarray(g, F32)
    d = (F32(1.0) + np_exp_repro(-g)).astype(F32)
    return (u * (g / d).astype(F32)).astype(F32)


def np_gemm_i8_i32(xq: np.ndarray, wq: np.ndarray) -> np.ndarray:
    acc = xq.astype(np.int64) @ wq.astype(np.int64).T
    assert np.all(np.abs(acc) < 2 ** 31)
    return acc.astype(np.int32)


def np_dequant_epilogue(acc, sx, sw, bias=None) -> np.ndarray:
    t = (acc.astype(F32) * sx.astype(F32)[:, None]).astype(F32)
    y = (t * sw.astype(F32)[None, :]).astype(F32)
    if bias is not None:
        y = (y + bias.astype(F32)[None, :]).astype(F32)
    return y


def np_linear_w8a8(x, wq, sw, bias=None) -> np.ndarray:
    xq, sx = np_quant_rowwise_i8(x)
    return np_dequant_epilogue(np_gemm_i8_i32(xq, wq), sx, sw, bias)


def np_quant_tensor_fp8(x: np.ndarray):
    x = np.ascontiguousarray(x, dtype=F32)
    amax = F32(np.max(np.abs(x))) if x.size else F32(0)
    s = F32(1.0) if amax == 0 else F32(amax / F32(448.0))
    v = np.clip((x / s).astype(F32), F32(-448.0), F32(448.0))
    return np_f32_to_e4m3fn(v), s


def np_linear_fp8(xq, sx, wq, sw, bias=None) -> np.ndarray:
    """Float64 accumulation of the decoded codes: the 'true' value the fp32
    accumulating implementations are held to within tolerance."""
    lut = np_e4m3fn_table().astype(np.float64)
    acc = lut[xq] @ lut[wq].T
    y = (acc * float(sx)) * float(sw)
    if bias is not None:
        y = y + np.asarray(bias, np.float64)[None, :]
    return y.astype(F32)


def np_linear_f32(x, w, bias=None) -> np.ndarray:
    y = x.astype(np.float64) @ w.astype(np.float64).T
    if bias is not None:
        y = y + bias.astype(np.float64)
    return y.astype(F32)


# --------------------------------------------------------------------------
# C oracle through ctypes
# --------------------------------------------------------------------------

def _load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        from . import build_oracle  # type: ignore

        build_oracle.build()
    lib = ctypes.CDLL(_LIB_PATH)
    i64, vp = ctypes.c_int64, ctypes.c_void_p
    lib.oq_num_threads.restype = ctypes.c_int
    lib.oq_set_num_threads.argtypes = [ctypes.c_int]
    lib.oq_bf16_to_f32.restype = ctypes.c_float
    lib.oq_bf16_to_f32.argtypes = [ctypes.c_uint16]
    lib.oq_f32_to_bf16.restype = ctypes.c_uint16
    lib.oq_f32_to_bf16.argtypes = [ctypes.c_float]
    lib.oq_e4m3fn_to_f32.restype = ctypes.c_float
    lib.oq_e4m3fn_to_f32.argtypes = [ctypes.c_uint8]
    lib.oq_f32_to_e4m3fn.restype = ctypes.c_uint8
    lib.oq_f32_to_e4m3fn.argtypes = [ctypes.c_float]
    lib.oq_quant_rowwise_i8_f32.argtypes = [vp, i64, i64, i64, vp, vp]
    lib.oq_quant_rowwise_i8_bf16.argtypes = [vp, i64, i64, i64, vp, vp]
    lib.oq_rmsnorm_quant_i8_f32.argtypes = [vp, vp, ctypes.c_float, i64, i64, i64, vp, vp, vp]
    lib.oq_rmsnorm_quant_i8_bf16.argtypes = [vp, vp, ctypes.c_float, i64, i64, i64, vp, vp, vp]
    lib.oq_swiglu_quant_i8_f32.argtypes = [vp, i64, i64, i64, vp, vp, vp]
    lib.oq_swiglu_quant_i8_bf16.argtypes = [vp, i64, i64, i64, vp, vp, vp]
    lib.oq_exp_repro.argtypes = [ctypes.c_float]
    lib.oq_exp_repro.restype = ctypes.c_float
    lib.oq_rope_kv_write.argtypes = [vp, vp, vp, i64, i64, i64, vp, vp, i64, vp, i64, i64, i64, i64]
    lib.oq_rope_kv_write_qknorm.argtypes = [vp, vp, vp, i64, i64, i64, vp, vp, i64, vp, i64, i64, i64, i64, vp, vp,
                                            ctypes.c_float]
    lib.oq_paged_attn_decode.argtypes = [vp, vp, vp, vp, i64, i64, vp, i64, i64, ctypes.c_float, vp, i64, i64, i64, i64]
    lib.oq_prefill_attn_causal.argtypes = [vp, vp, vp, ctypes.c_float, vp, i64, i64, i64, i64, i64]
    lib.oq_prefill_attn_offset.argtypes = [vp, vp, vp, ctypes.c_float, vp, i64, i64, i64, i64, i64, i64]
    lib.oq_gemm_i8_i32.argtypes = [vp, vp, vp, i64, i64, i64]
    lib.oq_dequant_epilogue.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64]
    lib.oq_linear_w8a8_f32.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64]
    lib.oq_linear_w8a8_bf16.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64]
    lib.oq_quant_tensor_fp8_f32.argtypes = [vp, i64, vp, vp]
    lib.oq_quant_tensor_fp8_bf16.argtypes = [vp, i64, vp, vp]
    lib.oq_one_step_divide_mismatches.argtypes = [ctypes.c_float, ctypes.c_int, ctypes.c_uint32, ctypes.c_uint32, vp]
    lib.oq_one_step_divide_mismatches.restype = ctypes.c_int64
    lib.oq_linear_fp8.argtypes = [vp, ctypes.c_float, vp, ctypes.c_float, vp, vp, vp, i64, i64, i64]
    lib.oq_linear_f32.argtypes = [vp, vp, vp, vp, i64, i64, i64]
    for name in (
        "oq_set_num_threads oq_quant_rowwise_i8_f32 oq_quant_rowwise_i8_bf16 oq_gemm_i8_i32 "
        "oq_dequant_epilogue oq_linear_w8a8_f32 oq_linear_w8a8_bf16 oq_quant_tensor_fp8_f32 "
        "oq_quant_tensor_fp8_bf16 oq_linear_fp8 oq_linear_f32 oq_rmsnorm_quant_i8_f32 oq_rmsnorm_quant_i8_bf16 "
        "oq_swiglu_quant_i8_f32 oq_swiglu_quant_i8_bf16 oq_rope_kv_write oq_paged_attn_decode oq_prefill_attn_causal "
        "oq_rope_kv_write_qknorm "
        "oq_prefill_attn_offset"
    ).split():
        getattr(lib, name).restype = None
    _lib = lib
    return lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


def c_num_threads() -> int:
    return int(_load().oq_num_threads())


def c_set_num_threads(n: int) -> None:
    _load().oq_set_num_threads(int(n))


def c_f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    lib = _load()
    flat = _c(x, F32).ravel()
    return np.array([lib.oq_f32_to_bf16(float(v)) for v in flat], dtype=np.uint16).reshape(np.shape(x))


def c_f32_to_e4m3fn(x: np.ndarray) -> np.ndarray:
    lib = _load()
    flat = _c(x, F32).ravel()
    return np.array([lib.oq_f32_to_e4m3fn(ctypes.c_float(v)) for v in flat], dtype=np.uint8).reshape(np.shape(x))


def c_e4m3fn_table() -> np.ndarray:
    lib = _load()
    return np.array([lib.oq_e4m3fn_to_f32(i) for i in range(256)], dtype=F32)


def c_quant_rowwise_i8(x: np.ndarray, bf16_bits: bool = False):
    """x: [M,K] fp32, or uint16 bf16 bit patterns when ``bf16_bits``."""
    lib = _load()
    x = _c(x, np.uint16 if bf16_bits else F32)
    M, K = x.shape
    q = np.empty((M, K), np.int8)
    s = np.empty((M,), F32)
    fn = lib.oq_quant_rowwise_i8_bf16 if bf16_bits else lib.oq_quant_rowwise_i8_f32
    fn(_p(x), M, K, K, _p(q), _p(s))
    return q, s


def c_rmsnorm_quant_i8(x: np.ndarray, gamma: np.ndarray, eps: float, bf16_bits: bool = False, want_y: bool = False):
    """x: [M,K] and gamma: [K], fp32 or (``bf16_bits``) uint16 bf16 patterns -> (codes, scale[, y fp32])."""
    lib = _load()
    dt = np.uint16 if bf16_bits else F32
    x, gamma = _c(x, dt), _c(gamma, dt)
    M, K = x.shape
    assert gamma.shape == (K,)
    q = np.empty((M, K), np.int8)
    s = np.empty((M,), F32)
    y = np.empty((M, K), F32) if want_y else None
    fn = lib.oq_rmsnorm_quant_i8_bf16 if bf16_bits else lib.oq_rmsnorm_quant_i8_f32
    fn(_p(x), _p(gamma), ctypes.c_float(eps), M, K, K, _p(q), _p(s), _p(y) if want_y else None)
    return (q, s, y) if want_y else (q, s)


def c_swiglu_quant_i8(ug: np.ndarray, bf16_bits: bool = False, want_h: bool = False):
    """ug: [M, 2F] = [up | gate], fp32 or (``bf16_bits``) uint16 bf16 patterns -> (codes [M,F], scale[, h fp32])."""
    lib = _load()
    ug = _c(ug, np.uint16 if bf16_bits else F32)
    M, F2 = ug.shape
    Fh = F2 // 2
    q = np.empty((M, Fh), np.int8)
    s = np.empty((M,), F32)
    h = np.empty((M, Fh), F32) if want_h else None
    fn = lib.oq_swiglu_quant_i8_bf16 if bf16_bits else lib.oq_swiglu_quant_i8_f32
    fn(_p(ug), M, Fh, F2, _p(q), _p(s), _p(h) if want_h else None)
    return (q, s, h) if want_h else (q, s)


def np_head_rmsnorm_bits(x_bits: np.ndarray, gain_bits: np.ndarray, eps: float) -> np.ndarray:
    """RMSNorm over the last axis of bf16 head vectors ``[..., D]`` (D a power of two times 8) as the
    qk-norm kernels do it: squares summed per 8 elements in memory order, the chunk sums pairwise over
    the chunk index; ``bf16((x * r) * gain)``.  Bit patterns in and out."""
    x = np_bf16_bits_to_f32(x_bits)
    D = x.shape[-1]
    sq = (x * x).astype(F32).reshape(*x.shape[:-1], D // 8, 8)
    part = np.zeros(sq.shape[:-1], F32)
    for e in range(8):
        part = (part + sq[..., e]).astype(F32)
    while part.shape[-1] > 1:
        part = (part[..., 0::2] + part[..., 1::2]).astype(F32)
    mean = (part / F32(D)).astype(F32)
    r = (F32(1.0) / np.sqrt((mean + F32(eps)).astype(F32)).astype(F32)).astype(F32)
    y = ((x * r).astype(F32) * np_bf16_bits_to_f32(gain_bits)).astype(F32)
    return np_f32_to_bf16_bits(y)


def c_rope_kv_write(qkv, freqs, table, pos, kc, vc, Hq, Hkv, qk_norm=None):
    """bf16 bit patterns (uint16) throughout; kc / vc [n_pages, page, Hkv, D] are updated in place.
    Returns the rotated q [B, Hq, D].  ``qk_norm = (q_gain bits [D], k_gain bits [D], eps)``: the
    rotated q and k heads are RMS-normalised over D (attention.py:86-89)."""
    lib = _load()
    qkv, freqs, table = _c(qkv, np.uint16), _c(freqs, F32), _c(table, np.int64)
    assert kc.dtype == np.uint16 and vc.dtype == np.uint16 and kc.flags.c_contiguous and vc.flags.c_contiguous
    B = qkv.shape[0]
    n_pages, page, _, D = kc.shape
    q = np.empty((B, Hq, D), np.uint16)
    if qk_norm is None:
        lib.oq_rope_kv_write(_p(qkv), _p(freqs), _p(table), table.shape[1], pos, page, _p(kc), _p(vc), n_pages, _p(q),
                             B, Hq, Hkv, D)
    else:
        qg, kg = _c(qk_norm[0], np.uint16), _c(qk_norm[1], np.uint16)
        assert qg.shape == (D,) and kg.shape == (D,)
        lib.oq_rope_kv_write_qknorm(_p(qkv), _p(freqs), _p(table), table.shape[1], pos, page, _p(kc), _p(vc), n_pages,
                                    _p(q), B, Hq, Hkv, D, _p(qg), _p(kg), float(qk_norm[2]))
    return q


def c_paged_attn_decode(q, kc, vc, table, total_len, scale, seq_lens=None):
    """seq_lens [B] (optional): positions at and past seq_lens[b] are masked for sequence b as the reference's
    position mask does (transformer.py:40-46)."""
    lib = _load()
    q, kc, vc, table = _c(q, np.uint16), _c(kc, np.uint16), _c(vc, np.uint16), _c(table, np.int64)
    B, Hq, D = q.shape
    n_pages, page, Hkv, _ = kc.shape
    out = np.empty((B, Hq, D), np.uint16)
    lens = None if seq_lens is None else _c(seq_lens, np.int64)
    lib.oq_paged_attn_decode(_p(q), _p(kc), _p(vc), _p(table), table.shape[1], total_len,
                             None if lens is None else _p(lens), page, n_pages,
                             ctypes.c_float(scale), _p(out), B, Hq, Hkv, D)
    return out


def c_prefill_attn_causal(q, k, v, scale):
    """q [B, S, Hq, D], k / v [B, S, Hkv, D] as uint16 bf16 patterns -> out [B, S, Hq, D] (uint16)."""
    lib = _load()
    q, k, v = _c(q, np.uint16), _c(k, np.uint16), _c(v, np.uint16)
    B, S, Hq, D = q.shape
    Hkv = k.shape[2]
    out = np.empty((B, S, Hq, D), np.uint16)
    lib.oq_prefill_attn_causal(_p(q), _p(k), _p(v), ctypes.c_float(scale), _p(out), B, S, Hq, Hkv, D)
    return out


def c_prefill_attn_offset(q, k, v, start, scale):
    """q [B, S, Hq, D] at positions start .. start + S, k / v [B, start + S, Hkv, D] (uint16 bf16 patterns)
    -> out [B, S, Hq, D] (uint16)."""
    lib = _load()
    q, k, v = _c(q, np.uint16), _c(k, np.uint16), _c(v, np.uint16)
    B, S, Hq, D = q.shape
    assert k.shape[1] == start + S and k.shape == v.shape
    out = np.empty((B, S, Hq, D), np.uint16)
    lib.oq_prefill_attn_offset(_p(q), _p(k), _p(v), ctypes.c_float(scale), _p(out), B, S, int(start), Hq, k.shape[2], D)
    return out


def c_gemm_i8_i32(xq: np.ndarray, wq: np.ndarray) -> np.ndarray:
    lib = _load()
    xq, wq = _c(xq, np.int8), _c(wq, np.int8)
    M, K = xq.shape
    N, K2 = wq.shape
    assert K == K2
    acc = np.empty((M, N), np.int32)
    lib.oq_gemm_i8_i32(_p(xq), _p(wq), _p(acc), M, N, K)
    return acc


def c_dequant_epilogue(acc, sx, sw, bias=None, bf16_out: bool = False) -> np.ndarray:
    lib = _load()
    acc, sx, sw = _c(acc, np.int32), _c(sx, F32), _c(sw, F32)
    bias = None if bias is None else _c(bias, F32)
    M, N = acc.shape
    y = np.empty((M, N), np.uint16 if bf16_out else F32)
    lib.oq_dequant_epilogue(_p(acc), _p(sx), _p(sw), _p(bias), None if bf16_out else _p(y),
                            _p(y) if bf16_out else None, M, N)
    return y


def c_linear_w8a8(x, wq, sw, bias=None, x_bf16_bits: bool = False, bf16_out: bool = False) -> np.ndarray:
    lib = _load()
    x = _c(x, np.uint16 if x_bf16_bits else F32)
    wq, sw = _c(wq, np.int8), _c(sw, F32)
    bias = None if bias is None else _c(bias, F32)
    M, K = x.shape
    N = wq.shape[0]
    y = np.empty((M, N), np.uint16 if bf16_out else F32)
    fn = lib.oq_linear_w8a8_bf16 if x_bf16_bits else lib.oq_linear_w8a8_f32
    fn(_p(x), _p(wq), _p(sw), _p(bias), None if bf16_out else _p(y), _p(y) if bf16_out else None, M, N, K)
    return y


def c_quant_tensor_fp8(x: np.ndarray, bf16_bits: bool = False):
    lib = _load()
    x = _c(x, np.uint16 if bf16_bits else F32)
    q = np.empty(x.shape, np.uint8)
    s = np.empty((1,), F32)
    fn = lib.oq_quant_tensor_fp8_bf16 if bf16_bits else lib.oq_quant_tensor_fp8_f32
    fn(_p(x), x.size, _p(q), _p(s))
    return q, F32(s[0])


def c_one_step_divide_mismatches(divisor: float, am_lo: int = 0, am_hi: int = 0x7F80, steps: int = 1):
    """(pairs whose code differs, pairs evaluated) for the one-correction divide on bf16 numbers: see the C source."""
    lib = _load()
    n = np.zeros((1,), np.int64)
    bad = lib.oq_one_step_divide_mismatches(float(divisor), int(steps), int(am_lo), int(am_hi), _p(n))
    return int(bad), int(n[0])


def c_linear_fp8(xq, sx, wq, sw, bf16_out: bool = False, bias=None) -> np.ndarray:
    lib = _load()
    xq, wq = _c(xq, np.uint8), _c(wq, np.uint8)
    bias = None if bias is None else _c(bias, F32)
    M, K = xq.shape
    N = wq.shape[0]
    y = np.empty((M, N), np.uint16 if bf16_out else F32)
    lib.oq_linear_fp8(_p(xq), float(sx), _p(wq), float(sw), _p(bias), None if bf16_out else _p(y),
                      _p(y) if bf16_out else None, M, N, K)
    return y


def c_linear_f32(x, w, bias=None) -> np.ndarray:
    lib = _load()
    x, w = _c(x, F32), _c(w, F32)
    bias = None if bias is None else _c(bias, F32)
    M, K = x.shape
    N = w.shape[0]
    y = np.empty((M, N), F32)
    lib.oq_linear_f32(_p(x), _p(w), _p(bias), _p(y), M, N, K)
    return y
