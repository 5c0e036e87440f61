"""Tensor-level operators over the C ABI.

Each function takes torch tensors that already live on the GPU, checks layout
the way the kernels assume it, and queues the work on torch's current HIP
stream.  torch is used for device memory and streams only; all arithmetic is in
libastrai_q.so.  Together these replace the single call
``F.linear(x, weight, bias)`` of astrai/model/components/linear.py:21.
"""
from __future__ import annotations

from typing import NamedTuple, Optional, Tuple

import torch

from . import _abi

_DT = {torch.float32: _abi.AQ_F32, torch.bfloat16: _abi.AQ_BF16}


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_cur_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream(t: torch.Tensor) -> int:
    """torch's current HIP stream on the tensor's device, as the raw handle the C ABI takes."""
    if _raw_stream is not None:
        return _raw_stream(t.device.index if t.device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(t.device).cuda_stream


class _OnDevice:
    """``torch.cuda.device(dev)`` that costs nothing when ``dev`` already is the current device (the
    usual case; a launch goes to the current device)."""
    __slots__ = ("ctx",)

    def __init__(self, dev: torch.device):
        self.ctx = None
        if _cur_device is None or dev.index is None or _cur_device() != dev.index:
            self.ctx = torch.cuda.device(dev)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            return self.ctx.__exit__(*exc)
        return False


def _need_gpu(*ts: Optional[torch.Tensor]) -> None:
    dev = None
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("astrai_q operators run on the GPU only; got a CPU tensor (no CPU fallback exists)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise ValueError("all tensors must be on the same device")


def _dt(t: torch.Tensor, what: str) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise ValueError(f"{what}: dtype {t.dtype} is not supported (float32 or bfloat16)") from None


def _rows(x: torch.Tensor, what: str) -> torch.Tensor:
    """View [..., K] as a contiguous [M, K]."""
    if x.dim() < 1:
        raise ValueError(f"{what}: needs at least one dimension")
    x2 = x.reshape(-1, x.shape[-1])
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    return x2


def _check_k(K: int) -> None:
    if K <= 0 or K % 16:
        raise ValueError(f"in_dim (K) must be a positive multiple of 16, got {K}")


def quant_rowwise_i8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Symmetric absmax int8 per row of ``x [..., K]`` -> (codes int8 [M, K], scale f32 [M])."""
    _need_gpu(x)
    x2 = _rows(x, "quant_rowwise_i8")
    M, K = x2.shape
    _check_k(K)
    q = torch.empty((M, K), dtype=torch.int8, device=x.device)
    s = torch.empty((M,), dtype=torch.float32, device=x.device)
    if M:
        with _OnDevice(x.device):
            rc = _abi.load().aq_quant_rowwise_i8(x2.data_ptr(), _dt(x2, "x"), M, K, x2.stride(0), q.data_ptr(),
                                                 s.data_ptr(), _stream(x))
        _abi.check(rc, "aq_quant_rowwise_i8")
    return q, s


# longest rows the fused row kernels keep in registers (elements): bf16, fp32
RMSNORM_QUANT_MAX_K = {torch.bfloat16: 12288, torch.float32: 6144}
SWIGLU_QUANT_MAX_F = {torch.bfloat16: 8192, torch.float32: 4096}


def rmsnorm_quant_rowwise_i8(x: torch.Tensor, gamma: torch.Tensor, eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """RMSNorm (gain ``gamma``, same dtype as ``x``) fused with the per-token quantisation of its
    output: ``[..., K]`` -> (codes int8 ``[M, K]``, scales float32 ``[M]``)."""
    _need_gpu(x, gamma)
    x2 = _rows(x, "x")
    M, K = x2.shape
    _check_k(K)
    if gamma.dtype != x2.dtype or gamma.numel() != K:
        raise ValueError("gamma must have the activations' dtype and K elements")
    gamma = gamma.contiguous()
    q = torch.empty((M, K), dtype=torch.int8, device=x2.device)
    s = torch.empty((M,), dtype=torch.float32, device=x2.device)
    if M:
        with _OnDevice(x2.device):
            rc = _abi.load().aq_rmsnorm_quant_rowwise_i8(x2.data_ptr(), _dt(x2, "x"), gamma.data_ptr(), _dt(gamma, "gamma"),
                                                         float(eps), M, K, x2.stride(0), q.data_ptr(), s.data_ptr(),
                                                         _stream(x2))
        _abi.check(rc, "aq_rmsnorm_quant_rowwise_i8")
    return q, s


def swiglu_quant_rowwise_i8(ug: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """``ug [..., 2F] = [up | gate]`` -> codes and scales of ``up * silu(gate)`` per row
    (int8 ``[M, F]``, float32 ``[M]``), without writing the product."""
    _need_gpu(ug)
    u2 = _rows(ug, "ug")
    M, F2 = u2.shape
    if F2 % 2:
        raise ValueError("the last dimension holds up and gate side by side: it must be even")
    F = F2 // 2
    _check_k(F)
    q = torch.empty((M, F), dtype=torch.int8, device=u2.device)
    s = torch.empty((M,), dtype=torch.float32, device=u2.device)
    if M:
        with _OnDevice(u2.device):
            rc = _abi.load().aq_swiglu_quant_rowwise_i8(u2.data_ptr(), _dt(u2, "ug"), M, F, u2.stride(0), q.data_ptr(),
                                                        s.data_ptr(), _stream(u2))
        _abi.check(rc, "aq_swiglu_quant_rowwise_i8")
    return q, s


# From this many input bytes on, the one-launch form of the per-tensor quantiser is the faster one (below, its
# exchange of partial maxima between workgroups costs more than the second launch: 6.9 against 4.6-5.2 us for small
# tensors, level at 16 MiB, 13.0 against 16.5 us at 32 MiB).
FP8_ONEPASS_MIN_BYTES = 16 << 20


def fp8_onepass_state(device) -> torch.Tensor:
    """The small piece of device state the one-launch per-tensor quantiser needs: zero-filled once, then reused
    for every call on that device and stream (calls that overlap in time must not share one)."""
    return torch.zeros((_abi.AQ_FP8_ONEPASS_WS_BYTES // 8,), dtype=torch.int64, device=device)


def quant_tensor_fp8(x: torch.Tensor, state: Optional[torch.Tensor] = None,
                     onepass: Optional[bool] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-tensor OCP e4m3fn -> (codes uint8 with x's shape, scale f32 [1]).
    ``state`` (from ``fp8_onepass_state``): allows the one-launch form, which reads x from HBM once instead of
    twice -- same codes and scale; taken for tensors of ``FP8_ONEPASS_MIN_BYTES`` and more, or as ``onepass`` says."""
    _need_gpu(x)
    xc = x.contiguous()
    n = xc.numel()
    if n % 16:
        raise ValueError(f"numel must be a multiple of 16, got {n}")
    q = torch.empty(xc.shape, dtype=torch.uint8, device=x.device)
    s = torch.empty((1,), dtype=torch.float32, device=x.device)
    if onepass is None:
        onepass = state is not None and n * xc.element_size() >= FP8_ONEPASS_MIN_BYTES
    if onepass:
        if state is None:
            raise ValueError("the one-launch form needs the state tensor of fp8_onepass_state()")
        _need_gpu(state)
        if state.dtype != torch.int64 or state.numel() * 8 < _abi.AQ_FP8_ONEPASS_WS_BYTES or not state.is_contiguous() \
                or state.device != x.device:
            raise ValueError("state must come from fp8_onepass_state() for x's device")
        with _OnDevice(x.device):
            rc = _abi.load().aq_quant_tensor_fp8_onepass(xc.data_ptr(), _dt(xc, "x"), n, q.data_ptr(), s.data_ptr(),
                                                         state.data_ptr(), state.numel() * 8, _stream(x))
        _abi.check(rc, "aq_quant_tensor_fp8_onepass")
        return q, s
    ws = torch.empty((_abi.AQ_FP8_AMAX_WS_BYTES // 4,), dtype=torch.int32, device=x.device)  # partial maxima, stateless
    with _OnDevice(x.device):
        rc = _abi.load().aq_quant_tensor_fp8(xc.data_ptr(), _dt(xc, "x"), n, q.data_ptr(), s.data_ptr(),
                                             ws.data_ptr(), ws.numel() * 4, _stream(x))
    _abi.check(rc, "aq_quant_tensor_fp8")
    return q, s


def gemm_i8_i32(xq: torch.Tensor, wq: torch.Tensor) -> torch.Tensor:
    """acc[m, n] = sum_k xq[m, k] * wq[n, k] in exact int32."""
    _need_gpu(xq, wq)
    if xq.dtype != torch.int8 or wq.dtype != torch.int8:
        raise ValueError("gemm_i8_i32 takes int8 codes")
    if xq.dim() != 2 or wq.dim() != 2 or xq.shape[1] != wq.shape[1]:
        raise ValueError(f"shape mismatch: xq {tuple(xq.shape)} vs wq {tuple(wq.shape)}")
    xq, wq = xq.contiguous(), wq.contiguous()
    M, K = xq.shape
    N = wq.shape[0]
    _check_k(K)
    acc = torch.empty((M, N), dtype=torch.int32, device=xq.device)
    if M and N:
        with _OnDevice(xq.device):
            rc = _abi.load().aq_gemm_i8_i32(xq.data_ptr(), wq.data_ptr(), acc.data_ptr(), M, N, K, _stream(xq))
        _abi.check(rc, "aq_gemm_i8_i32")
    return acc


def _bias_args(bias: Optional[torch.Tensor], N: int):
    if bias is None:
        return None, 0
    if bias.dim() != 1 or bias.shape[0] != N:
        raise ValueError(f"bias must have shape [{N}], got {tuple(bias.shape)}")
    b = bias.contiguous()
    return b, _dt(b, "bias")


def _residual_arg(residual, M, N, out_dtype, dev):
    """A residual is added to the rounded output (``y = round(linear) + residual``, rounded again:
    the bits of a separate elementwise add); it holds M*N elements of the output's dtype."""
    if residual is None:
        return None
    if residual.dtype != out_dtype or residual.numel() != M * N or residual.device != dev:
        raise ValueError(f"residual must hold {M}x{N} {out_dtype} elements on {dev}, got {residual.dtype} "
                         f"{tuple(residual.shape)} on {residual.device}")
    if residual.dim() < 1 or residual.shape[-1] != N:
        raise ValueError(f"residual's last dimension must be {N}, got {tuple(residual.shape)}")
    return residual.contiguous()


def linear_w8a8(xq, sx, wq, sw, bias=None, out_dtype=torch.bfloat16, residual=None) -> torch.Tensor:
    """MFMA GEMM with the fused epilogue y = (acc * sx[m]) * sw[n] (+ bias[n]) (+ residual[m, n])."""
    _need_gpu(xq, sx, wq, sw, bias, residual)
    if xq.dtype != torch.int8 or wq.dtype != torch.int8:
        raise ValueError("linear_w8a8 takes int8 codes")
    if xq.dim() != 2 or wq.dim() != 2 or xq.shape[1] != wq.shape[1]:
        raise ValueError(f"shape mismatch: xq {tuple(xq.shape)} vs wq {tuple(wq.shape)}")
    M, K = xq.shape
    N = wq.shape[0]
    _check_k(K)
    if sx.dtype != torch.float32 or sw.dtype != torch.float32 or sx.numel() != M or sw.numel() != N:
        raise ValueError("sx must be float32 [M] and sw float32 [N]")
    if out_dtype not in _DT:
        raise ValueError(f"out_dtype {out_dtype} is not supported")
    xq, wq, sx, sw = xq.contiguous(), wq.contiguous(), sx.contiguous(), sw.contiguous()
    b, bdt = _bias_args(bias, N)
    r = _residual_arg(residual, M, N, out_dtype, xq.device)
    y = torch.empty((M, N), dtype=out_dtype, device=xq.device)
    if M and N:
        with _OnDevice(xq.device):
            rc = _abi.load().aq_linear_w8a8_residual(xq.data_ptr(), sx.data_ptr(), wq.data_ptr(), sw.data_ptr(),
                                                     b.data_ptr() if b is not None else None, bdt,
                                                     r.data_ptr() if r is not None else None, y.data_ptr(),
                                                     _DT[out_dtype], M, N, K, _stream(xq))
        _abi.check(rc, "aq_linear_w8a8")
    elif r is not None:
        y.copy_(r.view(M, N))
    return y


def gemv_w8a8_decode(x, wq, sw, bias=None, out_dtype=None, workspace: Optional[torch.Tensor] = None,
                     residual=None, norm=None) -> torch.Tensor:
    """Decode path for at most 16 rows of ``x [M, K]``: fused per-token quantise + int8 GEMV + epilogue.
    ``norm = (gamma [K], eps)``: RMS-normalise the rows first (the codes ``rmsnorm_quant_rowwise_i8``
    gives), in the same launch for up to 8 bfloat16 rows of at most 2048 elements."""
    _need_gpu(x, wq, sw, bias, workspace, residual, norm[0] if norm is not None else None)
    x2 = _rows(x, "gemv_w8a8_decode")
    M, K = x2.shape
    N = wq.shape[0]
    if M > 16:
        raise ValueError(f"the decode path takes at most 16 rows, got {M}")
    if wq.dtype != torch.int8 or wq.dim() != 2 or wq.shape[1] != K:
        raise ValueError(f"wq must be int8 [N, {K}], got {wq.dtype} {tuple(wq.shape)}")
    _check_k(K)
    if sw.dtype != torch.float32 or sw.numel() != N:
        raise ValueError("sw must be float32 [N]")
    out_dtype = out_dtype or x.dtype
    if out_dtype not in _DT:
        raise ValueError(f"out_dtype {out_dtype} is not supported")
    wq, sw = wq.contiguous(), sw.contiguous()
    b, bdt = _bias_args(bias, N)
    lib = _abi.load()
    need = lib.aq_gemv_w8a8_workspace_bytes(M, K)
    if workspace is None:
        workspace = torch.empty((max(need, 16),), dtype=torch.uint8, device=x.device)
    elif workspace.numel() * workspace.element_size() < need:
        raise ValueError(f"workspace holds {workspace.numel() * workspace.element_size()} bytes, {need} needed")
    r = _residual_arg(residual, M, N, out_dtype, x.device)
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    if norm is not None:
        gamma, eps = norm
        if gamma.dtype != x2.dtype or gamma.numel() != K:
            raise ValueError(f"the norm's gain must be {x2.dtype} [{K}], got {gamma.dtype} {tuple(gamma.shape)}")
        gamma = gamma.contiguous()
    if M and N:
        with _OnDevice(x.device):
            if norm is None:
                rc = lib.aq_gemv_w8a8_decode_residual(x2.data_ptr(), _dt(x2, "x"), wq.data_ptr(), sw.data_ptr(),
                                                      b.data_ptr() if b is not None else None, bdt,
                                                      r.data_ptr() if r is not None else None, y.data_ptr(),
                                                      _DT[out_dtype], M, N, K, workspace.data_ptr(),
                                                      workspace.numel() * workspace.element_size(), _stream(x))
            else:
                rc = lib.aq_gemv_w8a8_decode_rmsnorm(x2.data_ptr(), _dt(x2, "x"), gamma.data_ptr(), float(eps),
                                                     wq.data_ptr(), sw.data_ptr(),
                                                     b.data_ptr() if b is not None else None, bdt,
                                                     r.data_ptr() if r is not None else None, y.data_ptr(),
                                                     _DT[out_dtype], M, N, K, workspace.data_ptr(),
                                                     workspace.numel() * workspace.element_size(), _stream(x))
        _abi.check(rc, "aq_gemv_w8a8_decode")
    elif r is not None:
        y.copy_(r.view(M, N))
    return y


def gemv_swiglu_ok(x: torch.Tensor, dim_ffn: int) -> bool:
    """Whether ``gemv_w8a8_decode_swiglu`` serves these rows (bf16, at most 16 of them, K <= 2048 in whole
    512-byte steps, dim_ffn a multiple of 16)."""
    if not x.is_cuda or x.dtype not in _DT:
        return False
    rows = x.numel() // x.shape[-1] if x.shape[-1] else 0
    return bool(_abi.load().aq_gemv_w8a8_decode_swiglu_ok(_DT[x.dtype], rows, dim_ffn, x.shape[-1]))


def gemv_w8a8_decode_swiglu(x, wq, sw, bias=None, out_dtype=None, norm=None) -> torch.Tensor:
    """``up(x) * silu(gate(x))`` of an MLP at decode in ONE launch: ``wq [2F, K]`` holds the up projection's rows and
    then the gate projection's (``QuantLinear.concat([up, gate])``); returns ``h [M, F]``.  ``norm = (gamma, eps)``:
    the RMSNorm in front, folded in as in ``gemv_w8a8_decode``.  Raises ``ValueError`` for shapes
    ``gemv_swiglu_ok`` refuses."""
    _need_gpu(x, wq, sw, bias, norm[0] if norm is not None else None)
    x2 = _rows(x, "gemv_w8a8_decode_swiglu")
    M, K = x2.shape
    if wq.dtype != torch.int8 or wq.dim() != 2 or wq.shape[1] != K or wq.shape[0] % 2:
        raise ValueError(f"wq must be int8 [2F, {K}], got {wq.dtype} {tuple(wq.shape)}")
    N = wq.shape[0]
    Fh = N // 2
    _check_k(K)
    if sw.dtype != torch.float32 or sw.numel() != N:
        raise ValueError("sw must be float32 [2F]")
    out_dtype = out_dtype or x.dtype
    if out_dtype not in _DT:
        raise ValueError(f"out_dtype {out_dtype} is not supported")
    wq, sw = wq.contiguous(), sw.contiguous()
    b, bdt = _bias_args(bias, N)
    gamma, eps = (None, 0.0)
    if norm is not None:
        gamma, eps = norm
        if gamma.dtype != x2.dtype or gamma.numel() != K:
            raise ValueError(f"the norm's gain must be {x2.dtype} [{K}], got {gamma.dtype} {tuple(gamma.shape)}")
        gamma = gamma.contiguous()
    h = torch.empty((M, Fh), dtype=out_dtype, device=x.device)
    if M and Fh:
        with _OnDevice(x.device):
            rc = _abi.load().aq_gemv_w8a8_decode_swiglu(x2.data_ptr(), _dt(x2, "x"),
                                                        gamma.data_ptr() if gamma is not None else None, float(eps),
                                                        wq.data_ptr(), sw.data_ptr(),
                                                        b.data_ptr() if b is not None else None, bdt, h.data_ptr(),
                                                        _DT[out_dtype], M, Fh, K, _stream(x))
        _abi.check(rc, "aq_gemv_w8a8_decode_swiglu")
    return h


def gemv_w8a8_codes(xq, sx, wq, sw, bias=None, out_dtype=torch.bfloat16, residual=None) -> torch.Tensor:
    """The decode GEMV on activation codes the caller already holds (at most 16 rows)."""
    _need_gpu(xq, sx, wq, sw, bias, residual)
    if xq.dtype != torch.int8 or wq.dtype != torch.int8:
        raise ValueError("gemv_w8a8_codes takes int8 codes")
    if xq.dim() != 2 or wq.dim() != 2 or xq.shape[1] != wq.shape[1]:
        raise ValueError(f"shape mismatch: xq {tuple(xq.shape)} vs wq {tuple(wq.shape)}")
    M, K = xq.shape
    N = wq.shape[0]
    if M > 16:
        raise ValueError(f"the decode path takes at most 16 rows, got {M}")
    _check_k(K)
    if sx.dtype != torch.float32 or sw.dtype != torch.float32 or sx.numel() != M or sw.numel() != N:
        raise ValueError("sx must be float32 [M] and sw float32 [N]")
    if out_dtype not in _DT:
        raise ValueError(f"out_dtype {out_dtype} is not supported")
    xq, wq, sx, sw = xq.contiguous(), wq.contiguous(), sx.contiguous(), sw.contiguous()
    b, bdt = _bias_args(bias, N)
    r = _residual_arg(residual, M, N, out_dtype, xq.device)
    y = torch.empty((M, N), dtype=out_dtype, device=xq.device)
    if M and N:
        with _OnDevice(xq.device):
            rc = _abi.load().aq_gemv_w8a8_codes_residual(xq.data_ptr(), sx.data_ptr(), wq.data_ptr(), sw.data_ptr(),
                                                         b.data_ptr() if b is not None else None, bdt,
                                                         r.data_ptr() if r is not None else None, y.data_ptr(),
                                                         _DT[out_dtype], M, N, K, _stream(xq))
        _abi.check(rc, "aq_gemv_w8a8_codes")
    elif r is not None:
        y.copy_(r.view(M, N))
    return y


def _rope_args(qkv, freqs, page_table, k_cache, v_cache, n_heads, n_kv_heads, what):
    """Checks shared by the rotary / KV-write entry points; returns (qkv [B, S, W], freqs as
    float32, its batch stride in floats, page_table), contiguous."""
    _need_gpu(qkv, freqs, page_table, k_cache, v_cache)
    D = k_cache.shape[-1]
    W = (n_heads + 2 * n_kv_heads) * D
    if qkv.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16 or v_cache.dtype != torch.bfloat16:
        raise ValueError(f"{what} takes bfloat16 activations and caches")
    if qkv.dim() not in (2, 3) or qkv.shape[-1] != W:
        raise ValueError(f"qkv must be [B, {W}] or [B, S, {W}], got {tuple(qkv.shape)}")
    if qkv.dim() == 2:
        qkv = qkv.unsqueeze(1)
    B, S = qkv.shape[0], qkv.shape[1]
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or k_cache.shape[2] != n_kv_heads:
        raise ValueError("caches must be [n_pages, page, Hkv, D] and alike")
    if not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise ValueError("caches must be contiguous")
    fr = torch.view_as_real(freqs) if freqs.is_complex() else freqs
    if fr.dtype != torch.float32 or fr.shape[0] != B or fr.numel() // max(B, 1) != S * D or fr.stride(-1) != 1:
        raise ValueError(f"freqs must be complex64 [B, (S,) {D // 2}] or float32 [B, (S,) {D // 2}, 2]")
    if B > 1 and fr.stride(0) == 0:      # one table broadcast to every sequence: no copy
        fr_stride, fr = 0, fr[0].contiguous()
    else:
        fr = fr.reshape(B, S * D).contiguous()
        fr_stride = S * D
    if fr.data_ptr() % 16:
        fr = fr.clone()
    if page_table.dtype != torch.int64 or page_table.dim() != 2 or page_table.shape[0] != B:
        raise ValueError("page_table must be int64 [B, P]")
    return qkv.contiguous(), fr, fr_stride, page_table.contiguous()


class QkNorm(NamedTuple):
    """Attention's qk-norm (``use_qk_norm``, astrai/model/components/attention.py:62-64, 86-89): the weights of the
    RMSNorm modules over the head dimension that follow the rotation of q and of k, and their epsilon."""
    q_gain: torch.Tensor
    k_gain: torch.Tensor
    eps: float


def _qk_norm_args(qk_norm, D: int, dev):
    """``(q_gain, k_gain, eps)`` checked for the kernels: bfloat16 ``[D]`` on ``dev``, 16-byte aligned."""
    if qk_norm is None:
        return None
    qg, kg, eps = qk_norm
    out = []
    for g in (qg, kg):
        if g.dtype != torch.bfloat16 or g.numel() != D or g.device != dev:
            raise ValueError(f"qk-norm gains must be bfloat16 [{D}] on {dev}, got {g.dtype} {tuple(g.shape)} on {g.device}")
        g = g.reshape(D).contiguous()
        out.append(g if g.data_ptr() % 16 == 0 else g.clone())
    if not eps >= 0.0:
        raise ValueError("qk-norm eps must not be negative")
    return out[0], out[1], float(eps)


def rope_kv_write(qkv: torch.Tensor, freqs: torch.Tensor, page_table: torch.Tensor, pos: int, k_cache: torch.Tensor,
                  v_cache: torch.Tensor, n_heads: int, n_kv_heads: int, return_k: bool = False,
                  qk_norm: Optional[QkNorm] = None):
    """New tokens of every sequence -- ``qkv [B, (Hq + 2 Hkv) * D]`` (one each, D = 64 or 128) or ``[B, S, ...]``:
    rotate q and k by ``freqs`` (complex64 ``[B, (S,) 64]`` or float32 ``[B, (S,) 64, 2]``), write k and
    v into the paged caches ``[n_pages, page, Hkv, D]`` at logical positions ``pos .. pos + S - 1``;
    returns the rotated ``q [B, (S,) Hq, D]``, and with ``return_k`` also the rotated
    ``k [B, (S,) Hkv, D]``.  With ``qk_norm`` the rotated q and k heads are RMS-normalised over D before they are
    returned and cached."""
    one = qkv.dim() == 2
    qkv, fr, fr_stride, page_table = _rope_args(qkv, freqs, page_table, k_cache, v_cache, n_heads, n_kv_heads,
                                                "rope_kv_write")
    B, S, D = qkv.shape[0], qkv.shape[1], k_cache.shape[-1]
    q = torch.empty((B, S, n_heads, D), dtype=torch.bfloat16, device=qkv.device)
    k = torch.empty((B, S, n_kv_heads, D), dtype=torch.bfloat16, device=qkv.device) if return_k else None
    norm = _qk_norm_args(qk_norm, D, qkv.device)
    if B and S:
        head = (qkv.data_ptr(), fr.data_ptr(), fr_stride, page_table.data_ptr(), page_table.shape[1], int(pos), S,
                k_cache.shape[1], k_cache.data_ptr(), v_cache.data_ptr(), k_cache.shape[0], q.data_ptr(),
                k.data_ptr() if return_k else None, B, n_heads, n_kv_heads, D)
        with _OnDevice(qkv.device):
            if norm is None:
                rc = _abi.load().aq_rope_kv_write(*head, _stream(qkv))
            else:
                rc = _abi.load().aq_rope_kv_write_qknorm(*head, norm[0].data_ptr(), norm[1].data_ptr(), norm[2],
                                                         _stream(qkv))
        _abi.check(rc, "aq_rope_kv_write" if norm is None else "aq_rope_kv_write_qknorm")
    if one:
        q, k = q.squeeze(1), (k.squeeze(1) if return_k else None)
    return (q, k) if return_k else q


def _attn_workspace(workspace, need, dev):
    if need and (workspace is None or not workspace.is_contiguous() or workspace.device != dev
                 or workspace.numel() * workspace.element_size() < need or workspace.data_ptr() % 16):
        workspace = torch.empty(need // 4, dtype=torch.float32, device=dev)
    if not need:
        return None, 0
    return workspace.data_ptr(), workspace.numel() * workspace.element_size()


class AttnPartials(NamedTuple):
    """A decode step's attention stopped before its position slices are combined: ``buf`` holds
    ``[B, n_heads, n_slices, D + 4]`` float32 (D numerators, maximum, denominator, padding)."""
    buf: torch.Tensor
    n_slices: int
    B: int
    n_heads: int
    head_dim: int


GEMV_ATTN_MAX_ROWS, GEMV_ATTN_MAX_K, GEMV_ATTN_MAX_SLICES = 8, 2048, 4


def attn_gemv_fusable(B: int, n_heads: int, head_dim: int, total_len: int) -> bool:
    """Whether ``gemv_w8a8_attn`` can, and should, combine this step's attention slices itself:
    within the kernel's limits, and more than one slice (a single slice has no merge launch to
    save, and the attention kernel's bf16 output is the smaller input)."""
    if not (0 < B <= GEMV_ATTN_MAX_ROWS and n_heads * head_dim <= GEMV_ATTN_MAX_K
            and 256 < total_len <= GEMV_ATTN_MAX_SLICES * 256):
        return False
    # Every workgroup of the projection repeats the merge of all rows, so it pays only while that is little work
    # (rows x row length x slices): 4 x 1536 x 3 saves 1.2 us per step over the separate merge launch, 8 x 2048 x 3
    # loses 0.8 us.
    slices = (total_len + 255) // 256
    return B * n_heads * head_dim * slices <= 32768


def rope_paged_attn_decode(qkv: torch.Tensor, freqs: torch.Tensor, page_table: torch.Tensor, total_len: int,
                           k_cache: torch.Tensor, v_cache: torch.Tensor, n_heads: int, n_kv_heads: int,
                           scale: Optional[float] = None, workspace: Optional[torch.Tensor] = None,
                           partials: bool = False, seq_lens: Optional[torch.Tensor] = None,
                           qk_norm: Optional[QkNorm] = None):
    """``rope_kv_write`` at position ``total_len - 1`` and ``paged_attn_decode`` over ``total_len``
    positions as one launch (plus the small merge launch for long sequences): same caches and
    outputs, bit for bit.  Returns the attention output ``[B, Hq, D]`` -- or, with ``partials``,
    the slices' partial results (no merge launch) for ``gemv_w8a8_attn`` to combine.
    ``seq_lens`` (int64 ``[B]`` on the device): sequence b attends to its first ``seq_lens[b]`` positions only.
    ``qk_norm``: as in ``rope_kv_write``, same bits."""
    if qkv.dim() != 2:
        raise ValueError(f"one new token per sequence: qkv must be [B, W], got {tuple(qkv.shape)}")
    qkv, fr, fr_stride, page_table = _rope_args(qkv, freqs, page_table, k_cache, v_cache, n_heads, n_kv_heads,
                                                "rope_paged_attn_decode")
    B, D = qkv.shape[0], k_cache.shape[-1]
    if total_len < 1:
        raise ValueError("total_len counts the new token: at least 1")
    lib = _abi.load()
    scale = float(scale if scale is not None else D ** -0.5)
    lens_ptr = _seq_lens_ptr(seq_lens, B, qkv.device)
    norm = _qk_norm_args(qk_norm, D, qkv.device)
    tail = () if norm is None else (norm[0].data_ptr(), norm[1].data_ptr(), norm[2])
    suffix = "" if norm is None else "_qknorm"
    if partials:
        if not B:
            raise ValueError("partial results need at least one sequence")
        need = int(lib.aq_paged_attn_decode_partials_bytes(B, n_heads, int(total_len)))
        if (workspace is None or not workspace.is_contiguous() or workspace.device != qkv.device
                or workspace.dtype != torch.float32 or workspace.numel() * 4 < need or workspace.data_ptr() % 16):
            workspace = torch.empty(need // 4, dtype=torch.float32, device=qkv.device)
        entry = "aq_rope_paged_attn_decode_partials" + suffix
        with _OnDevice(qkv.device):
            rc = getattr(lib, entry)(qkv.data_ptr(), fr.data_ptr(), fr_stride, page_table.data_ptr(),
                                     page_table.shape[1], int(total_len), lens_ptr, k_cache.shape[1],
                                     k_cache.data_ptr(), v_cache.data_ptr(), k_cache.shape[0],
                                     scale, B, n_heads, n_kv_heads, D, *tail, workspace.data_ptr(),
                                     workspace.numel() * 4, _stream(qkv))
        _abi.check(rc, entry)
        return AttnPartials(workspace, int(lib.aq_paged_attn_decode_slices(int(total_len))), B, n_heads, D)
    out = torch.empty((B, n_heads, D), dtype=torch.bfloat16, device=qkv.device)
    if B:
        ws_ptr, ws_bytes = _attn_workspace(workspace, paged_attn_workspace_bytes(B, n_heads, n_kv_heads, total_len),
                                           qkv.device)
        entry = "aq_rope_paged_attn_decode" + suffix
        with _OnDevice(qkv.device):
            rc = getattr(lib, entry)(qkv.data_ptr(), fr.data_ptr(), fr_stride, page_table.data_ptr(),
                                     page_table.shape[1], int(total_len), lens_ptr, k_cache.shape[1],
                                     k_cache.data_ptr(), v_cache.data_ptr(), k_cache.shape[0], scale,
                                     out.data_ptr(), B, n_heads, n_kv_heads, D, *tail, ws_ptr, ws_bytes,
                                     _stream(qkv))
        _abi.check(rc, entry)
    return out


def gemv_w8a8_attn(parts: AttnPartials, wq, sw, bias=None, out_dtype=torch.bfloat16, residual=None) -> torch.Tensor:
    """The output projection of a decode step on attention partial results: combines the slices
    (the merge kernel's arithmetic), quantises the ``[B, n_heads * D]`` rows and multiplies, one
    launch; the bits of ``rope_paged_attn_decode`` followed by ``gemv_w8a8_decode``."""
    _need_gpu(parts.buf, wq, sw, bias, residual)
    M, K = parts.B, parts.n_heads * parts.head_dim
    N = wq.shape[0]
    if wq.dtype != torch.int8 or wq.dim() != 2 or wq.shape[1] != K:
        raise ValueError(f"wq must be int8 [N, {K}], got {wq.dtype} {tuple(wq.shape)}")
    if sw.dtype != torch.float32 or sw.numel() != N:
        raise ValueError("sw must be float32 [N]")
    if out_dtype not in _DT:
        raise ValueError(f"out_dtype {out_dtype} is not supported")
    if M > GEMV_ATTN_MAX_ROWS or K > GEMV_ATTN_MAX_K or parts.n_slices > GEMV_ATTN_MAX_SLICES:
        raise ValueError(f"gemv_w8a8_attn takes at most {GEMV_ATTN_MAX_ROWS} rows of {GEMV_ATTN_MAX_K} elements in "
                         f"{GEMV_ATTN_MAX_SLICES} slices; got {M} x {K} in {parts.n_slices}")
    if parts.buf.dtype != torch.float32 or parts.buf.numel() < M * parts.n_heads * parts.n_slices * (parts.head_dim + 4):
        raise ValueError("the partial results do not cover [B, n_heads, n_slices, D + 4] float32")
    wq, sw = wq.contiguous(), sw.contiguous()
    b, bdt = _bias_args(bias, N)
    r = _residual_arg(residual, M, N, out_dtype, wq.device)
    y = torch.empty((M, N), dtype=out_dtype, device=wq.device)
    if N:
        with _OnDevice(wq.device):
            rc = _abi.load().aq_gemv_w8a8_decode_attn(parts.buf.data_ptr(), parts.n_slices, parts.head_dim,
                                                      wq.data_ptr(), sw.data_ptr(),
                                                      b.data_ptr() if b is not None else None, bdt,
                                                      r.data_ptr() if r is not None else None, y.data_ptr(),
                                                      _DT[out_dtype], M, N, K, _stream(wq))
        _abi.check(rc, "aq_gemv_w8a8_decode_attn")
    return y


def prefill_attn_causal(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: Optional[float] = None) -> torch.Tensor:
    """Causal attention of a prompt over itself: ``q [B, S, Hq, D]``, ``k`` / ``v [B, S, Hkv, D]`` (bfloat16,
    D = 64 or 128, last two dimensions contiguous, any token stride) -> ``[B, S, Hq, D]``."""
    _need_gpu(q, k, v)
    if q.dtype != torch.bfloat16 or k.dtype != torch.bfloat16 or v.dtype != torch.bfloat16:
        raise ValueError("prefill_attn_causal takes bfloat16 tensors")
    if q.dim() != 4 or k.dim() != 4 or k.shape != v.shape or q.shape[:2] != k.shape[:2] or q.shape[3] != k.shape[3]:
        raise ValueError("q must be [B, S, Hq, D] and k, v [B, S, Hkv, D]")
    B, S, Hq, D = q.shape
    Hkv = k.shape[2]

    def tokens(t, heads):
        # rows of heads*D contiguous elements, batch stride = S * token stride: otherwise copy
        if t.stride(3) == 1 and t.stride(2) == D and t.stride(0) == S * t.stride(1) and t.stride(1) % 8 == 0 \
                and t.data_ptr() % 16 == 0:
            return t, t.stride(1)
        return t.contiguous(), heads * D
    q, qs = tokens(q, Hq)
    k, ks = tokens(k, Hkv)
    v, vs = tokens(v, Hkv)
    out = torch.empty((B, S, Hq, D), dtype=torch.bfloat16, device=q.device)
    if B and S:
        with _OnDevice(q.device):
            rc = _abi.load().aq_prefill_attn_causal(q.data_ptr(), qs, k.data_ptr(), ks, v.data_ptr(), vs, out.data_ptr(),
                                                    float(scale if scale is not None else D ** -0.5), B, S, Hq, Hkv, D,
                                                    _stream(q))
        _abi.check(rc, "aq_prefill_attn_causal")
    return out


def prefill_attn_paged(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, page_table: torch.Tensor,
                       start: int, scale: Optional[float] = None) -> torch.Tensor:
    """Attention of ``S`` new tokens at positions ``start .. start + S`` over everything cached:
    ``q [B, S, Hq, D]`` against positions ``0 .. start + s`` of ``k_cache`` / ``v_cache
    [n_pages, page, Hkv, D]`` read through ``page_table [B, P]`` in place (the new tokens' rows
    written beforehand, ``rope_kv_write``) -> ``[B, S, Hq, D]``.  Unmapped pages are zero keys and
    values.  bfloat16, D = 64 or 128."""
    _need_gpu(q, k_cache, v_cache, page_table)
    if q.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16 or v_cache.dtype != torch.bfloat16:
        raise ValueError("prefill_attn_paged takes bfloat16 tensors")
    if q.dim() != 4 or k_cache.dim() != 4 or k_cache.shape != v_cache.shape or q.shape[3] != k_cache.shape[3]:
        raise ValueError("q must be [B, S, Hq, D] and the caches [n_pages, page, Hkv, D]")
    if page_table.dtype != torch.int64 or page_table.dim() != 2 or page_table.shape[0] != q.shape[0]:
        raise ValueError("page_table must be int64 [B, P]")
    B, S, Hq, D = q.shape
    n_pages, page, Hkv, _ = k_cache.shape
    if start < 0 or start + S > page_table.shape[1] * page:
        raise ValueError(f"positions {start} .. {start + S} fall outside the page table")
    if not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise ValueError("the caches must be contiguous")
    page_table = page_table.contiguous()
    if not (q.stride(3) == 1 and q.stride(2) == D and q.stride(0) == S * q.stride(1) and q.stride(1) % 8 == 0
            and q.data_ptr() % 16 == 0):
        q = q.contiguous()
    out = torch.empty((B, S, Hq, D), dtype=torch.bfloat16, device=q.device)
    if B and S:
        with _OnDevice(q.device):
            rc = _abi.load().aq_prefill_attn_paged(q.data_ptr(), q.stride(1), k_cache.data_ptr(), v_cache.data_ptr(),
                                                   page_table.data_ptr(), page_table.shape[1], int(start), page,
                                                   n_pages, out.data_ptr(),
                                                   float(scale if scale is not None else D ** -0.5), B, S, Hq, Hkv, D,
                                                   _stream(q))
        _abi.check(rc, "aq_prefill_attn_paged")
    return out


def paged_attn_workspace_bytes(B: int, n_heads: int, n_kv_heads: int, total_len: int) -> int:
    """Bytes of device workspace ``paged_attn_decode`` needs for this shape (0: none)."""
    return int(_abi.load().aq_paged_attn_decode_workspace_bytes(B, n_heads, n_kv_heads, int(total_len)))


def paged_attn_partials_bytes(B: int, n_heads: int, total_len: int) -> int:
    """Bytes the slices' partial results of a decode step take (also enough as its workspace)."""
    return int(_abi.load().aq_paged_attn_decode_partials_bytes(B, n_heads, int(total_len)))


def _seq_lens_ptr(seq_lens: Optional[torch.Tensor], B: int, device) -> Optional[int]:
    if seq_lens is None:
        return None
    if seq_lens.dtype != torch.int64 or seq_lens.shape != (B,) or seq_lens.device != device or not seq_lens.is_contiguous():
        raise ValueError(f"seq_lens must be a contiguous int64 [{B}] tensor on {device}")
    return seq_lens.data_ptr()


def paged_attn_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, page_table: torch.Tensor,
                      total_len: int, scale: Optional[float] = None,
                      workspace: Optional[torch.Tensor] = None, seq_lens: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``softmax(scale * q K^T) V`` for one query token per sequence over the first ``total_len``
    positions of each sequence's pages: ``q [B, Hq, D]`` -> ``[B, Hq, D]`` (bfloat16, D = 64 or 128).
    ``workspace``: a contiguous device tensor of at least ``paged_attn_workspace_bytes`` bytes
    to reuse across calls; allocated per call when omitted or too small."""
    _need_gpu(q, k_cache, v_cache, page_table)
    if q.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16 or v_cache.dtype != torch.bfloat16:
        raise ValueError("paged_attn_decode takes bfloat16 tensors")
    if q.dim() != 3 or k_cache.dim() != 4 or k_cache.shape != v_cache.shape or q.shape[2] != k_cache.shape[3]:
        raise ValueError("q must be [B, Hq, D] and the caches [n_pages, page, Hkv, D]")
    if not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise ValueError("caches must be contiguous")
    B, Hq, D = q.shape
    Hkv = k_cache.shape[2]
    if page_table.dtype != torch.int64 or page_table.dim() != 2 or page_table.shape[0] != B:
        raise ValueError("page_table must be int64 [B, P]")
    page_table, q = page_table.contiguous(), q.contiguous()
    out = torch.empty_like(q)
    if B:
        ws_ptr, ws_bytes = _attn_workspace(workspace, paged_attn_workspace_bytes(B, Hq, Hkv, total_len), q.device)
        with _OnDevice(q.device):
            rc = _abi.load().aq_paged_attn_decode(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                                  page_table.data_ptr(), page_table.shape[1], int(total_len),
                                                  _seq_lens_ptr(seq_lens, B, q.device), k_cache.shape[1], k_cache.shape[0],
                                                  float(scale if scale is not None else D ** -0.5), out.data_ptr(),
                                                  B, Hq, Hkv, D, ws_ptr, ws_bytes, _stream(q))
        _abi.check(rc, "aq_paged_attn_decode")
    return out


def linear_fp8(xq, sx, wq, sw, bias=None, out_dtype=torch.bfloat16, residual=None) -> torch.Tensor:
    """FP8 e4m3fn GEMM with fp32 accumulation: y = (acc * sx[0]) * sw[0] (+ bias), cast, (+ residual)."""
    _need_gpu(xq, sx, wq, sw, bias, residual)
    if xq.dtype != torch.uint8 or wq.dtype != torch.uint8:
        raise ValueError("linear_fp8 takes e4m3fn codes as uint8")
    if xq.dim() != 2 or wq.dim() != 2 or xq.shape[1] != wq.shape[1]:
        raise ValueError(f"shape mismatch: xq {tuple(xq.shape)} vs wq {tuple(wq.shape)}")
    M, K = xq.shape
    N = wq.shape[0]
    _check_k(K)
    if sx.dtype != torch.float32 or sw.dtype != torch.float32 or sx.numel() != 1 or sw.numel() != 1:
        raise ValueError("sx and sw must be float32 device scalars")
    if out_dtype not in _DT:
        raise ValueError(f"out_dtype {out_dtype} is not supported")
    xq, wq = xq.contiguous(), wq.contiguous()
    b, bdt = _bias_args(bias, N)
    r = _residual_arg(residual, M, N, out_dtype, xq.device)
    y = torch.empty((M, N), dtype=out_dtype, device=xq.device)
    if M and N:
        with _OnDevice(xq.device):
            rc = _abi.load().aq_linear_fp8_residual(xq.data_ptr(), sx.data_ptr(), wq.data_ptr(), sw.data_ptr(),
                                                    b.data_ptr() if b is not None else None, bdt,
                                                    r.data_ptr() if r is not None else None, y.data_ptr(),
                                                    _DT[out_dtype], M, N, K, _stream(xq))
        _abi.check(rc, "aq_linear_fp8")
    elif r is not None:
        y.copy_(r.view(M, N))
    return y


def gemv_fp8_codes(xq, sx, wq, sw, bias=None, out_dtype=torch.bfloat16, residual=None) -> torch.Tensor:
    """The FP8 decode GEMV on codes the caller already holds (at most 16 rows; ``sx``, ``sw`` device scalars)."""
    _need_gpu(xq, sx, wq, sw, bias, residual)
    if xq.dtype != torch.uint8 or wq.dtype != torch.uint8 or xq.dim() != 2 or wq.dim() != 2 or xq.shape[1] != wq.shape[1]:
        raise ValueError(f"gemv_fp8_codes takes e4m3fn codes as uint8 [M, K] and [N, K], got {tuple(xq.shape)} / {tuple(wq.shape)}")
    M, K = xq.shape
    N = wq.shape[0]
    if M > 16:
        raise ValueError(f"the decode path takes at most 16 rows, got {M}")
    _check_k(K)
    if sx.dtype != torch.float32 or sw.dtype != torch.float32 or sx.numel() != 1 or sw.numel() != 1:
        raise ValueError("sx and sw must be float32 device scalars")
    if out_dtype not in _DT:
        raise ValueError(f"out_dtype {out_dtype} is not supported")
    xq, wq = xq.contiguous(), wq.contiguous()
    b, bdt = _bias_args(bias, N)
    r = _residual_arg(residual, M, N, out_dtype, xq.device)
    y = torch.empty((M, N), dtype=out_dtype, device=xq.device)
    if M and N:
        with _OnDevice(xq.device):
            rc = _abi.load().aq_gemv_fp8_codes_residual(xq.data_ptr(), sx.data_ptr(), wq.data_ptr(), sw.data_ptr(),
                                                        b.data_ptr() if b is not None else None, bdt,
                                                        r.data_ptr() if r is not None else None, y.data_ptr(),
                                                        _DT[out_dtype], M, N, K, _stream(xq))
        _abi.check(rc, "aq_gemv_fp8_codes")
    elif r is not None:
        y.copy_(r.view(M, N))
    return y


def gemv_fp8_decode(x, wq, sw, bias=None, out_dtype=None, workspace: Optional[torch.Tensor] = None,
                    residual=None) -> torch.Tensor:
    """FP8 decode path for at most 16 rows of ``x [M, K]``: per-tensor e4m3 cast + GEMV + epilogue, one launch for
    bfloat16 rows of at most 2048 elements."""
    _need_gpu(x, wq, sw, bias, workspace, residual)
    x2 = _rows(x, "gemv_fp8_decode")
    M, K = x2.shape
    N = wq.shape[0]
    if M > 16:
        raise ValueError(f"the decode path takes at most 16 rows, got {M}")
    if wq.dtype != torch.uint8 or wq.dim() != 2 or wq.shape[1] != K:
        raise ValueError(f"wq must be uint8 (e4m3fn codes) [N, {K}], got {wq.dtype} {tuple(wq.shape)}")
    _check_k(K)
    if sw.dtype != torch.float32 or sw.numel() != 1:
        raise ValueError("sw must be a float32 device scalar")
    out_dtype = out_dtype or x.dtype
    if out_dtype not in _DT:
        raise ValueError(f"out_dtype {out_dtype} is not supported")
    wq = wq.contiguous()
    b, bdt = _bias_args(bias, N)
    lib = _abi.load()
    need = lib.aq_gemv_fp8_workspace_bytes(M, K)
    if workspace is None:
        workspace = torch.empty((max(need, 16),), dtype=torch.uint8, device=x.device)
    elif workspace.numel() * workspace.element_size() < need:
        raise ValueError(f"workspace holds {workspace.numel() * workspace.element_size()} bytes, {need} needed")
    r = _residual_arg(residual, M, N, out_dtype, x.device)
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    if M and N:
        with _OnDevice(x.device):
            rc = lib.aq_gemv_fp8_decode_residual(x2.data_ptr(), _dt(x2, "x"), wq.data_ptr(), sw.data_ptr(),
                                                 b.data_ptr() if b is not None else None, bdt,
                                                 r.data_ptr() if r is not None else None, y.data_ptr(), _DT[out_dtype],
                                                 M, N, K, workspace.data_ptr(),
                                                 workspace.numel() * workspace.element_size(), _stream(x))
        _abi.check(rc, "aq_gemv_fp8_decode")
    elif r is not None:
        y.copy_(r.view(M, N))
    return y
