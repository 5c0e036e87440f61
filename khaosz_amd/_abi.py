"""ctypes binding of libastrai_q.so (the C ABI in include/astrai_q.h).

The library is built in-tree by khaosz_amd/build.py.  There is no CPU
fallback: if the shared object is missing, loading raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("ASTRAI_Q_LIB") or os.path.join(_HERE, "lib", "libastrai_q.so")

AQ_F32, AQ_BF16 = 0, 1
AQ_FP8_AMAX_WS_BYTES = 1024  # include/astrai_q.h
AQ_FP8_ONEPASS_WS_BYTES = 2048  # include/astrai_q.h

# every symbol include/astrai_q.h declares: name -> (restype, argtypes)
_i64, _vp, _int, _sz = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
SYMBOLS = {
    "aq_version": (_int, []),
    "aq_error_string": (ctypes.c_char_p, [_int]),
    "aq_quant_rowwise_i8": (_int, [_vp, _int, _i64, _i64, _i64, _vp, _vp, _vp]),
    "aq_rmsnorm_quant_rowwise_i8": (_int, [_vp, _int, _vp, _int, ctypes.c_float, _i64, _i64, _i64, _vp, _vp, _vp]),
    "aq_swiglu_quant_rowwise_i8": (_int, [_vp, _int, _i64, _i64, _i64, _vp, _vp, _vp]),
    "aq_quant_tensor_fp8": (_int, [_vp, _int, _i64, _vp, _vp, _vp, _sz, _vp]),
    "aq_quant_tensor_fp8_onepass": (_int, [_vp, _int, _i64, _vp, _vp, _vp, _sz, _vp]),
    "aq_gemm_i8_i32": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "aq_linear_w8a8": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _vp, _int, _i64, _i64, _i64, _vp]),
    "aq_linear_w8a8_residual": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _vp, _vp, _int, _i64, _i64, _i64, _vp]),
    "aq_gemv_w8a8_workspace_bytes": (_sz, [_i64, _i64]),
    "aq_gemv_w8a8_decode": (_int, [_vp, _int, _vp, _vp, _vp, _int, _vp, _int, _i64, _i64, _i64, _vp, _sz, _vp]),
    "aq_gemv_w8a8_codes": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _vp, _int, _i64, _i64, _i64, _vp]),
    "aq_gemv_w8a8_decode_residual": (_int, [_vp, _int, _vp, _vp, _vp, _int, _vp, _vp, _int, _i64, _i64, _i64, _vp, _sz,
                                            _vp]),
    "aq_gemv_w8a8_decode_noalloc": (_int, [_vp, _int, _vp, _vp, _vp, _int, _vp, _vp, _int, _i64, _i64, _i64, _vp]),
    "aq_gemv_w8a8_decode_swiglu_ok": (_int, [_int, _i64, _i64, _i64]),
    "aq_gemv_w8a8_decode_swiglu": (_int, [_vp, _int, _vp, ctypes.c_float, _vp, _vp, _vp, _int, _vp, _int, _i64, _i64,
                                          _i64, _vp]),
    "aq_gemv_w8a8_decode_rmsnorm": (_int, [_vp, _int, _vp, ctypes.c_float, _vp, _vp, _vp, _int, _vp, _vp, _int, _i64, _i64,
                                           _i64, _vp, _sz, _vp]),
    "aq_gemv_w8a8_codes_residual": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _vp, _vp, _int, _i64, _i64, _i64, _vp]),
    "aq_linear_fp8": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _vp]),
    "aq_gemv_fp8_workspace_bytes": (_sz, [_i64, _i64]),
    "aq_gemv_fp8_codes_residual": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _vp, _vp, _int, _i64, _i64, _i64, _vp]),
    "aq_gemv_fp8_decode_residual": (_int, [_vp, _int, _vp, _vp, _vp, _int, _vp, _vp, _int, _i64, _i64, _i64, _vp,
                                           _sz, _vp]),
    "aq_linear_fp8_residual": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _vp, _vp, _int, _i64, _i64, _i64, _vp]),
    "aq_rope_kv_write": (_int, [_vp, _vp, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _i64, _vp, _vp, _i64, _i64, _i64,
                                _i64, _vp]),
    "aq_paged_attn_decode": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _vp, _i64, _i64, ctypes.c_float, _vp, _i64, _i64, _i64,
                                    _i64, _vp, _i64, _vp]),
    "aq_prefill_attn_causal": (_int, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, ctypes.c_float, _i64, _i64, _i64, _i64, _i64,
                                      _vp]),
    "aq_paged_attn_decode_workspace_bytes": (_i64, [_i64, _i64, _i64, _i64]),
    "aq_rope_paged_attn_decode": (_int, [_vp, _vp, _i64, _vp, _i64, _i64, _vp, _i64, _vp, _vp, _i64, ctypes.c_float, _vp,
                                         _i64, _i64, _i64, _i64, _vp, _i64, _vp]),
    "aq_paged_attn_decode_slices": (_i64, [_i64]),
    "aq_paged_attn_decode_partials_bytes": (_i64, [_i64, _i64, _i64]),
    "aq_paged_attn_decode_partials": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _vp, _i64, _i64, ctypes.c_float, _i64, _i64,
                                             _i64, _i64, _vp, _i64, _vp]),
    "aq_rope_paged_attn_decode_partials": (_int, [_vp, _vp, _i64, _vp, _i64, _i64, _vp, _i64, _vp, _vp, _i64, ctypes.c_float,
                                                  _i64, _i64, _i64, _i64, _vp, _i64, _vp]),
    "aq_rope_kv_write_qknorm": (_int, [_vp, _vp, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _i64, _vp, _vp, _i64, _i64,
                                       _i64, _i64, _vp, _vp, ctypes.c_float, _vp]),
    "aq_rope_paged_attn_decode_qknorm": (_int, [_vp, _vp, _i64, _vp, _i64, _i64, _vp, _i64, _vp, _vp, _i64, ctypes.c_float,
                                                _vp, _i64, _i64, _i64, _i64, _vp, _vp, ctypes.c_float, _vp, _i64, _vp]),
    "aq_rope_paged_attn_decode_partials_qknorm": (_int, [_vp, _vp, _i64, _vp, _i64, _i64, _vp, _i64, _vp, _vp, _i64,
                                                         ctypes.c_float, _i64, _i64, _i64, _i64, _vp, _vp, ctypes.c_float,
                                                         _vp, _i64, _vp]),
    "aq_gemv_w8a8_decode_attn": (_int, [_vp, _i64, _i64, _vp, _vp, _vp, _int, _vp, _vp, _int, _i64, _i64, _i64, _vp]),
    "aq_prefill_attn_paged": (_int, [_vp, _i64, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, ctypes.c_float, _i64, _i64, _i64,
                                     _i64, _i64, _vp]),
}

# csrc/aq_lab.h: the lab library's additions (measurement probes, the tile-forcing test hook)
LAB_LIB_PATH = os.path.join(_HERE, "lib", "libastrai_q_lab.so")
LAB_SYMBOLS = {
    "aq_lab_set_gemm_tile": (_int, [_int]),
    "aq_lab_choose_gemm_tile": (_int, [_i64, _i64, _int]),
    "aq_lab_probe_mfma": (_int, [_int, _int, _int, _int, _vp, _vp, _vp]),
    "aq_lab_probe_copy": (_int, [_vp, _vp, _i64, _int, _vp]),
    "aq_lab_probe_read": (_int, [_vp, _i64, _int, _int, _int, _vp, _vp]),
    "aq_lab_probe_empty": (_int, [_vp, _vp]),
    "aq_lab_probe_mfma_lds_issue": (_int, [_int, _int, _int, _vp, _vp, _vp]),
    "aq_lab_quant_tensor_fp8_onepass_spin": (_int, [_vp, _int, _i64, _vp, _vp, _vp, _sz, _int, _vp]),
    "aq_lab_probe_swiglu_bf16": (_int, [_vp, _vp, _i64, _vp, _vp, _vp]),
    "aq_lab_set_gemv_timeline": (_int, [_vp]),
    "aq_lab_read_clock": (_int, [_vp]),
    "aq_lab_set_gemv_skip_weights": (_int, [_int]),
}

_lib = None
_lab = None


def load() -> ctypes.CDLL:
    """Load the HIP library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m khaosz_amd.build` "
            "(hipcc, --offload-arch=gfx950). There is no fallback path."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def load_lab() -> ctypes.CDLL:
    """The lab library: every product symbol (from the same objects) plus LAB_SYMBOLS.  For the benchmark's
    ceiling probes and for tests; the product path never loads it."""
    global _lab
    if _lab is not None:
        return _lab
    if not os.path.exists(LAB_LIB_PATH):
        raise RuntimeError(f"{LAB_LIB_PATH} is missing: build it with `python -m khaosz_amd.build`")
    lib = ctypes.CDLL(LAB_LIB_PATH)
    for name, (res, args) in {**SYMBOLS, **LAB_SYMBOLS}.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lab = lib
    return lib


class lab_library:
    """Context manager for tests: inside it ``load()`` hands out the lab library, so that the host module's
    operators run the lab build (whose GEMM tile can be forced).  Not thread-safe; never used by the product."""

    def __enter__(self):
        global _lib
        self._saved = _lib
        _lib = load_lab()
        return _lib

    def __exit__(self, *exc):
        global _lib
        _lib.aq_lab_set_gemm_tile(0)
        _lib = self._saved
        return False


def check(code: int, what: str) -> None:
    """Reference convention: errors surface as Python exceptions
    (e.g. astrai/parallel/module.py:34-37), never as return codes."""
    if code != 0:
        msg = load().aq_error_string(code).decode()
        if code in (-2, -3, -4, -6):
            raise ValueError(f"{what}: {msg} (code {code})")
        raise RuntimeError(f"{what}: {msg} (code {code})")
