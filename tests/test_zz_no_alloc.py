"""The decode entry point that allocates nothing (aq_gemv_w8a8_decode_noalloc): its workspace is a device array the
library owns.  Called through the C ABI and compared bit for bit with aq_gemv_w8a8_decode_residual (caller's
workspace) on two calls in a row, the second with a smaller input -- the array then still holds the first call's
codes beyond what the second one writes."""
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from khaosz_amd import _abi  # noqa: E402

pytestmark = pytest.mark.gpu


def _both(lib, x, wq, sw, bias, res, out_dtype):
    M, K = x.shape
    N = wq.shape[0]
    dt = {torch.float32: 0, torch.bfloat16: 1}
    st = torch.cuda.current_stream().cuda_stream
    ws = torch.empty(lib.aq_gemv_w8a8_workspace_bytes(M, K), dtype=torch.uint8, device=x.device)
    y_ref = torch.full((M, N), float("nan"), dtype=out_dtype, device=x.device)
    y_new = torch.full((M, N), float("nan"), dtype=out_dtype, device=x.device)
    b_ptr, b_dt = (bias.data_ptr(), dt[bias.dtype]) if bias is not None else (None, 0)
    r_ptr = res.data_ptr() if res is not None else None
    rc = lib.aq_gemv_w8a8_decode_residual(x.data_ptr(), dt[x.dtype], wq.data_ptr(), sw.data_ptr(), b_ptr, b_dt, r_ptr,
                                          y_ref.data_ptr(), dt[out_dtype], M, N, K, ws.data_ptr(), ws.numel(), st)
    assert rc == 0, rc
    # "allocates nothing" is checked at the driver's level (hipMemGetInfo: a hipMalloc inside the library would
    # show there; torch's own counter only sees torch's caching allocator), around the call and its completion.
    # The symbol's address is resolved by the first call of the process, so that one is made outside the window.
    rc = lib.aq_gemv_w8a8_decode_noalloc(x.data_ptr(), dt[x.dtype], wq.data_ptr(), sw.data_ptr(), b_ptr, b_dt, r_ptr,
                                         y_new.data_ptr(), dt[out_dtype], M, N, K, st)
    assert rc == 0, rc
    torch.cuda.synchronize()
    y_new.fill_(float("nan"))
    torch.cuda.synchronize()
    free_before, torch_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
    rc = lib.aq_gemv_w8a8_decode_noalloc(x.data_ptr(), dt[x.dtype], wq.data_ptr(), sw.data_ptr(), b_ptr, b_dt, r_ptr,
                                         y_new.data_ptr(), dt[out_dtype], M, N, K, st)
    assert rc == 0, rc
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before and torch.cuda.memory_allocated() == torch_before
    return y_ref, y_new


def test_no_alloc_decode_matches_the_workspace_entry_point_twice_in_a_row():
    lib = _abi.load()
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(5)

    def case(M, N, K, x_dtype, out_dtype, with_bias, with_res):
        x = torch.randn(M, K, generator=g).to(x_dtype).to(dev)
        wq = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8).to(dev)
        sw = (torch.rand(N, generator=g) * 1e-2 + 1e-3).to(dev)
        bias = (torch.randn(N, generator=g) * 0.01).to(dev) if with_bias else None
        res = torch.randn(M, N, generator=g).to(out_dtype).to(dev) if with_res else None
        a, b = _both(lib, x, wq, sw, bias, res, out_dtype)
        assert not torch.isnan(a.float()).any()
        assert torch.equal(a.view(torch.int16 if out_dtype == torch.bfloat16 else torch.int32),
                           b.view(torch.int16 if out_dtype == torch.bfloat16 else torch.int32)), (M, N, K)

    # first call: 16 rows of 8192 (codes go through the library's array: 128 KiB of it)
    case(16, 1000, 8192, torch.bfloat16, torch.bfloat16, True, True)
    # second call, smaller: 11 rows of 1280; the array still holds the first call's codes behind them
    case(11, 520, 1280, torch.bfloat16, torch.bfloat16, False, True)
    # fp32 rows take the array at every row count; then a one-launch shape (rows quantised inside the GEMV)
    case(3, 300, 2048, torch.float32, torch.float32, True, False)
    case(4, 300, 2048, torch.bfloat16, torch.bfloat16, False, False)
    # rows too long for the GEMV kernels' LDS (16 x 16384): row quantiser into the array, then the token-group
    # kernel of the tiled path reads the codes from it
    case(16, 136, 16384, torch.bfloat16, torch.bfloat16, True, True)
    case(9, 72, 16384, torch.float32, torch.float32, False, False)


def test_no_alloc_decode_rejects_sizes_beyond_its_array():
    lib = _abi.load()
    dev = torch.device("cuda:0")
    x = torch.zeros(16, 16400, dtype=torch.bfloat16, device=dev)  # 16 x 16400 > 262144 codes
    wq = torch.zeros(8, 16400, dtype=torch.int8, device=dev)
    sw = torch.ones(8, device=dev)
    y = torch.zeros(16, 8, dtype=torch.bfloat16, device=dev)
    rc = lib.aq_gemv_w8a8_decode_noalloc(x.data_ptr(), 1, wq.data_ptr(), sw.data_ptr(), None, 0, None, y.data_ptr(), 1,
                                         16, 8, 16400, None)
    assert rc == -6
    assert b"beyond" in lib.aq_error_string(rc)
    with pytest.raises(ValueError):
        _abi.check(rc, "aq_gemv_w8a8_decode_noalloc")
    assert lib.aq_gemv_w8a8_decode_noalloc(x.data_ptr(), 1, wq.data_ptr(), sw.data_ptr(), None, 0, None, y.data_ptr(),
                                           1, 17, 8, 64, None) == -2
