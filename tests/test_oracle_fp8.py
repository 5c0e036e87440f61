"""Pins the oracle's FP8 (OCP e4m3fn) path: codes against torch's cast after the
clamp, the GEMM against float64 accumulation of the decoded codes, and the whole
Linear against F.linear (astrai/model/components/linear.py:20-21)."""
import numpy as np
import torch


def test_quant_tensor_fp8_codes_match_torch_cast(oracle):
    rng = np.random.default_rng(10)
    x = rng.standard_normal((64, 512)).astype(np.float32)
    x[3, 7] = 9.0  # the amax element must land exactly on 448
    qn, sn = oracle.np_quant_tensor_fp8(x)
    qc, sc = oracle.c_quant_tensor_fp8(x)
    assert sn == sc == np.float32(np.float32(9.0) / np.float32(448.0))
    assert np.array_equal(qn, qc)
    v = np.clip((x / sn).astype(np.float32), -448, 448)
    want = torch.from_numpy(v).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(qc, want)
    assert qc[3, 7] == 0x7E
    # zero tensor: scale 1, all codes zero
    q0, s0 = oracle.c_quant_tensor_fp8(np.zeros((4, 16), np.float32))
    assert s0 == 1.0 and not q0.any()
    # sign symmetry
    qm, sm = oracle.c_quant_tensor_fp8(-x)
    assert sm == sc and np.array_equal(qm, qc ^ 0x80)


def test_quant_tensor_fp8_bf16_input(oracle):
    rng = np.random.default_rng(11)
    bits = oracle.np_f32_to_bf16_bits(rng.standard_normal((8, 64)).astype(np.float32))
    q1, s1 = oracle.c_quant_tensor_fp8(bits, bf16_bits=True)
    q2, s2 = oracle.c_quant_tensor_fp8(oracle.np_bf16_bits_to_f32(bits))
    assert s1 == s2 and np.array_equal(q1, q2)


def test_linear_fp8_fp32_accumulate_within_tolerance_of_exact(oracle):
    rng = np.random.default_rng(12)
    x = rng.standard_normal((24, 1024)).astype(np.float32)
    w = (rng.standard_normal((40, 1024)) * 0.02).astype(np.float32)
    xq, sx = oracle.c_quant_tensor_fp8(x)
    wq, sw = oracle.c_quant_tensor_fp8(w)
    y = oracle.c_linear_fp8(xq, sx, wq, sw)
    exact = oracle.np_linear_fp8(xq, sx, wq, sw)
    rms = np.sqrt(np.mean(exact.astype(np.float64) ** 2))
    assert np.max(np.abs(y - exact)) <= 1e-4 * rms
    yb = oracle.c_linear_fp8(xq, sx, wq, sw, bf16_out=True)
    assert np.array_equal(yb, oracle.np_f32_to_bf16_bits(y))
    # with a bias (linear.py:11,21): one more rounded add, against the float64 sum and a hand value
    b = (rng.standard_normal(40) * 0.5).astype(np.float32)
    yb32 = oracle.c_linear_fp8(xq, sx, wq, sw, bias=b)
    assert np.array_equal(yb32, (y + b[None, :]).astype(np.float32))
    assert np.max(np.abs(yb32 - oracle.np_linear_fp8(xq, sx, wq, sw, bias=b))) <= 1e-4 * max(rms, 0.5)
    # one hand-checked product: 1.5 * -2 summed 16 times, scales 0.5 and 4
    a = np.full((1, 16), 0x3C, np.uint8)       # 1.5
    b = np.full((1, 16), 0xC0, np.uint8)       # -2.0
    assert oracle.c_linear_fp8(a, 0.5, b, 4.0)[0, 0] == 16 * 1.5 * -2.0 * 0.5 * 4.0
    assert oracle.c_linear_fp8(a, 0.5, b, 4.0, bias=np.array([100.25], np.float32))[0, 0] == 16 * 1.5 * -2.0 * 0.5 * 4.0 + 100.25
    # end to end against the float Linear: e4m3 carries 3 mantissa bits, so the
    # element error is about 2^-4/sqrt(3) relative and averages down over K
    ref = torch.nn.functional.linear(torch.from_numpy(x), torch.from_numpy(w)).numpy()
    rel = np.linalg.norm(y - ref) / np.linalg.norm(ref)
    assert 0.01 < rel < 0.06, rel
