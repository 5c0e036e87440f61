"""Pins the oracle's RMSNorm -> row quantise (CPU).

The norm restates ``F.rms_norm(x, (K,), weight, eps)`` (astrai/model/components/norm.py:14-15)
with a fixed fp32 summation order; the reference has no fused norm+quantise, so the checks
are: the mathematics (float64, closed forms), torch's own rms_norm, and the independent numpy
restatement bit for bit.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F


def _bf16_bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("M,K", [(3, 16), (5, 1040), (4, 2048), (2, 5632)])
def test_c_and_numpy_restatements_agree_bit_for_bit(oracle, M, K):
    g = torch.Generator().manual_seed(K)
    x = torch.randn(M, K, generator=g) * 3
    gamma = 1 + 0.1 * torch.randn(K, generator=g)
    q, s, y = oracle.c_rmsnorm_quant_i8(x.numpy(), gamma.numpy(), 1e-5, want_y=True)
    yn = oracle.np_rmsnorm(x.numpy(), gamma.numpy(), 1e-5, epv=4)
    assert np.array_equal(y.view(np.uint32), yn.view(np.uint32))
    qn, sn = oracle.np_quant_rowwise_i8(yn)
    assert np.array_equal(q, qn) and np.array_equal(s.view(np.uint32), sn.view(np.uint32))
    # bf16 input: 8-element vectors
    xb, gb = x.to(torch.bfloat16), gamma.to(torch.bfloat16)
    q, s, y = oracle.c_rmsnorm_quant_i8(_bf16_bits(xb), _bf16_bits(gb), 1e-5, bf16_bits=True, want_y=True)
    yn = oracle.np_rmsnorm(xb.float().numpy(), gb.float().numpy(), 1e-5, epv=8)
    assert np.array_equal(y.view(np.uint32), yn.view(np.uint32))


def test_norm_matches_float64_and_torch_rms_norm_within_rounding(oracle):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(6, 2048, generator=g) * torch.tensor([1e-3, 1.0, 7.0, 100.0, 1e4, 0.3])[:, None]
    gamma = 1 + 0.2 * torch.randn(2048, generator=g)
    _, _, y = oracle.c_rmsnorm_quant_i8(x.numpy(), gamma.numpy(), 1e-5, want_y=True)
    x64, g64 = x.double().numpy(), gamma.double().numpy()
    exact = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + 1e-5) * g64
    assert np.max(np.abs(y - exact) / (np.abs(exact) + 1e-30)) < 4e-7       # a few fp32 roundings
    ref = F.rms_norm(x, (2048,), gamma, 1e-5).numpy()                        # the reference's call
    assert np.max(np.abs(y - ref) / (np.abs(ref) + 1e-30)) < 1e-6


def test_closed_forms(oracle):
    K = 256
    # constant row, unit gain, eps = 0: y = sign(c) exactly 1 in magnitude -> codes +-127, scale 1/127
    x = np.full((2, K), 3.0, np.float32)
    x[1] = -0.125
    q, s, y = oracle.c_rmsnorm_quant_i8(x, np.ones(K, np.float32), 0.0, want_y=True)
    assert np.all(y[0] == 1.0) and np.all(y[1] == -1.0)
    assert np.all(q[0] == 127) and np.all(q[1] == -127) and np.all(s == np.float32(1.0) / np.float32(127.0))
    # zero row: y = 0 (eps keeps the root finite), codes 0, scale 1
    q, s, y = oracle.c_rmsnorm_quant_i8(np.zeros((1, K), np.float32), np.ones(K, np.float32), 1e-5, want_y=True)
    assert not y.any() and not q.any() and s[0] == 1.0
    # scale invariance: x -> 4x (a power of two, eps = 0) changes nothing
    g = np.random.default_rng(0)
    a = g.standard_normal((3, K)).astype(np.float32)
    gam = (1 + 0.1 * g.standard_normal(K)).astype(np.float32)
    q1, s1 = oracle.c_rmsnorm_quant_i8(a, gam, 0.0)
    q2, s2 = oracle.c_rmsnorm_quant_i8(a * 4, gam, 0.0)
    assert np.array_equal(q1, q2) and np.array_equal(s1, s2)
    # the gain multiplies after the normalisation: one-hot gain isolates one column
    gam1 = np.zeros(K, np.float32)
    gam1[7] = 2.0
    q, s, y = oracle.c_rmsnorm_quant_i8(a, gam1, 0.0, want_y=True)
    assert np.count_nonzero(y) == 3 and np.all(np.abs(q[:, 7]) == 127)
    rms = np.sqrt((a.astype(np.float64) ** 2).mean(axis=1))
    assert np.allclose(y[:, 7], 2.0 * a[:, 7] / rms, rtol=1e-6)
