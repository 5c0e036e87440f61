"""Pins the oracle's SwiGLU -> row quantise (CPU).

``down(up(x) * silu(gate(x)))`` is the reference's MLP (astrai/model/components/mlp.py:24-27).
The fused form has no reference counterpart; its arithmetic (an exponential made of fused
multiply-adds, a correctly rounded divide) is checked against libm / float64, torch's F.silu,
the numpy restatement bit for bit, and closed forms.
"""
import numpy as np
import torch
import torch.nn.functional as F


def test_exp_repro_is_within_two_ulp_of_the_true_exponential(oracle):
    lib = oracle._load()
    xs = np.concatenate([np.linspace(-87, 87, 20001), np.array([0.0, -0.0, 1e-8, -1e-8, 0.6931472, -0.6931472, 100, -100])])
    got = np.array([lib.oq_exp_repro(float(x)) for x in xs.astype(np.float32)], np.float32)
    want = np.exp(np.clip(xs.astype(np.float32).astype(np.float64), -87, 87))
    ulp = np.spacing(want.astype(np.float32)).astype(np.float64)
    assert np.max(np.abs(got.astype(np.float64) - want) / ulp) <= 2.0
    assert lib.oq_exp_repro(0.0) == 1.0
    # the numpy restatement (float64 products rounded once = fma) gives the same bits
    assert np.array_equal(oracle.np_exp_repro(xs.astype(np.float32)).view(np.uint32), got.view(np.uint32))


def test_swiglu_matches_float64_torch_and_numpy(oracle):
    g = torch.Generator().manual_seed(3)
    M, Fh = 6, 1040
    ug = torch.randn(M, 2 * Fh, generator=g) * torch.tensor([0.01, 1, 3, 10, 40, 0.3])[:, None]
    q, s, h = oracle.c_swiglu_quant_i8(ug.numpy(), want_h=True)
    u64, g64 = ug[:, :Fh].double().numpy(), ug[:, Fh:].double().numpy()
    exact = u64 * g64 / (1 + np.exp(-g64))
    # |gate| > 87 is clamped inside the exponential: those products are below 1e-30 either way
    assert np.all(np.abs(h - exact) <= 1e-6 * np.abs(exact) + 1e-30)
    ref = (ug[:, :Fh] * F.silu(ug[:, Fh:])).numpy()                      # the reference's expression, fp32
    assert np.all(np.abs(h - ref) <= 2e-6 * np.abs(ref) + 1e-30)
    hn = oracle.np_swiglu(ug[:, :Fh].numpy(), ug[:, Fh:].numpy())
    assert np.array_equal(h.view(np.uint32), hn.view(np.uint32))
    qn, sn = oracle.np_quant_rowwise_i8(hn)
    assert np.array_equal(q, qn) and np.array_equal(s.view(np.uint32), sn.view(np.uint32))
    # bf16 input
    ub = ug.to(torch.bfloat16)
    bits = ub.contiguous().view(torch.int16).numpy().view(np.uint16)
    qb, sb, hb = oracle.c_swiglu_quant_i8(bits, bf16_bits=True, want_h=True)
    hn = oracle.np_swiglu(ub[:, :Fh].float().numpy(), ub[:, Fh:].float().numpy())
    assert np.array_equal(hb.view(np.uint32), hn.view(np.uint32))


def test_swiglu_closed_forms(oracle):
    Fh = 64
    ug = np.zeros((4, 2 * Fh), np.float32)
    ug[0, :Fh] = 5.0                      # gate = 0: silu(0) = 0 -> h = 0 -> zero row
    ug[1, :Fh] = 2.0
    ug[1, Fh:] = 200.0                    # large gate: silu(g) = g exactly (e underflows against 1)
    ug[2, :Fh] = 2.0
    ug[2, Fh:] = -200.0                   # very negative gate: h is tiny and negative
    ug[3, :Fh] = np.linspace(-1, 1, Fh)
    ug[3, Fh:] = 1.0                      # constant gate: h proportional to up
    q, s, h = oracle.c_swiglu_quant_i8(ug, want_h=True)
    assert not h[0].any() and not q[0].any() and s[0] == 1.0
    assert np.all(h[1] == 400.0) and np.all(q[1] == 127)
    assert np.all(h[2] < 0) and np.all(np.abs(h[2]) < 1e-30)
    silu1 = 1.0 / (1.0 + np.exp(-1.0))
    assert np.allclose(h[3], ug[3, :Fh] * silu1, rtol=1e-6)
    assert q[3, 0] == -127 and q[3, -1] == 127 and q[3, Fh // 2 - 1] == -q[3, Fh // 2]
