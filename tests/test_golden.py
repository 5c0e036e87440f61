"""Golden fixtures (tests/golden/, written by make_golden.py from the CPU oracle):
the oracle must keep reproducing them on CPU, and the HIP path must reproduce
them on the GPU."""
import json
import os

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
G = os.path.join(HERE, "golden")


@pytest.fixture(scope="module")
def small():
    return dict(np.load(os.path.join(G, "small.npz")))


@pytest.fixture(scope="module")
def config1():
    import sys
    sys.path.insert(0, G)
    import make_golden

    x, w = make_golden.config1_inputs()
    return x, w, json.load(open(os.path.join(G, "config1.json"))), make_golden.sha


def test_oracle_reproduces_small_fixture(oracle, small):
    s = small
    for q, sc in (oracle.c_quant_rowwise_i8(s["x"]), oracle.np_quant_rowwise_i8(s["x"])):
        assert np.array_equal(q, s["xq"]) and np.array_equal(sc, s["sx"])
    q, sc = oracle.c_quant_rowwise_i8(s["x_bf16"], bf16_bits=True)
    assert np.array_equal(q, s["xq_from_bf16"]) and np.array_equal(sc, s["sx_from_bf16"])
    assert s["xq"][4, :4].tolist() == [2, 2, 0, 127] and s["sx"][4] == 1.0 and not s["xq"][3].any()
    assert np.array_equal(oracle.c_gemm_i8_i32(s["xq"], s["wq"]), s["acc"])
    assert np.array_equal(oracle.np_gemm_i8_i32(s["xq"], s["wq"]), s["acc"])
    assert np.array_equal(oracle.c_dequant_epilogue(s["acc"], s["sx"], s["sw"], s["bias"]), s["y"])
    assert np.array_equal(oracle.np_f32_to_bf16_bits(s["y"]), s["y_bf16"])
    q8, s8 = oracle.np_quant_tensor_fp8(s["x"])
    assert np.array_equal(q8, s["x_fp8"]) and s8 == s["sx_fp8"]


def test_oracle_reproduces_config1_hashes(oracle, config1):
    x, w, want, sha = config1
    assert sha(x) == want["x"] and sha(w) == want["w"], "the seeded inputs changed (torch RNG stream?)"
    xq, sx = oracle.c_quant_rowwise_i8(x)
    wq, sw = oracle.c_quant_rowwise_i8(w)
    acc = oracle.c_gemm_i8_i32(xq, wq)
    assert (sha(xq), sha(sx), sha(wq), sha(sw)) == (want["xq"], want["sx"], want["wq"], want["sw"])
    assert sha(acc) == want["acc"] and int(acc.astype(np.int64).sum()) == want["acc_sum"]
    assert sha(oracle.c_dequant_epilogue(acc, sx, sw)) == want["y_f32"]


@pytest.mark.gpu
def test_hip_reproduces_small_fixture(small):
    from khaosz_amd import ops

    s, dev = small, "cuda:0"
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    q, sc = ops.quant_rowwise_i8(t(s["x"]))
    assert np.array_equal(q.cpu().numpy(), s["xq"]) and np.array_equal(sc.cpu().numpy(), s["sx"])
    xb = t(s["x_bf16"].view(np.int16)).view(torch.bfloat16)
    q, sc = ops.quant_rowwise_i8(xb)
    assert np.array_equal(q.cpu().numpy(), s["xq_from_bf16"]) and np.array_equal(sc.cpu().numpy(), s["sx_from_bf16"])
    acc = ops.gemm_i8_i32(t(s["xq"]), t(s["wq"]))
    assert np.array_equal(acc.cpu().numpy(), s["acc"])
    y = ops.linear_w8a8(t(s["xq"]), t(s["sx"]), t(s["wq"]), t(s["sw"]), t(s["bias"]), out_dtype=torch.float32)
    assert np.array_equal(y.cpu().numpy(), s["y"])
    yb = ops.linear_w8a8(t(s["xq"]), t(s["sx"]), t(s["wq"]), t(s["sw"]), t(s["bias"]), out_dtype=torch.bfloat16)
    assert np.array_equal(yb.cpu().view(torch.int16).numpy().view(np.uint16), s["y_bf16"])
    yd = ops.gemv_w8a8_decode(xb, t(s["wq"]), t(s["sw"]), None, out_dtype=torch.bfloat16)
    assert np.array_equal(yd.cpu().view(torch.int16).numpy().view(np.uint16), s["y_bf16_from_bf16_x"])
    q8, s8 = ops.quant_tensor_fp8(t(s["x"]))
    assert np.array_equal(q8.cpu().numpy(), s["x_fp8"]) and np.float32(s8.item()) == s["sx_fp8"]
    y8 = ops.linear_fp8(t(s["x_fp8"]), t(np.array([s["sx_fp8"]])), t(s["w_fp8"]), t(np.array([s["sw_fp8"]])),
                        out_dtype=torch.float32)
    rms = float(np.sqrt(np.mean(s["y_fp8_exact"].astype(np.float64) ** 2)))
    assert np.max(np.abs(y8.cpu().numpy() - s["y_fp8_exact"])) <= 1e-3 * rms  # stated FP8 tolerance is 1e-2


@pytest.mark.gpu
def test_hip_reproduces_config1_hashes(config1):
    from khaosz_amd import ops

    x, w, want, sha = config1
    dev = "cuda:0"
    xq, sx = ops.quant_rowwise_i8(torch.from_numpy(x).to(dev))
    wq, sw = ops.quant_rowwise_i8(torch.from_numpy(w).to(dev))
    acc = ops.gemm_i8_i32(xq, wq)
    y = ops.linear_w8a8(xq, sx, wq, sw, None, out_dtype=torch.float32)
    got = {"xq": sha(xq.cpu().numpy()), "sx": sha(sx.cpu().numpy()), "wq": sha(wq.cpu().numpy()),
           "sw": sha(sw.cpu().numpy()), "acc": sha(acc.cpu().numpy()), "y_f32": sha(y.cpu().numpy())}
    assert got == {k: want[k] for k in got}


@pytest.fixture(scope="module")
def fused():
    return dict(np.load(os.path.join(G, "fused_small.npz")))


def _bf16_close(a_bits, b_bits, ulps=2):
    """bf16 bit patterns within a few units in the last place (libm's expf may differ between hosts)."""
    a = torch.from_numpy(a_bits.view(np.int16).copy()).view(torch.bfloat16).float()
    b = torch.from_numpy(b_bits.view(np.int16).copy()).view(torch.bfloat16).float()
    return bool(((a - b).abs() <= ulps * 2.0 ** -8 * b.abs().clamp(min=2.0 ** -6)).all())


def test_oracle_reproduces_fused_fixture(oracle, fused):
    f = fused
    q, s = oracle.c_rmsnorm_quant_i8(f["norm_x"], f["norm_gamma"], 1e-5, bf16_bits=True)
    assert np.array_equal(q, f["norm_codes"]) and np.array_equal(s, f["norm_scale"])
    q, s = oracle.c_swiglu_quant_i8(f["swiglu_ug"], bf16_bits=True)
    assert np.array_equal(q, f["swiglu_codes"]) and np.array_equal(s, f["swiglu_scale"])
    kc, vc = f["kc"].copy(), f["vc"].copy()
    qr = oracle.c_rope_kv_write(f["rope_qkv"], f["rope_freqs"], f["table"], int(f["pos"]), kc, vc, 4, 2)
    assert np.array_equal(qr, f["q_rot"]) and np.array_equal(kc, f["kc_after"]) and np.array_equal(vc, f["vc_after"])
    # position 37 = slot 5 of logical page 2: pages 7 (sequence 0) and 4 (sequence 1) took the new rows, nothing else
    changed = {(int(p), int(sl)) for p, sl in zip(*np.nonzero((kc != f["kc"]).any(axis=(2, 3))))}
    assert changed == {(7, 5), (4, 5)}
    out = oracle.c_paged_attn_decode(f["q_rot"], f["kc_after"], f["vc_after"], f["table"], int(f["pos"]) + 1, 0.125)
    assert _bf16_close(out, f["attn_decode"])
    assert _bf16_close(oracle.c_prefill_attn_causal(f["pre_q"], f["pre_k"], f["pre_v"], 0.125), f["pre_out"])
    assert _bf16_close(oracle.c_prefill_attn_offset(f["chunk_q"], f["chunk_k"], f["chunk_v"], int(f["chunk_start"]), 0.125),
                       f["chunk_out"])


@pytest.mark.gpu
def test_hip_reproduces_fused_fixture(fused):
    from khaosz_amd import ops

    f, dev = fused, "cuda:0"
    bf = lambda a: torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16).to(dev)
    bits = lambda t: t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)
    q, s = ops.rmsnorm_quant_rowwise_i8(bf(f["norm_x"]), bf(f["norm_gamma"]), 1e-5)
    assert np.array_equal(q.cpu().numpy(), f["norm_codes"]) and np.array_equal(s.cpu().numpy(), f["norm_scale"])
    q, s = ops.swiglu_quant_rowwise_i8(bf(f["swiglu_ug"]))
    assert np.array_equal(q.cpu().numpy(), f["swiglu_codes"]) and np.array_equal(s.cpu().numpy(), f["swiglu_scale"])
    kc, vc = bf(f["kc"]), bf(f["vc"])
    fr = torch.from_numpy(f["rope_freqs"].copy())
    freqs = torch.view_as_complex(fr).to(dev)
    table = torch.from_numpy(f["table"].copy()).to(dev)
    pos = int(f["pos"])
    qr = ops.rope_kv_write(bf(f["rope_qkv"]), freqs, table, pos, kc, vc, 4, 2)
    assert np.array_equal(bits(qr), f["q_rot"]) and np.array_equal(bits(kc), f["kc_after"])
    assert np.array_equal(bits(vc), f["vc_after"])
    out = ops.paged_attn_decode(qr, kc, vc, table, pos + 1)
    tol = lambda t, want: torch.allclose(t.float().cpu(), torch.from_numpy(want.view(np.int16).copy()).view(torch.bfloat16).float(),
                                         rtol=1e-2, atol=1e-2)   # the stated tolerance of the attention kernels
    assert tol(out, f["attn_decode"])
    kc2, vc2 = bf(f["kc"]), bf(f["vc"])
    fused_out = ops.rope_paged_attn_decode(bf(f["rope_qkv"]), freqs, table, pos + 1, kc2, vc2, 4, 2)
    assert torch.equal(fused_out, out) and np.array_equal(bits(kc2), f["kc_after"])
    pre = ops.prefill_attn_causal(bf(f["pre_q"]), bf(f["pre_k"]), bf(f["pre_v"]))
    assert tol(pre, f["pre_out"])
    # the chunk on top of cached tokens: its keys and values laid into pages first
    ck, cv, start = bf(f["chunk_k"]), bf(f["chunk_v"]), int(f["chunk_start"])
    B, T, Hkv, D = ck.shape
    page, P = 8, (T + 7) // 8
    kp = torch.zeros(B * P, page, Hkv, D, dtype=torch.bfloat16, device=dev)
    vp = torch.zeros_like(kp)
    tb = torch.arange(B * P, device=dev).view(B, P).flip(1).contiguous()
    for b in range(B):
        for t in range(T):
            kp[tb[b, t // page], t % page], vp[tb[b, t // page], t % page] = ck[b, t], cv[b, t]
    got = ops.prefill_attn_paged(bf(f["chunk_q"]), kp, vp, tb, start)
    assert tol(got, f["chunk_out"])
