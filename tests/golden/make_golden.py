"""Writes the golden fixtures of the quantized-Linear path.

The reference (astrai/model/components/linear.py:20-21) holds no quantized
arithmetic and its tests pin no numeric output of Linear, so these vectors are
produced by this build's CPU oracle (whose functions are pinned independently
in tests/test_oracle_*.py) -- never by importing the reference.  Inputs are
seeded torch/numpy draws, so the fixtures can be regenerated bit for bit:

    python tests/golden/make_golden.py

small.npz      full tensors of a tiny case (M=8, K=64, N=16) for every stage
fused_small.npz  tiny cases of the operators between the projections: RMSNorm + quantise,
               SwiGLU + quantise, rotation + page write, decode attention over pages, causal
               prefill attention (from position 0 and on top of cached tokens)
config1.json   SHA-256 of the codes / scales / accumulators / outputs of
               benchmark configuration 1 (X 64x2048 with 4 outlier columns x20,
               W 2048x2048 N(0, 0.02), seed 0)
"""
import hashlib
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import oracle  # noqa: E402


def small_case():
    rng = np.random.default_rng(2024)
    M, K, N = 8, 64, 16
    x = rng.standard_normal((M, K)).astype(np.float32)
    x[:, 5] *= 20
    x[3] = 0
    x[4, :4] = [1.5, 2.5, -0.5, 127.0]  # with amax 127 these are exact ties
    x[4, 4:] = 0
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.01).astype(np.float32)
    xb = oracle.np_f32_to_bf16_bits(x)
    xq, sx = oracle.c_quant_rowwise_i8(x)
    xq_b, sx_b = oracle.c_quant_rowwise_i8(xb, bf16_bits=True)
    wq, sw = oracle.c_quant_rowwise_i8(w)
    acc = oracle.c_gemm_i8_i32(xq, wq)
    y = oracle.c_dequant_epilogue(acc, sx, sw, bias)
    y_bf16 = oracle.c_dequant_epilogue(acc, sx, sw, bias, bf16_out=True)
    y_from_bf16 = oracle.c_linear_w8a8(xb, wq, sw, None, x_bf16_bits=True, bf16_out=True)
    x8, s8x = oracle.c_quant_tensor_fp8(x)
    w8, s8w = oracle.c_quant_tensor_fp8(w)
    y8 = oracle.np_linear_fp8(x8, s8x, w8, s8w)
    return dict(x=x, w=w, bias=bias, x_bf16=xb, xq=xq, sx=sx, xq_from_bf16=xq_b, sx_from_bf16=sx_b, wq=wq, sw=sw,
                acc=acc, y=y, y_bf16=y_bf16, y_bf16_from_bf16_x=y_from_bf16, x_fp8=x8, sx_fp8=np.float32(s8x),
                w_fp8=w8, sw_fp8=np.float32(s8w), y_fp8_exact=y8)


def fused_case():
    rng = np.random.default_rng(7)
    bits = oracle.np_f32_to_bf16_bits
    # RMSNorm + quantise and SwiGLU + quantise on bf16 rows
    x = bits((rng.standard_normal((5, 96)) * 2).astype(np.float32))
    gamma = bits((rng.random(96) + 0.5).astype(np.float32))
    nq, ns = oracle.c_rmsnorm_quant_i8(x, gamma, 1e-5, bf16_bits=True)
    ug = bits((rng.standard_normal((4, 2 * 48)) * 3).astype(np.float32))
    hq, hs = oracle.c_swiglu_quant_i8(ug, bf16_bits=True)
    # one decode step on a paged cache: B = 2, 4 query / 2 KV heads of 64, 16-token pages, position 37
    B, Hq, Hkv, D, page, pos = 2, 4, 2, 64, 16, 37
    P, n_pages = 3, 8
    qkv = bits(rng.standard_normal((B, (Hq + 2 * Hkv) * D)).astype(np.float32))
    ang = (rng.random((B, D // 2)) * 6.28).astype(np.float32)
    freqs = np.stack([np.cos(ang), np.sin(ang)], -1).astype(np.float32)
    table = np.array([[5, 2, 7], [1, -1, 4]], np.int64)
    kc = bits(rng.standard_normal((n_pages, page, Hkv, D)).astype(np.float32))
    vc = bits(rng.standard_normal((n_pages, page, Hkv, D)).astype(np.float32))
    kc_after, vc_after = kc.copy(), vc.copy()
    q_rot = oracle.c_rope_kv_write(qkv, freqs, table, pos, kc_after, vc_after, Hq, Hkv)
    attn = oracle.c_paged_attn_decode(q_rot, kc_after, vc_after, table, pos + 1, D ** -0.5)
    # prefill attention: 9 tokens from position 0, and 5 tokens on top of 20 cached ones
    S = 9
    pq = bits(rng.standard_normal((B, S, Hq, D)).astype(np.float32))
    pk = bits(rng.standard_normal((B, S, Hkv, D)).astype(np.float32))
    pv = bits(rng.standard_normal((B, S, Hkv, D)).astype(np.float32))
    pout = oracle.c_prefill_attn_causal(pq, pk, pv, D ** -0.5)
    start, S2 = 20, 5
    cq = bits(rng.standard_normal((B, S2, Hq, D)).astype(np.float32))
    ck = bits(rng.standard_normal((B, start + S2, Hkv, D)).astype(np.float32))
    cv = bits(rng.standard_normal((B, start + S2, Hkv, D)).astype(np.float32))
    cout = oracle.c_prefill_attn_offset(cq, ck, cv, start, D ** -0.5)
    return dict(norm_x=x, norm_gamma=gamma, norm_codes=nq, norm_scale=ns, swiglu_ug=ug, swiglu_codes=hq, swiglu_scale=hs,
                rope_qkv=qkv, rope_freqs=freqs, table=table, pos=np.int64(pos), kc=kc, vc=vc, kc_after=kc_after,
                vc_after=vc_after, q_rot=q_rot, attn_decode=attn, pre_q=pq, pre_k=pk, pre_v=pv, pre_out=pout,
                chunk_q=cq, chunk_k=ck, chunk_v=cv, chunk_start=np.int64(start), chunk_out=cout)


def config1_inputs():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(64, 2048, generator=g)
    cols = torch.randperm(2048, generator=g)[:4]
    x[:, cols] *= 20
    w = torch.randn(2048, 2048, generator=g) * 0.02
    return x.numpy(), w.numpy()


def sha(a: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def config1_hashes():
    x, w = config1_inputs()
    xq, sx = oracle.c_quant_rowwise_i8(x)
    wq, sw = oracle.c_quant_rowwise_i8(w)
    acc = oracle.c_gemm_i8_i32(xq, wq)
    y = oracle.c_dequant_epilogue(acc, sx, sw)
    return {"x": sha(x), "w": sha(w), "xq": sha(xq), "sx": sha(sx), "wq": sha(wq), "sw": sha(sw),
            "acc": sha(acc), "y_f32": sha(y), "acc_sum": int(acc.astype(np.int64).sum())}


if __name__ == "__main__":
    np.savez(os.path.join(HERE, "small.npz"), **small_case())
    np.savez(os.path.join(HERE, "fused_small.npz"), **fused_case())
    with open(os.path.join(HERE, "config1.json"), "w") as f:
        json.dump(config1_hashes(), f, indent=1, sort_keys=True)
    print("wrote small.npz, fused_small.npz and config1.json")
