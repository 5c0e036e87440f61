"""GPU parity on seeded random shapes: the quantisers, the decode GEMV (with and without the norm in front, with and
without a bias) and the Linear on codes, at shapes drawn inside the documented limits rather than picked by hand,
bit for bit against the CPU oracle.  The draws are fixed by the seed, so a failure names a reproducible case."""
import random
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from khaosz_amd import ops  # noqa: E402

DEV = "cuda:0"


def _say(*a):
    print(*a, file=sys.stderr, flush=True)


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _rows(M, K, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g) * scale
    if K >= 8:
        x[:, torch.randperm(K, generator=g)[:max(1, K // 64)]] *= 15.0  # outlier columns
    return x


def _same_codes(q, s, qo, so):
    return np.array_equal(q.cpu().numpy(), qo) and np.array_equal(s.cpu().numpy().view(np.uint32), so.view(np.uint32))


@pytest.mark.parametrize("seed", [7, 11])
def test_quantisers_on_random_shapes(oracle, seed):
    rng = random.Random(seed)
    for it in range(30):
        bf = rng.random() < 0.6
        M, K = rng.randint(1, 300), 16 * rng.randint(1, 700)
        _say("quant_rowwise", M, K, bf)
        x = _rows(M, K, it).to(DEV, torch.bfloat16 if bf else torch.float32)
        q, s = ops.quant_rowwise_i8(x)
        qo, so = (oracle.c_quant_rowwise_i8(_bits(x), bf16_bits=True) if bf
                  else oracle.c_quant_rowwise_i8(x.cpu().numpy()))
        assert _same_codes(q, s, qo, so), ("quant_rowwise", M, K, bf)

        bf = rng.random() < 0.6
        M, K = rng.randint(1, 200), 16 * rng.randint(1, 512 if bf else 384)  # 24 vectors per lane at most
        _say("rmsnorm_quant", M, K, bf)
        dt = torch.bfloat16 if bf else torch.float32
        x = _rows(M, K, 100 + it).to(DEV, dt)
        gam = (1 + 0.2 * torch.randn(K, generator=torch.Generator().manual_seed(it))).to(DEV, dt)
        q, s = ops.rmsnorm_quant_rowwise_i8(x, gam, 1e-5)
        qo, so = (oracle.c_rmsnorm_quant_i8(_bits(x), _bits(gam), 1e-5, bf16_bits=True) if bf
                  else oracle.c_rmsnorm_quant_i8(x.cpu().numpy(), gam.cpu().numpy(), 1e-5))
        assert _same_codes(q, s, qo, so), ("rmsnorm_quant", M, K, bf)

        bf = rng.random() < 0.6
        M, F = rng.randint(1, 1300), 16 * rng.randint(1, 512 if bf else 256)  # 16 vector pairs per lane at most
        _say("swiglu_quant", M, F, bf)
        ug = _rows(M, 2 * F, 200 + it, 1.5).to(DEV, torch.bfloat16 if bf else torch.float32)
        q, s = ops.swiglu_quant_rowwise_i8(ug)
        qo, so = (oracle.c_swiglu_quant_i8(_bits(ug), bf16_bits=True) if bf
                  else oracle.c_swiglu_quant_i8(ug.cpu().numpy()))
        assert _same_codes(q, s, qo, so), ("swiglu_quant", M, F, bf)


@pytest.mark.parametrize("seed", [7, 11])
def test_decode_gemv_and_linear_on_random_shapes(oracle, seed):
    rng = random.Random(seed)
    for it in range(30):
        M, N, K = rng.randint(1, 16), rng.randint(1, 3000), 16 * rng.randint(1, 512)
        if rng.random() < 0.5:
            K = 256 * rng.randint(1, 32)  # the matrix-core kernels' K steps
        use_bias, use_norm = rng.random() < 0.5, rng.random() < 0.3
        _say("gemv_decode", M, N, K, use_bias, use_norm)
        x = _rows(M, K, 300 + it).to(torch.bfloat16)
        wq, sw = oracle.c_quant_rowwise_i8((_rows(N, K, 400 + it) * 0.02).numpy())
        b = torch.randn(N, generator=torch.Generator().manual_seed(it)) * 0.01 if use_bias else None
        wd, swd = torch.from_numpy(wq).to(DEV), torch.from_numpy(sw).to(DEV)
        bd, bn = (None, None) if b is None else (b.to(DEV), b.numpy())
        if use_norm:
            gam = (1 + 0.2 * torch.randn(K, generator=torch.Generator().manual_seed(it))).to(torch.bfloat16)
            y = ops.gemv_w8a8_decode(x.to(DEV), wd, swd, bd, out_dtype=torch.bfloat16, norm=(gam.to(DEV), 1e-5))
            qx, sx = oracle.c_rmsnorm_quant_i8(_bits(x), _bits(gam), 1e-5, bf16_bits=True)
            want = oracle.c_dequant_epilogue(oracle.c_gemm_i8_i32(qx, wq), sx, sw, bn, bf16_out=True)
        else:
            y = ops.gemv_w8a8_decode(x.to(DEV), wd, swd, bd, out_dtype=torch.bfloat16)
            want = oracle.c_linear_w8a8(_bits(x), wq, sw, bn, x_bf16_bits=True, bf16_out=True)
        assert np.array_equal(_bits(y), want), ("gemv_decode", M, N, K, use_bias, use_norm)

        M, N, K = rng.randint(17, 700), rng.randint(1, 1500), 16 * rng.randint(1, 256)
        f32_out = rng.random() < 0.3
        _say("linear_w8a8", M, N, K, f32_out)
        xq, sx = oracle.c_quant_rowwise_i8(_rows(M, K, 500 + it).numpy())
        wq, sw = oracle.c_quant_rowwise_i8((_rows(N, K, 600 + it) * 0.02).numpy())
        y = ops.linear_w8a8(torch.from_numpy(xq).to(DEV), torch.from_numpy(sx).to(DEV), torch.from_numpy(wq).to(DEV),
                            torch.from_numpy(sw).to(DEV), None, out_dtype=torch.float32 if f32_out else torch.bfloat16)
        want = oracle.c_dequant_epilogue(oracle.c_gemm_i8_i32(xq, wq), sx, sw, None, bf16_out=not f32_out)
        if f32_out:
            assert np.array_equal(y.cpu().numpy().view(np.uint32), want.view(np.uint32)), ("linear_w8a8", M, N, K)
        else:
            assert np.array_equal(_bits(y), want), ("linear_w8a8", M, N, K)
