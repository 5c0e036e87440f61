"""Decode-step attention kernels against the oracle, through the C ABI (GPU)."""
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
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16).copy()


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("B,Hq,Hkv,page,pos", [(1, 1, 1, 4, 0), (3, 4, 2, 8, 13), (8, 16, 4, 64, 575), (5, 8, 1, 16, 31)])
def test_rope_kv_write_bit_exact(oracle, B, Hq, Hkv, page, pos, D):
    _say("rope_kv_write", B, Hq, Hkv, page, pos, D)
    P = pos // page + 2
    n_pages = B * P + 3
    g = torch.Generator().manual_seed(B * 100 + pos)
    qkv = torch.randn(B, (Hq + 2 * Hkv) * D, generator=g).to(torch.bfloat16)
    ang = torch.rand(B, D // 2, generator=g) * 6.28
    freqs = torch.polar(torch.ones_like(ang), ang)
    table = torch.randperm(n_pages, generator=g)[:B * P].view(B, P)
    if B > 2:
        table[1, pos // page] = -1                      # this sequence's token has no page: skipped
    kc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16)
    vc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16)
    kb, vb = _bits(kc), _bits(vc)
    qo = oracle.c_rope_kv_write(_bits(qkv), torch.view_as_real(freqs).numpy(), table.numpy(), pos, kb, vb, Hq, Hkv)
    kd, vd = kc.to(DEV), vc.to(DEV)
    q = ops.rope_kv_write(qkv.to(DEV), freqs.to(DEV), table.to(DEV), pos, kd, vd, Hq, Hkv)
    assert np.array_equal(_bits(q), qo)
    assert np.array_equal(_bits(kd), kb) and np.array_equal(_bits(vd), vb)


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("B,S,Hq,Hkv,page,pos", [(1, 5, 1, 1, 4, 0), (3, 21, 4, 2, 8, 13), (2, 130, 16, 4, 64, 0)])
def test_rope_kv_write_several_tokens_bit_exact(oracle, B, S, Hq, Hkv, page, pos, D):
    """A prompt (or a chunk of one) in one launch: the oracle applied token by token."""
    _say("rope_kv_write seq", B, S, Hq, Hkv, page, pos, D)
    P = (pos + S + page - 1) // page + 1
    n_pages = B * P + 3
    g = torch.Generator().manual_seed(B * 100 + S)
    qkv = torch.randn(B, S, (Hq + 2 * Hkv) * D, generator=g).to(torch.bfloat16)
    ang = torch.rand(B, S, D // 2, generator=g) * 6.28
    freqs = torch.polar(torch.ones_like(ang), ang)
    table = torch.randperm(n_pages, generator=g)[:B * P].view(B, P)
    if B > 2:
        table[1, (pos + 3) // page] = -1                # tokens of that page are dropped
    kc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16)
    vc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16)
    kb, vb = _bits(kc), _bits(vc)
    fr = torch.view_as_real(freqs).numpy()
    qo = np.stack([oracle.c_rope_kv_write(_bits(qkv[:, s]), np.ascontiguousarray(fr[:, s]), table.numpy(), pos + s,
                                          kb, vb, Hq, Hkv) for s in range(S)], axis=1)
    kd, vd = kc.to(DEV), vc.to(DEV)
    q, k = ops.rope_kv_write(qkv.to(DEV), freqs.to(DEV), table.to(DEV), pos, kd, vd, Hq, Hkv, return_k=True)
    assert q.shape == (B, S, Hq, D) and k.shape == (B, S, Hkv, D)
    assert np.array_equal(_bits(q), qo.reshape(B, S, Hq, D))
    assert np.array_equal(_bits(kd), kb) and np.array_equal(_bits(vd), vb)
    # the returned keys are what went into the mapped slots
    mapped = table[torch.arange(B)[:, None], (pos + torch.arange(S))[None, :] // page] >= 0
    slot = (table[torch.arange(B)[:, None], (pos + torch.arange(S))[None, :] // page].clamp(min=0),
            ((pos + torch.arange(S)) % page)[None, :].expand(B, -1))
    assert torch.equal(k.cpu()[mapped], kd.cpu()[slot[0], slot[1]][mapped])
    # one table shared by all sequences (batch stride 0)
    shared = freqs[:1].expand(B, -1, -1)
    qs = ops.rope_kv_write(qkv.to(DEV), shared.to(DEV), table.to(DEV), pos, kd, vd, Hq, Hkv)
    qw = ops.rope_kv_write(qkv.to(DEV), shared.contiguous().to(DEV), table.to(DEV), pos, kd, vd, Hq, Hkv)
    assert torch.equal(qs, qw)


@pytest.mark.parametrize("B,Hq,Hkv,page,T", [(1, 1, 1, 4, 1), (2, 8, 2, 16, 70), (8, 16, 4, 64, 576), (3, 8, 1, 16, 1000),
                                              (2, 4, 2, 64, 513), (1, 2, 2, 8, 64), (2, 2, 1, 4, 65), (1, 4, 4, 32, 256),
                                              (2, 16, 2, 16, 257), (40, 8, 8, 16, 300), (1, 8, 1, 64, 5000),
                                              (4, 24, 4, 128, 640), (2, 6, 2, 16, 100)])
@pytest.mark.parametrize("D", [128, 64])
def test_paged_attn_decode_within_bf16_rounding(oracle, B, Hq, Hkv, page, T, D):
    _say("paged_attn_decode", B, Hq, Hkv, page, T, D)
    P = (T + page - 1) // page
    n_pages = B * P + 2
    g = torch.Generator().manual_seed(T)
    q = (torch.randn(B, Hq, D, generator=g) * 1.5).to(torch.bfloat16)
    kc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16)
    vc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16)
    table = torch.randperm(n_pages, generator=g)[:B * P].view(B, P)
    if P > 2:
        table[B - 1, 1] = -1                             # an unmapped page in the middle: zero keys and values
    want = torch.from_numpy(oracle.c_paged_attn_decode(_bits(q), _bits(kc), _bits(vc), table.numpy(), T,
                                                       D ** -0.5).view(np.int16)).view(torch.bfloat16).float()
    out = ops.paged_attn_decode(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), T).cpu().float()
    # stated tolerance: 1e-2 relative for bf16 outputs (different summation order, exp2 instead of exp)
    assert torch.allclose(out, want, rtol=1e-2, atol=1e-2)
    assert ((out - want).norm() / want.norm()).item() < 4e-3


@pytest.mark.parametrize("B,Hq,Hkv,page,T,D,lens", [
    (3, 4, 2, 16, 61, 64, [61, 1, 33]),
    (4, 16, 4, 64, 700, 128, [700, 5, 256, 513]),       # three slices: one sequence ends inside the first, one on a boundary
    (2, 8, 8, 32, 300, 128, [0, 299]),                  # nothing visible: the reference's uniform average
])
def test_paged_attn_decode_sequences_at_different_positions(oracle, B, Hq, Hkv, page, T, D, lens):
    """seq_lens: sequence b attends to its first lens[b] positions (the reference's position mask for a decode
    batch at mixed positions), against the oracle; slices that lie wholly past a sequence's length drop out of
    the merge.  Both the plain kernel and the one that also rotates and writes the new token."""
    _say("paged_attn_decode lens", B, Hq, Hkv, page, T, D, lens)
    P = (T + page - 1) // page
    n_pages = B * P + 2
    g = torch.Generator().manual_seed(T + 1)
    q = (torch.randn(B, Hq, D, generator=g) * 1.5).to(torch.bfloat16)
    kc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16)
    vc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16)
    table = torch.randperm(n_pages, generator=g)[:B * P].view(B, P)
    lens_t = torch.tensor(lens, dtype=torch.int64)
    want = torch.from_numpy(oracle.c_paged_attn_decode(_bits(q), _bits(kc), _bits(vc), table.numpy(), T, D ** -0.5,
                                                       seq_lens=lens_t.numpy()).view(np.int16)).view(torch.bfloat16).float()
    out = ops.paged_attn_decode(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), T, seq_lens=lens_t.to(DEV)).cpu().float()
    assert torch.allclose(out, want, rtol=1e-2, atol=1e-2)
    assert ((out - want).norm() / want.norm()).item() < 4e-3
    # the fused form (rotation + write of the new token at T - 1 + attention) against rope_kv_write + the plain kernel
    qkv = torch.randn(B, (Hq + 2 * Hkv) * D, generator=g).to(torch.bfloat16).to(DEV)
    ang = torch.rand(B, D // 2, generator=g) * 6.28
    freqs = torch.polar(torch.ones_like(ang), ang).to(DEV)
    k1, v1, k2, v2 = kc.to(DEV), vc.to(DEV), kc.to(DEV), vc.to(DEV)
    q1 = ops.rope_kv_write(qkv, freqs, table.to(DEV), T - 1, k1, v1, Hq, Hkv)
    a = ops.paged_attn_decode(q1.view(B, Hq, D), k1, v1, table.to(DEV), T, seq_lens=lens_t.to(DEV))
    b = ops.rope_paged_attn_decode(qkv, freqs, table.to(DEV), T, k2, v2, Hq, Hkv, seq_lens=lens_t.to(DEV))
    assert torch.equal(a, b) and torch.equal(k1, k2) and torch.equal(v1, v2)


def test_paged_attn_workspace_reuse_and_checks(oracle):
    """A caller-owned workspace gives the same bits as a per-call one; a short one is refused."""
    _say("paged_attn_workspace")
    from khaosz_amd import _abi
    B, Hq, Hkv, page, T, D = 4, 8, 2, 16, 700, 128
    P = (T + page - 1) // page
    g = torch.Generator().manual_seed(5)
    q = torch.randn(B, Hq, D, generator=g).to(torch.bfloat16).to(DEV)
    kc = torch.randn(B * P, page, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    vc = torch.randn(B * P, page, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    table = torch.randperm(B * P, generator=g).view(B, P).to(DEV)
    need = ops.paged_attn_workspace_bytes(B, Hq, Hkv, T)
    assert need > 0 and need % 16 == 0
    assert ops.paged_attn_workspace_bytes(1, 1, 1, 10) == 0
    ws = torch.full((need // 4 + 64,), float("nan"), device=DEV)      # stale contents must not matter
    a = ops.paged_attn_decode(q, kc, vc, table, T)
    b = ops.paged_attn_decode(q, kc, vc, table, T, workspace=ws)
    c = ops.paged_attn_decode(q, kc, vc, table, T, workspace=ws)
    assert torch.equal(a, b) and torch.equal(a, c)
    out = torch.empty_like(q)
    lib = _abi.load()
    args = (q.data_ptr(), kc.data_ptr(), vc.data_ptr(), table.data_ptr(), P, T, None, page, B * P, D ** -0.5,
            out.data_ptr(), B, Hq, Hkv, D)
    assert lib.aq_paged_attn_decode(*args, ws.data_ptr(), need - 16, None) == -5    # AQ_E_WORKSPACE
    assert lib.aq_paged_attn_decode(*args, None, 0, None) == -1                  # AQ_E_NULL
    torch.cuda.synchronize()


@pytest.mark.parametrize("B,Hq,Hkv,page,T", [(1, 1, 1, 4, 1), (2, 8, 2, 16, 70), (8, 16, 4, 64, 576), (3, 8, 1, 16, 1000),
                                              (2, 4, 2, 64, 513), (2, 2, 1, 4, 65), (1, 4, 4, 32, 256), (5, 16, 2, 16, 257),
                                              (4, 24, 4, 128, 640), (2, 6, 2, 16, 100)])
@pytest.mark.parametrize("D", [128, 64])
def test_rope_paged_attn_decode_equals_the_two_launches(B, Hq, Hkv, page, T, D):
    """The fused decode step (rotate, write the new token, attend) against rope_kv_write followed by
    paged_attn_decode: caches and outputs bit for bit, including a sequence whose new page is unmapped."""
    _say("rope_paged_attn_decode", B, Hq, Hkv, page, T, D)
    P = (T + page - 1) // page
    n_pages = B * P + 2
    g = torch.Generator().manual_seed(T + 1)
    qkv = torch.randn(B, (Hq + 2 * Hkv) * D, generator=g).to(torch.bfloat16).to(DEV)
    ang = torch.rand(B, D // 2, generator=g) * 6.28
    freqs = torch.polar(torch.ones_like(ang), ang).to(DEV)
    kc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    vc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    table = torch.randperm(n_pages, generator=g)[:B * P].view(B, P)
    if B > 2:
        table[1, (T - 1) // page] = -1
    table = table.to(DEV)
    k1, v1, k2, v2 = kc.clone(), vc.clone(), kc.clone(), vc.clone()
    q = ops.rope_kv_write(qkv, freqs, table, T - 1, k1, v1, Hq, Hkv)
    want = ops.paged_attn_decode(q, k1, v1, table, T)
    out = ops.rope_paged_attn_decode(qkv, freqs, table, T, k2, v2, Hq, Hkv)
    assert torch.equal(k1, k2) and torch.equal(v1, v2)
    assert not torch.equal(k1, kc)
    assert torch.equal(out, want)
    # one rotary table shared by the batch (stride 0)
    if B > 1:
        shared = freqs[:1].expand(B, -1)
        q = ops.rope_kv_write(qkv, shared, table, T - 1, k1, v1, Hq, Hkv)
        want = ops.paged_attn_decode(q, k1, v1, table, T)
        assert torch.equal(ops.rope_paged_attn_decode(qkv, shared, table, T, k2, v2, Hq, Hkv), want)
        assert torch.equal(k1, k2) and torch.equal(v1, v2)


@pytest.mark.parametrize("B,S,Hq,Hkv,D", [(1, 1, 1, 1, 64), (2, 37, 6, 2, 64), (1, 129, 4, 4, 128), (2, 300, 8, 2, 128),
                                          (4, 512, 24, 4, 64), (1, 640, 4, 1, 128), (3, 64, 3, 1, 64)])
def test_prefill_attn_causal_within_bf16_rounding(oracle, B, S, Hq, Hkv, D):
    _say("prefill_attn_causal", B, S, Hq, Hkv, D)
    g = torch.Generator().manual_seed(S + D)
    q = (torch.randn(B, S, Hq, D, generator=g) * 1.5).to(torch.bfloat16)
    # k contiguous, v a strided view into a wider tensor (as in the fused q/k/v projection's output)
    k = torch.randn(B, S, Hkv, D, generator=g).to(torch.bfloat16)
    wide = torch.randn(B, S, (Hq + 2 * Hkv) * D, generator=g).to(torch.bfloat16)
    v = wide[..., (Hq + Hkv) * D:].view(B, S, Hkv, D)
    want = torch.from_numpy(oracle.c_prefill_attn_causal(_bits(q), _bits(k), _bits(v.contiguous()), D ** -0.5)
                            .view(np.int16)).view(torch.bfloat16).float()
    wd = wide.to(DEV)
    out = ops.prefill_attn_causal(q.to(DEV), k.to(DEV), wd[..., (Hq + Hkv) * D:].view(B, S, Hkv, D)).cpu().float()
    # stated tolerance: 1e-2 for bf16 outputs (probabilities rounded to bf16, exp2, block-wise summation)
    assert torch.allclose(out, want, rtol=1e-2, atol=1e-2)
    assert ((out - want).norm() / want.norm()).item() < 5e-3


def test_attn_argument_checks():
    q = torch.zeros(2, 4, 32, dtype=torch.bfloat16, device=DEV)
    kc = torch.zeros(4, 8, 2, 32, dtype=torch.bfloat16, device=DEV)
    tab = torch.zeros(2, 2, dtype=torch.int64, device=DEV)
    with pytest.raises(ValueError):
        ops.paged_attn_decode(q, kc, kc.clone(), tab, 5)          # head dimension 32 is not supported
    q = torch.zeros(2, 10, 128, dtype=torch.bfloat16, device=DEV)
    kc = torch.zeros(4, 8, 2, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError):
        ops.paged_attn_decode(q, kc, kc.clone(), tab, 5)          # 5 query heads per KV head


@pytest.mark.parametrize("B,Hq,Hkv,page,T", [(1, 8, 2, 16, 1), (4, 24, 4, 128, 640), (8, 16, 4, 64, 576), (3, 8, 1, 16, 1000),
                                              (2, 4, 2, 64, 513), (5, 16, 2, 16, 257), (7, 6, 2, 16, 100), (8, 8, 8, 32, 1024), (2, 32, 8, 16, 300)])
@pytest.mark.parametrize("D", [128, 64])
def test_output_projection_on_attention_partials_equals_the_three_launches(B, Hq, Hkv, page, T, D):
    """attention stopped before its merge + the output projection that combines the slices itself,
    against attention (with its merge launch) + the decode GEMV: outputs bit for bit, with and
    without a residual, bf16 and fp32 outputs; the caches see the same writes."""
    _say("gemv_w8a8_attn", B, Hq, Hkv, page, T, D)
    P = (T + page - 1) // page
    n_pages = B * P + 2
    K, N = Hq * D, 200
    g = torch.Generator().manual_seed(T + D)
    qkv = torch.randn(B, (Hq + 2 * Hkv) * D, generator=g).to(torch.bfloat16).to(DEV)
    ang = torch.rand(B, D // 2, generator=g) * 6.28
    freqs = torch.polar(torch.ones_like(ang), ang).to(DEV)
    kc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    vc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    table = torch.randperm(n_pages, generator=g)[:B * P].view(B, P)
    if B > 2 and P > 1:
        table[1, 0] = -1                                  # a hole: zero keys and values there
    table = table.to(DEV)
    wq = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8).to(DEV)
    sw = (torch.rand(N, generator=g) * 0.01 + 1e-3).to(DEV)
    bias = torch.randn(N, generator=g).to(DEV)
    k1, v1, k2, v2 = kc.clone(), vc.clone(), kc.clone(), vc.clone()
    # can (limits of the in-kernel merge) and should (every workgroup repeats the merge: only while it is small)
    assert ops.attn_gemv_fusable(B, Hq, D, T) == (K <= 2048 and T > 256 and B * K * ((T + 255) // 256) <= 32768)
    attn = ops.rope_paged_attn_decode(qkv, freqs, table, T, k1, v1, Hq, Hkv)
    if K > 2048:
        parts = ops.rope_paged_attn_decode(qkv, freqs, table, T, k2, v2, Hq, Hkv, partials=True)
        with pytest.raises(ValueError):
            ops.gemv_w8a8_attn(parts, wq, sw)
        return
    parts = ops.rope_paged_attn_decode(qkv, freqs, table, T, k2, v2, Hq, Hkv, partials=True)
    assert parts.n_slices == (T + 255) // 256 and (parts.B, parts.n_heads, parts.head_dim) == (B, Hq, D)
    assert torch.equal(k1, k2) and torch.equal(v1, v2)
    for dt in (torch.bfloat16, torch.float32):
        res = torch.randn(B, N, generator=g).to(dt).to(DEV)
        for b_, r_ in ((None, None), (bias, res)):
            want = ops.gemv_w8a8_decode(attn.view(B, K), wq, sw, b_, out_dtype=dt, residual=r_)
            got = ops.gemv_w8a8_attn(parts, wq, sw, b_, out_dtype=dt, residual=r_)
            assert torch.equal(got, want)


def test_attention_partials_entry_points_check_their_arguments():
    from khaosz_amd import _abi
    lib = _abi.load()
    _say("attention partials checks")
    assert lib.aq_paged_attn_decode_slices(0) == 0 and lib.aq_paged_attn_decode_slices(256) == 1
    assert lib.aq_paged_attn_decode_slices(257) == 2
    assert lib.aq_paged_attn_decode_partials_bytes(2, 4, 300) == 2 * 4 * 2 * 132 * 4
    buf = torch.zeros(4096, dtype=torch.float32, device=DEV)
    w = torch.zeros(64, 2048, dtype=torch.int8, device=DEV)
    sw = torch.ones(64, device=DEV)
    y = torch.zeros(8, 64, dtype=torch.bfloat16, device=DEV)
    call = lambda ns, d, m, k: lib.aq_gemv_w8a8_decode_attn(buf.data_ptr(), ns, d, w.data_ptr(), sw.data_ptr(), None, 0,
                                                            None, y.data_ptr(), 1, m, 64, k, None)
    assert call(5, 128, 1, 2048) == -6      # more slices than the kernel holds: AQ_E_RANGE
    assert call(1, 128, 9, 2048) == -6      # more rows
    assert call(1, 128, 1, 4096) == -6      # longer rows
    assert call(1, 96, 1, 1920) == -2       # head dimension: AQ_E_SHAPE
    assert call(1, 128, 1, 2000) == -2      # K not whole heads
    assert call(0, 128, 1, 2048) == -2
    # partial results need their buffer even for one slice
    q = torch.zeros(1, 2, 64, dtype=torch.bfloat16, device=DEV)
    kc = torch.zeros(2, 16, 1, 64, dtype=torch.bfloat16, device=DEV)
    tb = torch.zeros(1, 1, dtype=torch.int64, device=DEV)
    rc = lib.aq_paged_attn_decode_partials(q.data_ptr(), kc.data_ptr(), kc.data_ptr(), tb.data_ptr(), 1, 10, None, 16, 2, 0.125,
                                           1, 2, 1, 64, None, 0, None)
    assert rc == -1                         # AQ_E_NULL
    rc = lib.aq_paged_attn_decode_partials(q.data_ptr(), kc.data_ptr(), kc.data_ptr(), tb.data_ptr(), 1, 10, None, 16, 2, 0.125,
                                           1, 2, 1, 64, buf.data_ptr(), 64, None)
    assert rc == -5                         # AQ_E_WORKSPACE


@pytest.mark.parametrize("B,S,start,Hq,Hkv,page", [(1, 1, 0, 1, 1, 4), (2, 37, 0, 6, 2, 16), (2, 40, 100, 8, 2, 16), (3, 130, 257, 4, 1, 64),
                                                    (4, 200, 312, 24, 4, 128), (1, 300, 5, 4, 4, 32), (2, 64, 64, 3, 1, 8)])
@pytest.mark.parametrize("D", [128, 64])
def test_prefill_attn_paged_within_bf16_rounding(oracle, B, S, start, Hq, Hkv, page, D):
    """A chunk of S new tokens over start cached ones, K / V read through the page table (one sequence
    with an unmapped page: zero keys and values there), against the oracle on the gathered rows."""
    _say("prefill_attn_paged", B, S, start, Hq, Hkv, page, D)
    T = start + S
    P = (T + page - 1) // page + 1
    n_pages = B * P + 2
    g = torch.Generator().manual_seed(S + start + D)
    q = (torch.randn(B, S, Hq, D, generator=g) * 1.5).to(torch.bfloat16)
    kc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16)
    vc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16)
    table = torch.randperm(n_pages, generator=g)[:B * P].view(B, P)
    if B > 1 and T > page:
        table[1, 0] = -1
    # what gather gives: [B, T, Hkv, D], zeros where unmapped
    idx = torch.arange(T)
    rows = []
    for b in range(B):
        phys = table[b, idx // page]
        kk, vv = kc[phys.clamp(min=0), idx % page], vc[phys.clamp(min=0), idx % page]
        kk[phys < 0], vv[phys < 0] = 0, 0
        rows.append((kk, vv))
    k = torch.stack([r[0] for r in rows])
    v = torch.stack([r[1] for r in rows])
    want = torch.from_numpy(oracle.c_prefill_attn_offset(_bits(q), _bits(k), _bits(v), start, D ** -0.5)
                            .view(np.int16)).view(torch.bfloat16).float()
    out = ops.prefill_attn_paged(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), start).cpu().float()
    assert torch.allclose(out, want, rtol=1e-2, atol=1e-2)      # stated tolerance for bf16 outputs
    assert ((out - want).norm() / want.norm()).item() < 5e-3
    if start == 0 and not (table < 0).any():                     # on an empty cache: the contiguous kernel's bits
        same = ops.prefill_attn_causal(q.to(DEV), k.to(DEV), v.to(DEV)).cpu().float()
        assert torch.equal(out, same)


def test_prefill_attn_paged_checks_its_arguments():
    from khaosz_amd import _abi
    lib = _abi.load()
    q = torch.zeros(1, 4, 2, 64, dtype=torch.bfloat16, device=DEV)
    kc = torch.zeros(3, 16, 1, 64, dtype=torch.bfloat16, device=DEV)
    tb = torch.zeros(1, 2, dtype=torch.int64, device=DEV)
    out = torch.zeros_like(q)
    call = lambda start, S, P=2, D=64: lib.aq_prefill_attn_paged(q.data_ptr(), 128, kc.data_ptr(), kc.data_ptr(), tb.data_ptr(),
                                                                 P, start, 16, 3, out.data_ptr(), 0.125, 1, S, 2, 1, D, None)
    assert call(0, 4) == 0
    assert call(29, 4) == -2        # positions past the page table: AQ_E_SHAPE
    assert call(-1, 4) == -2
    assert call(0, 4, D=96) == -2
    with pytest.raises(ValueError):
        ops.prefill_attn_paged(q, kc, kc, tb, 30)


def _gains(D, g):
    return ((1.0 + 0.3 * torch.randn(D, generator=g)).to(torch.bfloat16),
            (1.0 + 0.3 * torch.randn(D, generator=g)).to(torch.bfloat16))


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("B,S,Hq,Hkv,page,pos", [(1, 1, 1, 1, 4, 0), (3, 1, 4, 2, 8, 13), (3, 21, 4, 2, 8, 13),
                                                 (2, 130, 16, 4, 64, 0), (5, 1, 8, 1, 16, 31)])
def test_rope_kv_write_qknorm_bit_exact(oracle, B, S, Hq, Hkv, page, pos, D):
    """Rotation, RMSNorm of the rotated q and k heads, page writes: q, the cached keys and values bit for bit
    against the oracle applied token by token (attention.py:86-92: the normalised key is what is cached)."""
    _say("rope_kv_write_qknorm", B, S, Hq, Hkv, page, pos, D)
    P = (pos + S + page - 1) // page + 1
    n_pages = B * P + 3
    g = torch.Generator().manual_seed(B * 100 + S + D)
    qkv = (torch.randn(B, S, (Hq + 2 * Hkv) * D, generator=g) * 1.5).to(torch.bfloat16)
    ang = torch.rand(B, S, D // 2, generator=g) * 6.28
    freqs = torch.polar(torch.ones_like(ang), ang)
    qg, kg = _gains(D, g)
    eps = 1e-5
    table = torch.randperm(n_pages, generator=g)[:B * P].view(B, P)
    if B > 2:
        table[1, (pos + S // 2) // page] = -1
    kc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16)
    vc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16)
    kb, vb = _bits(kc), _bits(vc)
    fr = torch.view_as_real(freqs).numpy()
    qo = np.stack([oracle.c_rope_kv_write(_bits(qkv[:, s]), np.ascontiguousarray(fr[:, s]), table.numpy(), pos + s,
                                          kb, vb, Hq, Hkv, qk_norm=(_bits(qg), _bits(kg), eps)) for s in range(S)], 1)
    kd, vd = kc.to(DEV), vc.to(DEV)
    norm = ops.QkNorm(qg.to(DEV), kg.to(DEV), eps)
    q, k = ops.rope_kv_write(qkv.to(DEV), freqs.to(DEV), table.to(DEV), pos, kd, vd, Hq, Hkv, return_k=True,
                             qk_norm=norm)
    assert np.array_equal(_bits(q), qo)
    assert np.array_equal(_bits(kd), kb) and np.array_equal(_bits(vd), vb)
    # the returned keys are the cached ones
    for b in range(B):
        for s in range(S):
            phys = int(table[b, (pos + s) // page])
            if phys >= 0:
                assert torch.equal(k[b, s], kd[phys, (pos + s) % page])
    # without the norm the same call stores other bits: the argument is not ignored
    k2, v2 = kc.to(DEV), vc.to(DEV)
    q2 = ops.rope_kv_write(qkv.to(DEV), freqs.to(DEV), table.to(DEV), pos, k2, v2, Hq, Hkv)
    assert not torch.equal(q2, q)


@pytest.mark.parametrize("B,Hq,Hkv,page,T,D", [(1, 1, 1, 4, 1, 128), (3, 4, 2, 8, 14, 128), (3, 8, 2, 16, 300, 64),
                                               (2, 16, 4, 64, 700, 128), (5, 8, 1, 16, 32, 64), (2, 6, 2, 16, 90, 128),
                                               (4, 12, 4, 32, 260, 64)])
def test_rope_paged_attn_decode_qknorm_equals_the_two_launches(oracle, B, Hq, Hkv, page, T, D):
    """The decode step with qk-norm in one launch against rope_kv_write with qk-norm followed by the plain
    attention kernel: same cache bits (hence the oracle's), same output bits; partial results likewise.
    Per-sequence lengths included."""
    _say("rope_paged_attn_decode_qknorm", B, Hq, Hkv, page, T, D)
    P = (T + page - 1) // page
    n_pages = B * P + 2
    g = torch.Generator().manual_seed(T + D)
    qkv = (torch.randn(B, (Hq + 2 * Hkv) * D, generator=g) * 1.5).to(torch.bfloat16).to(DEV)
    ang = torch.rand(B, D // 2, generator=g) * 6.28
    freqs = torch.polar(torch.ones_like(ang), ang).to(DEV)
    qg, kg = _gains(D, g)
    norm = ops.QkNorm(qg.to(DEV), kg.to(DEV), 1e-6)
    table = torch.randperm(n_pages, generator=g)[:B * P].view(B, P).to(DEV)
    kc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    vc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    k1, v1, k2, v2, k3, v3 = kc.clone(), vc.clone(), kc.clone(), vc.clone(), kc.clone(), vc.clone()
    q = ops.rope_kv_write(qkv, freqs, table, T - 1, k1, v1, Hq, Hkv, qk_norm=norm)
    want = ops.paged_attn_decode(q, k1, v1, table, T)
    out = ops.rope_paged_attn_decode(qkv, freqs, table, T, k2, v2, Hq, Hkv, qk_norm=norm)
    assert torch.equal(k1, k2) and torch.equal(v1, v2)
    assert torch.equal(out, want)
    # and the cache row is the oracle's
    kb, vb = _bits(kc), _bits(vc)
    oracle.c_rope_kv_write(_bits(qkv), torch.view_as_real(freqs).cpu().numpy(), table.cpu().numpy(), T - 1, kb, vb, Hq, Hkv,
                           qk_norm=(_bits(qg), _bits(kg), 1e-6))
    assert np.array_equal(_bits(k2), kb) and np.array_equal(_bits(v2), vb)
    parts = ops.rope_paged_attn_decode(qkv, freqs, table, T, k3, v3, Hq, Hkv, partials=True, qk_norm=norm)
    assert torch.equal(k3, k1)
    if T > 1:
        lens = torch.randint(1, T + 1, (B,), generator=g)
        lens[0] = T
        k4, v4, k5, v5 = kc.clone(), vc.clone(), kc.clone(), vc.clone()
        q = ops.rope_kv_write(qkv, freqs, table, T - 1, k4, v4, Hq, Hkv, qk_norm=norm)
        a = ops.paged_attn_decode(q, k4, v4, table, T, seq_lens=lens.to(DEV))
        b = ops.rope_paged_attn_decode(qkv, freqs, table, T, k5, v5, Hq, Hkv, seq_lens=lens.to(DEV), qk_norm=norm)
        assert torch.equal(a, b) and torch.equal(k4, k5)
    # the partial results, combined by the output projection, against the projection of the merged output
    K, N = Hq * D, 72
    if B <= ops.GEMV_ATTN_MAX_ROWS and K <= ops.GEMV_ATTN_MAX_K and parts.n_slices <= ops.GEMV_ATTN_MAX_SLICES:
        wq = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8).to(DEV)
        sw = (torch.rand(N, generator=g) * 0.01 + 1e-3).to(DEV)
        assert torch.equal(ops.gemv_w8a8_attn(parts, wq, sw), ops.gemv_w8a8_decode(want.view(B, K), wq, sw))


def test_qknorm_arguments_are_checked():
    D, Hq, Hkv = 64, 2, 1
    qkv = torch.zeros(1, (Hq + 2 * Hkv) * D, dtype=torch.bfloat16, device=DEV)
    freqs = torch.ones(1, D // 2, dtype=torch.complex64, device=DEV)
    table = torch.zeros(1, 1, dtype=torch.int64, device=DEV)
    kc = torch.zeros(1, 4, Hkv, D, dtype=torch.bfloat16, device=DEV)
    g = torch.ones(D, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError):
        ops.rope_kv_write(qkv, freqs, table, 0, kc, kc.clone(), Hq, Hkv, qk_norm=ops.QkNorm(g.float(), g, 1e-5))
    with pytest.raises(ValueError):
        ops.rope_kv_write(qkv, freqs, table, 0, kc, kc.clone(), Hq, Hkv, qk_norm=ops.QkNorm(g[:32], g, 1e-5))
    with pytest.raises(ValueError):
        ops.rope_paged_attn_decode(qkv, freqs, table, 1, kc, kc.clone(), Hq, Hkv, qk_norm=ops.QkNorm(g, g, -1.0))
