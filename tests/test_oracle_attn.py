"""Pins the oracle's decode attention over a paged KV cache (CPU) against torch: the complex
multiply of apply_rotary_emb (astrai/model/components/rope.py:26-33), index writes and gathers
through a page table (astrai/inference/core/cache.py:216-274) and scaled_dot_product_attention
with repeated KV heads (astrai/model/components/attention.py:15-23,93-103)."""
import numpy as np
import torch
import torch.nn.functional as F


def _bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def _bf16(a):
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def test_rope_and_page_write_match_torch(oracle):
    B, Hq, Hkv, D, page, n_pages, pos = 3, 4, 2, 128, 8, 12, 13
    g = torch.Generator().manual_seed(0)
    qkv = torch.randn(B, (Hq + 2 * Hkv) * D, generator=g).to(torch.bfloat16)
    ang = torch.rand(B, D // 2, generator=g) * 6.28
    freqs = torch.polar(torch.ones_like(ang), ang)                       # complex64 [B, D/2]
    table = torch.tensor([[5, 2, 9], [0, -1, 11], [3, 7, 1]])            # sequence 1: page of pos 13 unmapped
    kc = torch.zeros(n_pages, page, Hkv, D, dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    kb, vb = _bits(kc), _bits(vc)
    q = oracle.c_rope_kv_write(_bits(qkv), torch.view_as_real(freqs).numpy(), table.numpy(), pos, kb, vb, Hq, Hkv)
    # torch: the reference's expression
    x = qkv.view(B, 1, Hq + 2 * Hkv, D)
    xr = torch.view_as_real(torch.view_as_complex(x.float().reshape(B, 1, -1, D // 2, 2)) *
                            freqs.view(B, 1, 1, D // 2)).flatten(-2).to(torch.bfloat16)
    assert torch.equal(_bf16(q), xr[:, 0, :Hq])
    for b in range(B):
        phys = table[b, pos // page].item()
        if phys < 0:
            continue
        assert torch.equal(_bf16(kb)[phys, pos % page], xr[b, 0, Hq:Hq + Hkv])
        assert torch.equal(_bf16(vb)[phys, pos % page], x[b, 0, Hq + Hkv:])
    untouched = torch.ones(n_pages, page, dtype=torch.bool)
    untouched[5 // 1 * 0 + table[0, 1], pos % page] = False
    untouched[table[2, 1], pos % page] = False
    assert not _bf16(kb)[untouched].any() and not _bf16(vb)[untouched].any()


def test_paged_attention_matches_torch_sdpa(oracle):
    B, Hq, Hkv, D, page, n_pages, T = 2, 8, 2, 128, 16, 10, 70
    g = torch.Generator().manual_seed(1)
    q = torch.randn(B, Hq, D, generator=g).to(torch.bfloat16)
    kc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16)
    vc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16)
    table = torch.tensor([[4, 0, 7, 2, 9], [1, 8, -1, 3, 5]])           # an unmapped page inside sequence 1
    out = _bf16(oracle.c_paged_attn_decode(_bits(q), _bits(kc), _bits(vc), table.numpy(), T, D ** -0.5)).float()
    # torch: gather with zero fill, repeat heads, attention in fp32
    safe = table.clamp(min=0)
    k = kc[safe].flatten(1, 2).float()
    v = vc[safe].flatten(1, 2).float()
    hole = (table < 0).unsqueeze(-1).expand(-1, -1, page).flatten(1, 2)[:, :, None, None]
    k, v = k.masked_fill(hole, 0.0)[:, :T], v.masked_fill(hole, 0.0)[:, :T]
    k, v = k.repeat_interleave(Hq // Hkv, dim=2), v.repeat_interleave(Hq // Hkv, dim=2)
    ref = F.scaled_dot_product_attention(q.float().unsqueeze(2), k.transpose(1, 2), v.transpose(1, 2))[:, :, 0]
    assert torch.allclose(out, ref, rtol=1e-2, atol=1e-2)
    assert (out - ref).norm() / ref.norm() < 3e-3


def test_paged_attention_with_sequence_lengths_matches_torch_under_the_position_mask(oracle):
    """A decode batch whose sequences sit at different positions: the oracle's seq_lens against torch's attention
    under the additive mask the reference builds from position_ids (transformer.py:40-46: 0 where
    t <= position, -finfo.max / 2 elsewhere), and against the closed form for a sequence of length 1 (its
    output is the first value row)."""
    B, Hq, Hkv, D, page, n_pages, T = 3, 4, 2, 64, 16, 12, 61
    g = torch.Generator().manual_seed(2)
    q = torch.randn(B, Hq, D, generator=g).to(torch.bfloat16)
    kc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16)
    vc = torch.randn(n_pages, page, Hkv, D, generator=g).to(torch.bfloat16)
    table = torch.tensor([[4, 0, 7, 2], [1, 8, 11, 3], [5, 9, 10, 6]])
    lens = torch.tensor([61, 1, 33])
    out = _bf16(oracle.c_paged_attn_decode(_bits(q), _bits(kc), _bits(vc), table.numpy(), T, D ** -0.5,
                                           seq_lens=lens.numpy())).float()
    k = kc[table].flatten(1, 2).float()[:, :T].repeat_interleave(Hq // Hkv, dim=2)
    v = vc[table].flatten(1, 2).float()[:, :T].repeat_interleave(Hq // Hkv, dim=2)
    pos = (lens - 1).view(B, 1)
    attend = pos >= torch.arange(T)                                       # [B, T]
    mask = torch.full((B, 1, 1, T), -torch.finfo(torch.bfloat16).max / 2).masked_fill_(attend.view(B, 1, 1, T), 0.0)
    ref = F.scaled_dot_product_attention(q.float().unsqueeze(2), k.transpose(1, 2), v.transpose(1, 2), mask)[:, :, 0]
    assert torch.allclose(out, ref, rtol=1e-2, atol=1e-2)
    assert (out - ref).norm() / ref.norm() < 3e-3
    first_v = vc[table[1, 0], 0].float().repeat_interleave(Hq // Hkv, dim=0)  # sequence 1 sees position 0 only
    assert torch.equal(out[1], first_v)
    # lengths equal to T change nothing
    full = _bf16(oracle.c_paged_attn_decode(_bits(q), _bits(kc), _bits(vc), table.numpy(), T, D ** -0.5)).float()
    same = _bf16(oracle.c_paged_attn_decode(_bits(q), _bits(kc), _bits(vc), table.numpy(), T, D ** -0.5,
                                            seq_lens=np.full(B, T))).float()
    assert torch.equal(full, same) and torch.equal(full[0], out[0])


def test_prefill_attention_matches_torch_sdpa_and_closed_forms(oracle):
    """Causal attention over a prompt: against torch's scaled_dot_product_attention in fp32, with
    enable_gqa and with explicitly repeated KV heads (the reference's repeat_kv), and on inputs
    whose answer is known in closed form."""
    for (B, S, Hq, Hkv, D) in [(2, 37, 6, 2, 64), (1, 70, 4, 4, 128), (2, 5, 3, 1, 64)]:
        g = torch.Generator().manual_seed(S)
        q = torch.randn(B, S, Hq, D, generator=g).to(torch.bfloat16)
        k = torch.randn(B, S, Hkv, D, generator=g).to(torch.bfloat16)
        v = torch.randn(B, S, Hkv, D, generator=g).to(torch.bfloat16)
        out = _bf16(oracle.c_prefill_attn_causal(_bits(q), _bits(k), _bits(v), D ** -0.5)).float()
        qt, kt, vt = (t.float().transpose(1, 2) for t in (q, k, v))
        rep = Hq // Hkv
        want = F.scaled_dot_product_attention(qt, kt.repeat_interleave(rep, dim=1), vt.repeat_interleave(rep, dim=1),
                                              is_causal=True).transpose(1, 2)
        assert torch.allclose(out, want, rtol=1e-2, atol=1e-2)
        assert ((out - want).norm() / want.norm()).item() < 4e-3
        want2 = F.scaled_dot_product_attention(qt, kt, vt, is_causal=True, enable_gqa=True).transpose(1, 2)
        assert torch.allclose(want, want2, rtol=1e-5, atol=1e-5)
        # the first position attends to itself only: its output is its own value row, bit for bit
        assert torch.equal(_bf16(oracle.c_prefill_attn_causal(_bits(q), _bits(k), _bits(v), D ** -0.5))[:, 0],
                           v[:, 0].repeat_interleave(rep, dim=1))
    # equal keys: uniform weights, so position s returns the mean of the first s + 1 value rows
    B, S, Hq, Hkv, D = 1, 9, 2, 1, 64
    q = torch.randn(B, S, Hq, D).to(torch.bfloat16)
    k = torch.ones(B, S, Hkv, D).to(torch.bfloat16)
    v = torch.randn(B, S, Hkv, D).to(torch.bfloat16)
    out = _bf16(oracle.c_prefill_attn_causal(_bits(q), _bits(k), _bits(v), 0.125)).float()
    mean = v.float().cumsum(1) / torch.arange(1, S + 1).view(1, S, 1, 1)
    assert torch.allclose(out, mean.expand(B, S, Hq, D), rtol=1e-2, atol=1e-2)


def test_prefill_attention_with_a_position_offset_matches_the_masked_torch_attention(oracle):
    """A chunk of new tokens on top of cached ones: start = 0 is the causal oracle bit for bit; a
    later chunk is the tail of the full causal result, and agrees with torch's attention under the
    explicit position mask the reference builds (transformer.py:17-46)."""
    for (B, S, start, Hq, Hkv, D) in [(2, 11, 0, 4, 2, 64), (2, 9, 30, 6, 2, 64), (1, 33, 70, 4, 4, 128), (2, 1, 17, 3, 1, 64)]:
        g = torch.Generator().manual_seed(S + start)
        T = start + S
        qf = torch.randn(B, T, Hq, D, generator=g).to(torch.bfloat16)     # queries of every position
        k = torch.randn(B, T, Hkv, D, generator=g).to(torch.bfloat16)
        v = torch.randn(B, T, Hkv, D, generator=g).to(torch.bfloat16)
        q = qf[:, start:].contiguous()
        out = oracle.c_prefill_attn_offset(_bits(q), _bits(k), _bits(v), start, D ** -0.5)
        full = oracle.c_prefill_attn_causal(_bits(qf), _bits(k), _bits(v), D ** -0.5)
        assert np.array_equal(out, full[:, start:])                      # same arithmetic, same bits
        rep = Hq // Hkv
        pos = torch.arange(start, T)
        mask = torch.zeros(S, T).masked_fill_(pos.view(S, 1) < torch.arange(T).view(1, T), float("-inf"))
        want = F.scaled_dot_product_attention(q.float().transpose(1, 2), k.float().transpose(1, 2).repeat_interleave(rep, 1),
                                              v.float().transpose(1, 2).repeat_interleave(rep, 1), mask).transpose(1, 2)
        got = _bf16(out).float()
        assert torch.allclose(got, want, rtol=1e-2, atol=1e-2)
        assert ((got - want).norm() / want.norm()).item() < 4e-3


def _qknorm_case(D, seed, gains="random"):
    B, Hq, Hkv, page, n_pages, pos = 3, 4, 2, 8, 12, 13
    g = torch.Generator().manual_seed(seed)
    qkv = (torch.randn(B, (Hq + 2 * Hkv) * D, generator=g) * 1.7).to(torch.bfloat16)
    ang = torch.rand(B, D // 2, generator=g) * 6.28
    freqs = torch.view_as_real(torch.polar(torch.ones_like(ang), ang)).numpy()
    table = torch.tensor([[5, 2, 9], [0, -1, 11], [3, 7, 1]])
    if gains == "random":
        qg = (1.0 + 0.3 * torch.randn(D, generator=g)).to(torch.bfloat16)
        kg = (1.0 + 0.3 * torch.randn(D, generator=g)).to(torch.bfloat16)
    else:
        qg = kg = torch.ones(D, dtype=torch.bfloat16)
    return B, Hq, Hkv, page, n_pages, pos, qkv, freqs, table, qg, kg


def test_qknorm_of_the_rotated_heads_matches_rms_norm_and_numpy(oracle):
    """oq_rope_kv_write_qknorm against (a) F.rms_norm applied to the heads that oq_rope_kv_write stores -- the
    reference's order, rotation then q_norm / k_norm (attention.py:86-89) -- within one bf16 step; (b) the
    numpy restatement of the fixed summation order bit for bit; (c) v and the pages of unmapped sequences
    untouched."""
    eps = 1e-5
    for D, seed in ((128, 3), (64, 4)):
        B, Hq, Hkv, page, n_pages, pos, qkv, freqs, table, qg, kg = _qknorm_case(D, seed)
        k0, v0 = np.zeros((n_pages, page, Hkv, D), np.uint16), np.zeros((n_pages, page, Hkv, D), np.uint16)
        k1, v1 = k0.copy(), v0.copy()
        q_plain = oracle.c_rope_kv_write(_bits(qkv), freqs, table.numpy(), pos, k0, v0, Hq, Hkv)
        q_norm = oracle.c_rope_kv_write(_bits(qkv), freqs, table.numpy(), pos, k1, v1, Hq, Hkv,
                                        qk_norm=(_bits(qg), _bits(kg), eps))
        assert np.array_equal(v0, v1)
        # (b) bit for bit against numpy on the un-normalised heads
        assert np.array_equal(q_norm, oracle.np_head_rmsnorm_bits(q_plain, _bits(qg), eps))
        assert np.array_equal(k1, np.where((k0 != 0).any(-1, keepdims=True),
                                           oracle.np_head_rmsnorm_bits(k0, _bits(kg), eps), 0))
        # (a) torch's rms_norm on the same heads, fp32 arithmetic, then rounded once
        want_q = F.rms_norm(_bf16(q_plain).float(), (D,), qg.float(), eps)
        got_q = _bf16(q_norm).float()
        step = torch.maximum(want_q.abs(), torch.tensor(1e-30)) * 2.0 ** -7     # one bf16 step, generously
        assert ((got_q - want_q).abs() <= step).all()
        assert (got_q == want_q.to(torch.bfloat16).float()).float().mean() > 0.97
        want_k = F.rms_norm(_bf16(k0).float(), (D,), kg.float(), eps)
        assert ((_bf16(k1).float() - want_k).abs() <= want_k.abs() * 2.0 ** -7 + 1e-30).all()
        # a plausible mistake -- the norm before the rotation, or the other head's gain -- does not pass (a)
        swapped = oracle.np_head_rmsnorm_bits(q_plain, _bits(kg), eps)
        assert not np.array_equal(swapped, q_norm)


def test_qknorm_closed_forms(oracle):
    """Unit gains and a head of equal magnitudes +-a: the mean square is a^2 exactly, so every element becomes
    +-a / sqrt(a^2 + eps); with eps = 0 exactly +-1.  A rotation by angle 0 keeps the head."""
    D, Hq, Hkv, page = 64, 2, 1, 4
    a = 0.75
    sign = np.where(np.arange((Hq + 2 * Hkv) * D) % 3 == 0, -1.0, 1.0).astype(np.float32)
    qkv = torch.from_numpy(sign * a).to(torch.bfloat16).view(1, -1)
    freqs = np.zeros((1, D // 2, 2), np.float32)
    freqs[..., 0] = 1.0
    table = np.array([[0]], np.int64)
    ones = _bits(torch.ones(D, dtype=torch.bfloat16))
    for eps, want in ((0.0, 1.0), (0.4375, a / np.sqrt(np.float32(a * a + 0.4375)))):
        kc, vc = np.zeros((1, page, Hkv, D), np.uint16), np.zeros((1, page, Hkv, D), np.uint16)
        q = oracle.c_rope_kv_write(_bits(qkv), freqs, table, 2, kc, vc, Hq, Hkv, qk_norm=(ones, ones, eps))
        got = _bf16(q).float().view(-1)
        want_t = torch.tensor(float(want)).to(torch.bfloat16).float()
        assert torch.equal(got, torch.from_numpy(sign[:Hq * D]) * want_t)
        assert torch.equal(_bf16(kc)[0, 2].float().view(-1), torch.from_numpy(sign[Hq * D:(Hq + Hkv) * D]) * want_t)
        assert torch.equal(_bf16(vc)[0, 2].view(-1), qkv[0, (Hq + Hkv) * D:])


def test_qknorm_then_attention_matches_the_reference_sequence_in_torch(oracle):
    """Decode steps of an attention with use_qk_norm written as the reference does (rotate, norm, cache the
    normed key, attend: attention.py:83-103) in torch fp32 against the oracle's qk-norm write + paged attention."""
    D, Hq, Hkv, page, n_pages, B = 64, 4, 2, 4, 8, 2
    g = torch.Generator().manual_seed(9)
    qg = (1.0 + 0.3 * torch.randn(D, generator=g)).to(torch.bfloat16)
    kg = (1.0 + 0.3 * torch.randn(D, generator=g)).to(torch.bfloat16)
    table = torch.tensor([[3, 0, 6], [5, 1, 2]])
    kc, vc = np.zeros((n_pages, page, Hkv, D), np.uint16), np.zeros((n_pages, page, Hkv, D), np.uint16)
    ks, vs = [], []
    for pos in range(9):
        qkv = torch.randn(B, (Hq + 2 * Hkv) * D, generator=g).to(torch.bfloat16)
        ang = torch.rand(B, D // 2, generator=g) * 6.28
        fr = torch.polar(torch.ones_like(ang), ang)
        q = oracle.c_rope_kv_write(_bits(qkv), torch.view_as_real(fr).numpy(), table.numpy(), pos, kc, vc, Hq, Hkv,
                                   qk_norm=(_bits(qg), _bits(kg), 1e-6))
        out = _bf16(oracle.c_paged_attn_decode(q, kc, vc, table.numpy(), pos + 1, D ** -0.5)).float()
        x = qkv.view(B, 1, Hq + 2 * Hkv, D)
        rot = torch.view_as_real(torch.view_as_complex(x[:, :, :Hq + Hkv].float().reshape(B, 1, -1, D // 2, 2)) *
                                 fr.view(B, 1, 1, D // 2)).flatten(-2).to(torch.bfloat16)
        qn = F.rms_norm(rot[:, :, :Hq], (D,), qg, 1e-6)
        kn = F.rms_norm(rot[:, :, Hq:], (D,), kg, 1e-6)
        ks.append(kn)
        vs.append(x[:, :, Hq + Hkv:])
        k_all = torch.cat(ks, 1).float().repeat_interleave(Hq // Hkv, dim=2)
        v_all = torch.cat(vs, 1).float().repeat_interleave(Hq // Hkv, dim=2)
        ref = F.scaled_dot_product_attention(qn.float().transpose(1, 2), k_all.transpose(1, 2), v_all.transpose(1, 2))
        assert torch.allclose(out, ref[:, :, 0], rtol=2e-2, atol=2e-2)
        assert (out - ref[:, :, 0]).norm() / ref.norm() < 8e-3
