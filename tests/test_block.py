"""The decoder block that hosts the quantized Linears (benchmark configuration 5).
CPU tests pin the float restatement against closed forms and a hand-written
attention; GPU tests put QuantLinear into it through quantize_model."""
import math

import pytest
import torch
import torch.nn.functional as F

from khaosz_amd.block import (ContiguousKV, DecoderBlock, GQA, PagedKV, RMSNorm, apply_rotary, decode_mask,
                              rotary_table)
from khaosz_amd.linear import QuantLinear, quantize_model


def _freqs(table, B, start, S):
    return table[start:start + S].unsqueeze(0).expand(B, -1, -1)


def test_rotary_is_a_position_dependent_rotation():
    tab = rotary_table(16, 32)
    assert tab.shape == (32, 8) and tab.dtype == torch.complex64
    assert torch.allclose(tab[0], torch.ones(8, dtype=torch.complex64))
    theta = 10000.0 ** (-torch.arange(0, 16, 2, dtype=torch.float64) / 16)
    assert torch.allclose(torch.angle(tab[5]).double(), (5 * theta + math.pi) % (2 * math.pi) - math.pi, atol=1e-6)
    x = torch.randn(2, 4, 3, 16)
    y = apply_rotary(x, _freqs(tab, 2, 7, 4))
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-5)           # rotations keep the norm
    assert torch.allclose(apply_rotary(x, _freqs(tab, 2, 0, 1).expand(2, 4, 8)), x)  # position 0 is the identity
    # pair (2i, 2i+1) is rotated by angle p * theta_i
    p, i = 9, 3
    a = torch.zeros(1, 1, 1, 16)
    a[..., 2 * i] = 1.0
    r = apply_rotary(a, _freqs(tab, 1, p, 1))[0, 0, 0]
    assert abs(r[2 * i].item() - math.cos(p * theta[i])) < 1e-6 and abs(r[2 * i + 1].item() - math.sin(p * theta[i])) < 1e-6
    # scores depend on the position difference only
    q, k = torch.randn(1, 1, 1, 16), torch.randn(1, 1, 1, 16)
    s1 = (apply_rotary(q, _freqs(tab, 1, 12, 1)) * apply_rotary(k, _freqs(tab, 1, 5, 1))).sum()
    s2 = (apply_rotary(q, _freqs(tab, 1, 20, 1)) * apply_rotary(k, _freqs(tab, 1, 13, 1))).sum()
    assert abs(s1 - s2) < 1e-4


def test_rmsnorm_closed_form():
    n = RMSNorm(24, 1e-5)
    with torch.no_grad():
        n.weight.copy_(torch.randn(24))
    x = torch.randn(3, 5, 24)
    want = x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5) * n.weight
    assert torch.allclose(n(x), want, atol=1e-5)


def test_gqa_matches_a_hand_written_causal_attention():
    torch.manual_seed(0)
    dim, H, Hkv, B, S = 32, 4, 2, 2, 6
    att = GQA(dim, H, Hkv)
    for l in (att.q_proj, att.k_proj, att.v_proj, att.o_proj):
        l.reset_parameters()
    x = torch.randn(B, S, dim)
    tab = rotary_table(dim // H, 16)
    fr = _freqs(tab, B, 0, S)
    y = att(x, fr)
    D = dim // H
    q = apply_rotary((x @ att.q_proj.weight.T).view(B, S, H, D), fr)
    k = apply_rotary((x @ att.k_proj.weight.T).view(B, S, Hkv, D), fr)
    v = (x @ att.v_proj.weight.T).view(B, S, Hkv, D)
    out = torch.zeros(B, S, H, D)
    for b in range(B):
        for h in range(H):
            g = h // (H // Hkv)
            for i in range(S):
                sc = torch.stack([(q[b, i, h] * k[b, j, g]).sum() / math.sqrt(D) for j in range(i + 1)])
                w = torch.softmax(sc, 0)
                out[b, i, h] = sum(w[j] * v[b, j, g] for j in range(i + 1))
    want = out.reshape(B, S, dim) @ att.o_proj.weight.T
    assert torch.allclose(y, want, atol=1e-4)


def test_gqa_options_qk_norm_and_output_gate_by_hand():
    """use_qk_norm: RMSNorm over the head dimension of q and k after the rotation
    (attention.py:86-89); use_gated_attention: the attention output times sigmoid(gate(x)) before
    o_proj (attention.py:105-108).  Parameter names as in the reference."""
    torch.manual_seed(1)
    dim, H, Hkv, B, S = 32, 4, 2, 2, 5
    att = GQA(dim, H, Hkv, use_qk_norm=True, norm_eps=1e-5, use_gated_attention=True)
    for l in (att.q_proj, att.k_proj, att.v_proj, att.o_proj, att.gate):
        l.reset_parameters()
    with torch.no_grad():
        att.q_norm.weight.copy_(torch.rand(dim // H) + 0.5)
        att.k_norm.weight.copy_(torch.rand(dim // H) + 0.5)
    assert {"q_norm.weight", "k_norm.weight", "gate.weight"} <= set(att.state_dict())
    x = torch.randn(B, S, dim)
    tab = rotary_table(dim // H, 16)
    fr = _freqs(tab, B, 0, S)
    y = att(x, fr)
    D = dim // H
    rms = lambda t, w: t / torch.sqrt((t * t).mean(-1, keepdim=True) + 1e-5) * w
    q = rms(apply_rotary((x @ att.q_proj.weight.T).view(B, S, H, D), fr), att.q_norm.weight)
    k = rms(apply_rotary((x @ att.k_proj.weight.T).view(B, S, Hkv, D), fr), att.k_norm.weight)
    v = (x @ att.v_proj.weight.T).view(B, S, Hkv, D)
    out = torch.zeros(B, S, H, D)
    for b in range(B):
        for h in range(H):
            g = h // (H // Hkv)
            for i in range(S):
                sc = torch.stack([(q[b, i, h] * k[b, j, g]).sum() / math.sqrt(D) for j in range(i + 1)])
                w = torch.softmax(sc, 0)
                out[b, i, h] = sum(w[j] * v[b, j, g] for j in range(i + 1))
    gated = out.reshape(B, S, dim) * torch.sigmoid(x @ att.gate.weight.T)
    assert torch.allclose(y, gated @ att.o_proj.weight.T, atol=1e-4)
    # the cached key is the normalised one: a decode step on a cache equals the full pass
    blk = DecoderBlock(dim, H, 88, Hkv, use_qk_norm=True, use_gated_attention=True)
    blk.reset_parameters()
    xs = torch.randn(B, S + 1, dim)
    full = blk(xs, _freqs(tab, B, 0, S + 1))
    cache = ContiguousKV(B, 16, Hkv, D, "cpu", torch.float32)
    blk(xs[:, :S], _freqs(tab, B, 0, S), None, cache.bind(S))
    step = blk(xs[:, S:], _freqs(tab, B, S, 1), decode_mask(B, S + 1, "cpu", torch.float32), cache.bind(S + 1))
    assert torch.allclose(step[:, 0], full[:, S], atol=1e-5)
    assert not blk.attention.fuse_decode_attention()           # needs the fused, quantized q/k/v projection


def _block(dim=64, heads=4, kv=2, ffn=176, seed=0):
    torch.manual_seed(seed)
    b = DecoderBlock(dim, heads, ffn, kv)
    b.reset_parameters()
    return b


def test_block_residual_structure_and_decode_equals_prefill_on_cpu():
    blk = _block()
    B, S, dim = 2, 9, 64
    tab = rotary_table(16, 32)
    x = torch.randn(B, S + 1, dim)
    full = blk(x, _freqs(tab, B, 0, S + 1))
    # by hand: x1 = x + attn(norm(x)); y = x1 + mlp(norm(x1))
    x1 = x + blk.attention(blk.input_norm(x), _freqs(tab, B, 0, S + 1))
    assert torch.allclose(full, x1 + blk.mlp(blk.post_attention_norm(x1)), atol=1e-6)
    cache = ContiguousKV(B, 32, 2, 16, "cpu", torch.float32)
    pre = blk(x[:, :S], _freqs(tab, B, 0, S), None, cache.bind(S))
    assert torch.allclose(pre, full[:, :S], atol=1e-5)
    step = blk(x[:, S:], _freqs(tab, B, S, 1), decode_mask(B, S + 1, "cpu", torch.float32), cache.bind(S + 1))
    assert torch.allclose(step[:, 0], full[:, S], atol=1e-5)


def test_paged_kv_write_gather_round_trip_and_unmapped_pages():
    """What the reference's cache tests check for Storage (tests/inference/test_cache.py:210-279):
    tokens written through a page table come back in order through gather, across page borders,
    in scattered physical pages, chunk by chunk; unmapped logical pages are skipped on write
    and read back as zeros."""
    B, H, D, ps = 3, 2, 4, 8
    cache = PagedKV(n_pages=16, page_size=ps, n_kv_heads=H, head_dim=D, device="cpu", dtype=torch.float32)
    table = torch.tensor([[5, 2, 9], [0, 7, 11], [3, 14, 1]])
    g = torch.Generator().manual_seed(0)
    k = torch.randn(B, 21, H, D, generator=g)
    v = torch.randn(B, 21, H, D, generator=g)
    cache.bind(table, 13).write(0, k[:, :13], v[:, :13])           # spans pages 0 and 1
    cache.bind(table, 14).write(0, k[:, 13:14], v[:, 13:14])       # one decode token
    cache.bind(table, 21).write(0, k[:, 14:], v[:, 14:])           # crosses into page 2
    kk, vv = cache.bind(table, 21).gather(0)
    assert torch.equal(kk, k) and torch.equal(vv, v)
    kk, _ = cache.bind(table, 10).gather(0)
    assert torch.equal(kk, k[:, :10])
    assert torch.equal(cache.k[9, :5], k[0, 16:21])                 # sequence 0, logical page 2 -> physical 9
    # sequence 1 has no third page: its tokens there are dropped, the others are kept
    cache2 = PagedKV(16, ps, H, D, "cpu", torch.float32)
    holes = torch.tensor([[5, 2, 9], [0, 7, -1], [3, 14, 1]])
    cache2.bind(holes, 21).write(0, k, v)
    kk, vv = cache2.gather(0)
    assert torch.equal(kk[0], k[0]) and torch.equal(kk[2], k[2])
    assert torch.equal(kk[1, :16], k[1, :16]) and not kk[1, 16:].any() and not vv[1, 16:].any()
    with pytest.raises(ValueError):
        cache.bind(table, 25).write(0, k[:, :1], v[:, :1])          # beyond the table


def test_paged_cache_gives_the_block_the_same_outputs_as_the_contiguous_one():
    blk = _block()
    B, S, dim = 2, 9, 64
    tab = rotary_table(16, 32)
    x = torch.randn(B, S + 2, dim)
    outs = []
    for cache, bind in ((ContiguousKV(B, 32, 2, 16, "cpu", torch.float32), lambda c, n: c.bind(n)),
                        (PagedKV(8, 4, 2, 16, "cpu", torch.float32),
                         lambda c, n, t=torch.tensor([[6, 1, 3], [0, 5, 2]]): c.bind(t, n))):
        o = [blk(x[:, :S], _freqs(tab, B, 0, S), None, bind(cache, S))]
        for t in range(2):
            o.append(blk(x[:, S + t:S + t + 1], _freqs(tab, B, S + t, 1),
                         decode_mask(B, S + t + 1, "cpu", torch.float32), bind(cache, S + t + 1)))
        outs.append(torch.cat(o, dim=1))
    assert torch.equal(outs[0], outs[1])


@pytest.mark.gpu
def test_quantized_block_tracks_the_float_block():
    dev = "cuda:0"
    blk = _block(dim=256, heads=4, kv=2, ffn=704).to(dev)
    B, S = 2, 40
    tab = rotary_table(64, 128, device=dev)
    x = torch.randn(B, S, 256, device=dev)
    with torch.inference_mode():
        ref = blk(x, _freqs(tab, B, 0, S))
        assert quantize_model(blk) == 7
        assert all(isinstance(m, QuantLinear) for m in (blk.attention.q_proj, blk.attention.o_proj, blk.mlp.down))
        y = blk(x, _freqs(tab, B, 0, S))
    rel = ((y - ref).norm() / ref.norm()).item()
    assert rel < 3e-2, rel


@pytest.mark.gpu
def test_config5_block_prefill_then_decode_bf16():
    """hidden 2048, 16 query / 4 KV heads of 128, FFN 5632, all 7 Linears W8A8, bf16 activations;
    a shortened run of the config (2 x 96 prefill, 3 decode steps) checked against the float block, and
    each decode step against the same token's row of a longer prefill."""
    dev, dt = "cuda:0", torch.bfloat16
    torch.manual_seed(5)
    blk = DecoderBlock(2048, 16, 5632, 4)
    blk.reset_parameters()
    blk = blk.to(dev)
    B, S, steps = 2, 96, 3
    tab = rotary_table(128, 256, device=dev)
    x = torch.randn(B, S + steps, 2048, device=dev)
    with torch.inference_mode():
        ref = blk(x, _freqs(tab, B, 0, S + steps))                  # float32 block, whole sequence
        fblk = blk.to(dt)
        assert quantize_model(fblk) == 7
        xb = x.to(dt)
        full = fblk(xb, _freqs(tab, B, 0, S + steps))               # quantized, whole sequence (MFMA path)
        cache = PagedKV(8, 64, 4, 128, dev, dt)                     # paged, 64-token pages, scattered
        table = torch.tensor([[5, 0], [2, 7]], device=dev)
        pre = fblk(xb[:, :S], _freqs(tab, B, 0, S), None, cache.bind(table, S))
        outs = [pre]
        for t in range(steps):                                      # decode path (M = B = 2)
            pos = S + t
            outs.append(fblk(xb[:, pos:pos + 1], _freqs(tab, B, pos, 1), decode_mask(B, pos + 1, dev, dt),
                             cache.bind(table, pos + 1)))
        seq = torch.cat(outs, dim=1)
    assert seq.shape == (B, S + steps, 2048) and seq.dtype == dt
    rel = ((full.float() - ref).norm() / ref.norm()).item()
    assert rel < 3e-2, rel
    # decode rows equal the prefill rows of the same tokens up to bf16 attention numerics
    rel_d = ((seq.float() - full.float()).norm() / full.float().norm()).item()
    assert rel_d < 1e-2, rel_d


@pytest.mark.gpu
def test_quantized_block_checkpoint_round_trip_through_safetensors(tmp_path):
    """The reference saves and loads weights as safetensors state dicts (astrai/serialization.py:19-25,
    astrai/model/automodel.py:54-91).  A quantized block's state dict (qweight / w_scale per
    projection) survives that path bit for bit, and a float checkpoint with the reference's
    ``*.weight`` keys loads into an already quantized block (quantised on load)."""
    from safetensors.torch import load_file, save_file

    dev = "cuda:0"
    flt = _block(dim=256, heads=4, kv=2, ffn=704).to(dev)
    save_file({k: v.contiguous() for k, v in flt.state_dict().items()}, str(tmp_path / "float.safetensors"))
    qblk = _block(dim=256, heads=4, kv=2, ffn=704).to(dev)
    qblk.load_state_dict(flt.state_dict())
    assert quantize_model(qblk) == 7
    sd = qblk.state_dict()
    assert "attention.q_proj.qweight" in sd and "attention.q_proj.w_scale" in sd and "mlp.down.qweight" in sd
    assert not any(k.endswith("_proj.weight") for k in sd)
    save_file({k: v.contiguous() for k, v in sd.items()}, str(tmp_path / "quant.safetensors"))

    x = torch.randn(2, 24, 256, device=dev)
    tab = rotary_table(64, 64, device=dev)
    with torch.inference_mode():
        want = qblk(x, _freqs(tab, 2, 0, 24))
        # quantized checkpoint -> fresh quantized block
        a = _block(dim=256, heads=4, kv=2, ffn=704).to(dev)
        quantize_model(a)
        a.load_state_dict(load_file(str(tmp_path / "quant.safetensors"), device=dev))
        assert torch.equal(a(x, _freqs(tab, 2, 0, 24)), want)
        # float checkpoint with the reference's key names -> fresh quantized block
        b = _block(dim=256, heads=4, kv=2, ffn=704).to(dev)
        quantize_model(b)
        b.load_state_dict(load_file(str(tmp_path / "float.safetensors"), device=dev))
        assert torch.equal(b.attention.q_proj.qweight, qblk.attention.q_proj.qweight)
        assert torch.equal(b(x, _freqs(tab, 2, 0, 24)), want)


@pytest.mark.gpu
def test_fused_shared_input_projections_are_bit_identical():
    """q/k/v and up/gate run as one concatenated projection each: same bits as the seven separate
    modules on both the prefill (MFMA GEMM) and the decode (GEMV) path, same state-dict keys, and a
    later load_state_dict reaches the fused storage because the parts are views of it."""
    from khaosz_amd import fuse_shared_inputs

    dev, dt = "cuda:0", torch.bfloat16
    a = _block(dim=256, heads=4, kv=2, ffn=704).to(dev).to(dt)
    b = _block(dim=256, heads=4, kv=2, ffn=704).to(dev).to(dt)
    b.load_state_dict(a.state_dict())
    assert quantize_model(a) == 7 and quantize_model(b) == 7
    keys = set(b.state_dict().keys())
    assert fuse_shared_inputs(b) == 2 and fuse_shared_inputs(b) == 0
    assert set(b.state_dict().keys()) == keys
    assert b.attention._qkv.out_dim == 256 + 2 * 128 and b.mlp._upgate.out_dim == 2 * 704
    assert b.attention.k_proj.qweight.data_ptr() == b.attention._qkv.qweight[256:].data_ptr()
    tab = rotary_table(64, 64, device=dev)
    x = torch.randn(2, 40, 256, device=dev).to(dt)
    with torch.inference_mode():
        assert torch.equal(b(x, _freqs(tab, 2, 0, 40)), a(x, _freqs(tab, 2, 0, 40)))          # M = 80
        xd = x[:, :3].contiguous()
        assert torch.equal(b(xd, _freqs(tab, 2, 0, 3)), a(xd, _freqs(tab, 2, 0, 3)))          # M = 6
        # new weights loaded after fusing land in the fused buffers
        c = _block(dim=256, heads=4, kv=2, ffn=704).to(dev).to(dt)
        quantize_model(c)
        b.load_state_dict(c.state_dict())
        assert torch.equal(b(x, _freqs(tab, 2, 0, 40)), c(x, _freqs(tab, 2, 0, 40)))


@pytest.mark.gpu
def test_residual_adds_in_the_projection_epilogue_are_bit_identical():
    """o_proj and down add the residual stream in their epilogue (GEMM for prefill, GEMV for
    decode rows, with and without the fused norms): the same bits as the separate adds."""
    from khaosz_amd import fuse_shared_inputs

    dev, dt = "cuda:0", torch.bfloat16
    for norms in (False, True):
        a = _block(dim=256, heads=4, kv=2, ffn=704).to(dev).to(dt)
        b = _block(dim=256, heads=4, kv=2, ffn=704).to(dev).to(dt)
        b.load_state_dict(a.state_dict())
        quantize_model(a), quantize_model(b)
        fuse_shared_inputs(a, norms=norms)
        fuse_shared_inputs(b, norms=norms, residuals=True)
        tab = rotary_table(64, 64, device=dev)
        x = (torch.randn(2, 40, 256, device=dev) * 3).to(dt)
        with torch.inference_mode():
            assert torch.equal(b(x, _freqs(tab, 2, 0, 40)), a(x, _freqs(tab, 2, 0, 40)))      # M = 80
            for rows in (1, 3, 6):                                                            # M = 2, 6, 12
                xd = x[:, :rows].contiguous()
                assert torch.equal(b(xd, _freqs(tab, 2, 0, rows)), a(xd, _freqs(tab, 2, 0, rows)))
    # a float block takes the same flag and simply adds
    f = _block(dim=256, heads=4, kv=2, ffn=704).to(dev).to(dt)
    want = f(x, _freqs(tab, 2, 0, 40))
    fuse_shared_inputs(f, residuals=True)
    assert torch.equal(f(x, _freqs(tab, 2, 0, 40)), want)


@pytest.mark.gpu
def test_fused_norm_quantise_stays_inside_the_quantisation_noise():
    """RMSNorm + per-token quantisation in one launch for both norms of the block: outputs move by
    far less than the quantisation error itself (the bf16 rounding of the norm output is gone),
    on the prefill and the decode path."""
    from khaosz_amd import fuse_shared_inputs

    dev, dt = "cuda:0", torch.bfloat16
    flt = _block(dim=256, heads=4, kv=2, ffn=704).to(dev)
    a = _block(dim=256, heads=4, kv=2, ffn=704).to(dev).to(dt)
    a.load_state_dict({k: v.to(dt) for k, v in flt.state_dict().items()})
    b = _block(dim=256, heads=4, kv=2, ffn=704).to(dev).to(dt)
    b.load_state_dict(a.state_dict())
    quantize_model(a), quantize_model(b)
    fuse_shared_inputs(a)
    fuse_shared_inputs(b, norms=True)
    assert b._norm_quant and not a._norm_quant
    tab = rotary_table(64, 64, device=dev)
    x = torch.randn(2, 40, 256, device=dev)
    with torch.inference_mode():
        ref = flt(x, _freqs(tab, 2, 0, 40))
        for xs in (x.to(dt), x[:, :3].contiguous().to(dt)):            # M = 80 and M = 6
            S = xs.shape[1]
            ya, yb = a(xs, _freqs(tab, 2, 0, S)), b(xs, _freqs(tab, 2, 0, S))
            r = ref[:, :S]
            err_a = ((ya.float() - r).norm() / r.norm()).item()
            err_b = ((yb.float() - r).norm() / r.norm()).item()
            assert err_b < 3e-2 and err_b < 1.2 * err_a + 1e-3, (err_a, err_b)
            assert ((ya.float() - yb.float()).norm() / r.norm()).item() < 1.5e-2


@pytest.mark.gpu
def test_decode_attention_kernels_track_the_torch_attention_path():
    """Single-token steps on a paged cache through rope_kv_write + paged_attn_decode against the
    same quantized block running gather / repeat_kv / scaled_dot_product_attention: same cache
    contents up to one bf16 step of the rotation, outputs within bf16 rounding, for several steps."""
    from khaosz_amd import fuse_shared_inputs

    dev, dt = "cuda:0", torch.bfloat16
    torch.manual_seed(3)
    a = DecoderBlock(512, 4, 1408, 2)             # head dimension 128, two query heads per KV head
    a.reset_parameters()
    a = a.to(dev).to(dt)
    b = DecoderBlock(512, 4, 1408, 2).to(dev).to(dt)
    b.load_state_dict(a.state_dict())
    quantize_model(a), quantize_model(b)
    fuse_shared_inputs(a)
    fuse_shared_inputs(b, decode_attention=True)
    assert b.attention._decode_attention and not a.attention._decode_attention
    B, S, steps, page = 3, 70, 4, 16
    tab = rotary_table(128, 128, device=dev)
    table = torch.tensor([[7, 0, 9, 3, 12], [1, 8, 4, 10, 5], [2, 11, 6, 13, 14]], device=dev)
    ca, cb = PagedKV(16, page, 2, 128, dev, dt), PagedKV(16, page, 2, 128, dev, dt)
    x = torch.randn(B, S + steps, 512, device=dev).to(dt)
    with torch.inference_mode():
        pa = a(x[:, :S], _freqs(tab, B, 0, S), None, ca.bind(table, S))
        pb = b(x[:, :S], _freqs(tab, B, 0, S), None, cb.bind(table, S))
        # prefill: rope_kv_write over the prompt + attention over the new keys directly
        assert ((pa.float() - pb.float()).norm() / pa.float().norm()).item() < 1e-2
        assert torch.allclose(ca.k.float(), cb.k.float(), rtol=1e-2, atol=1e-2) and torch.equal(ca.v, cb.v)
        for t in range(steps):
            pos = S + t
            mask = decode_mask(B, pos + 1, dev, dt)
            ya = a(x[:, pos:pos + 1], _freqs(tab, B, pos, 1), mask, ca.bind(table, pos + 1))
            yb = b(x[:, pos:pos + 1], _freqs(tab, B, pos, 1), None, cb.bind(table, pos + 1))  # no mask tensor: the kernels
            rel = ((ya.float() - yb.float()).norm() / ya.float().norm()).item()
            assert rel < 1e-2, (t, rel)
        assert torch.allclose(ca.k.float(), cb.k.float(), rtol=1e-2, atol=1e-2) and torch.equal(ca.v, cb.v)
        # a second chunk of several tokens on top of the cached ones, and a table with an unmapped
        # page: both go through the gather, like the reference flow
        more = torch.randn(B, 5, 512, device=dev).to(dt)
        T = S + steps + 5
        cm = torch.zeros(B, 1, 5, T, device=dev, dtype=dt)
        cm[:, :, :, T - 5:] = torch.full((5, 5), float("-inf"), device=dev, dtype=dt).triu(1)
        ya = a(more, _freqs(tab, B, S + steps, 5), cm, ca.bind(table, T))
        yb = b(more, _freqs(tab, B, S + steps, 5), cm, cb.bind(table, T))
        assert ((ya.float() - yb.float()).norm() / ya.float().norm()).item() < 1e-2
        holes = table.clone()
        holes[1, 2] = -1
        ca2, cb2 = PagedKV(16, page, 2, 128, dev, dt), PagedKV(16, page, 2, 128, dev, dt)
        pa = a(x[:, :S], _freqs(tab, B, 0, S), None, ca2.bind(holes, S))
        pb = b(x[:, :S], _freqs(tab, B, 0, S), None, cb2.bind(holes, S))
        assert ((pa.float() - pb.float()).norm() / pa.float().norm()).item() < 1e-2
        assert torch.allclose(ca2.k.float(), cb2.k.float(), rtol=1e-2, atol=1e-2) and torch.equal(ca2.v, cb2.v)


@pytest.mark.gpu
def test_decode_step_with_the_merge_inside_the_output_projection_is_bit_identical(monkeypatch):
    """Past 256 cached positions the attention runs in slices; the output projection then combines them
    itself (one launch less).  Same bits as the path with the separate merge launch, with and without
    the residual in the epilogue."""
    from khaosz_amd import fuse_shared_inputs, ops

    dev, dt = "cuda:0", torch.bfloat16
    torch.manual_seed(5)
    for residuals in (False, True):
        blk = DecoderBlock(512, 8, 1408, 2)       # head dimension 64, four query heads per KV head
        blk.reset_parameters()
        blk = blk.to(dev).to(dt)
        quantize_model(blk)
        fuse_shared_inputs(blk, norms=True, decode_attention=True, residuals=residuals)
        B, S, page = 3, 300, 32
        P = (S + 8 + page - 1) // page
        tab = rotary_table(64, 512, device=dev)
        table = torch.randperm(B * P, device=dev).view(B, P)
        c1, c2 = PagedKV(B * P, page, 2, 64, dev, dt), PagedKV(B * P, page, 2, 64, dev, dt)
        x = torch.randn(B, S + 3, 512, device=dev).to(dt)
        calls = []
        real = ops.gemv_w8a8_attn
        monkeypatch.setattr(ops, "gemv_w8a8_attn", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
        with torch.inference_mode():
            blk(x[:, :S], _freqs(tab, B, 0, S), None, c1.bind(table, S))
            blk(x[:, :S], _freqs(tab, B, 0, S), None, c2.bind(table, S))
            for t in range(3):
                pos = S + t
                y1 = blk(x[:, pos:pos + 1], _freqs(tab, B, pos, 1), None, c1.bind(table, pos + 1))
                n = len(calls)
                assert n == t + 1                                      # the fused path ran
                with monkeypatch.context() as m:
                    m.setattr(ops, "attn_gemv_fusable", lambda *a: False)
                    y2 = blk(x[:, pos:pos + 1], _freqs(tab, B, pos, 1), None, c2.bind(table, pos + 1))
                assert len(calls) == n                                 # and here it did not
                assert torch.equal(y1, y2)
        assert torch.equal(c1.k, c2.k) and torch.equal(c1.v, c2.v)
        monkeypatch.undo()


@pytest.mark.gpu
def test_gated_attention_block_quantized_and_fused_paths_agree():
    """A block with the output gate: the gate is a fifth quantized Linear on the attention input; the
    fused paths (norm inside the projections, paged-cache kernels, residual epilogues) give the
    outputs of the plain quantized block within bf16 rounding, prefill and decode, and the
    quantized block tracks the float one."""
    from khaosz_amd import fuse_shared_inputs

    dev, dt = "cuda:0", torch.bfloat16
    torch.manual_seed(9)
    f = DecoderBlock(512, 8, 1408, 2, use_gated_attention=True)
    f.reset_parameters()
    f = f.to(dev).to(dt)
    a = DecoderBlock(512, 8, 1408, 2, use_gated_attention=True).to(dev).to(dt)
    b = DecoderBlock(512, 8, 1408, 2, use_gated_attention=True).to(dev).to(dt)
    a.load_state_dict(f.state_dict()), b.load_state_dict(f.state_dict())
    quantize_model(a), quantize_model(b)
    assert isinstance(a.attention.gate, QuantLinear)
    fuse_shared_inputs(b, norms=True, decode_attention=True, residuals=True)
    assert b.attention._decode_attention
    B, S, page = 3, 300, 32
    P = (S + 4 + page - 1) // page
    tab = rotary_table(64, 512, device=dev)
    table = torch.randperm(B * P, device=dev).view(B, P)
    cf, ca, cb = (PagedKV(B * P, page, 2, 64, dev, dt) for _ in range(3))
    x = torch.randn(B, S + 2, 512, device=dev).to(dt)
    rel = lambda u, w: ((u.float() - w.float()).norm() / w.float().norm()).item()
    with torch.inference_mode():
        pf = f(x[:, :S], _freqs(tab, B, 0, S), None, cf.bind(table, S))
        pa = a(x[:, :S], _freqs(tab, B, 0, S), None, ca.bind(table, S))
        pb = b(x[:, :S], _freqs(tab, B, 0, S), None, cb.bind(table, S))
        assert rel(pa, pf) < 3e-2 and rel(pb, pa) < 1e-2
        for t in range(2):
            pos = S + t
            mask = decode_mask(B, pos + 1, dev, dt)
            ya = a(x[:, pos:pos + 1], _freqs(tab, B, pos, 1), mask, ca.bind(table, pos + 1))
            yb = b(x[:, pos:pos + 1], _freqs(tab, B, pos, 1), None, cb.bind(table, pos + 1))  # no mask tensor: the kernels
            assert rel(yb, ya) < 1e-2, (t, rel(yb, ya))


@pytest.mark.gpu
def test_chunked_prefill_on_cached_tokens_uses_the_paged_kernel_and_tracks_the_masked_attention():
    """A second chunk of a prompt on top of cached tokens (a prefix-cache hit, executor.py:32-57 with
    start_pos > 0): the fused block reads K / V through the page table with causality by position; the
    plain quantized block runs gather + the stock attention under the explicit mask.  Outputs agree
    within bf16 rounding, the caches hold the same rows, and prefill in two chunks equals one pass."""
    from khaosz_amd import fuse_shared_inputs, ops

    dev, dt = "cuda:0", torch.bfloat16
    torch.manual_seed(21)
    a = DecoderBlock(512, 8, 1408, 2)
    a.reset_parameters()
    a = a.to(dev).to(dt)
    b = DecoderBlock(512, 8, 1408, 2).to(dev).to(dt)
    b.load_state_dict(a.state_dict())
    quantize_model(a), quantize_model(b)
    fuse_shared_inputs(a)
    fuse_shared_inputs(b, norms=False, decode_attention=True)
    B, S1, S2, page = 2, 150, 90, 32
    T = S1 + S2
    P = (T + page - 1) // page
    tab = rotary_table(64, 512, device=dev)
    table = torch.randperm(B * P, device=dev).view(B, P)
    ca, cb, cc = (PagedKV(B * P, page, 2, 64, dev, dt) for _ in range(3))
    x = torch.randn(B, T, 512, device=dev).to(dt)
    mask = torch.zeros(B, 1, S2, T, device=dev, dtype=dt)
    mask[:, :, :, S1:] = torch.full((S2, S2), float("-inf"), device=dev, dtype=dt).triu(1)
    rel = lambda u, w: ((u.float() - w.float()).norm() / w.float().norm()).item()
    calls = []
    real = ops.prefill_attn_paged
    ops.prefill_attn_paged = lambda *args, **kw: (calls.append(1), real(*args, **kw))[1]
    try:
        with torch.inference_mode():
            a(x[:, :S1], _freqs(tab, B, 0, S1), None, ca.bind(table, S1))
            b(x[:, :S1], _freqs(tab, B, 0, S1), None, cb.bind(table, S1))
            assert not calls                                       # an empty cache: the direct kernel
            ya = a(x[:, S1:], _freqs(tab, B, S1, S2), mask, ca.bind(table, T))
            yb = b(x[:, S1:], _freqs(tab, B, S1, S2), None, cb.bind(table, T))
            assert len(calls) == 1
            assert rel(yb, ya) < 1e-2
            assert torch.allclose(ca.k.float(), cb.k.float(), rtol=1e-2, atol=1e-2) and torch.equal(ca.v, cb.v)
            one = b(x, _freqs(tab, B, 0, T), None, cc.bind(table, T))
            assert rel(yb, one[:, S1:]) < 1e-2
    finally:
        ops.prefill_attn_paged = real


@pytest.mark.gpu
@pytest.mark.parametrize("B", [24, 40, 100])
def test_decode_batches_beyond_sixteen_sequences_fused_against_unfused(B):
    """Decode steps of more than 16 sequences leave the decode GEMV: the projections run as row quantiser (with
    the norm or the activation folded in) + the Linear on codes, which takes 17..32 rows on the weight-streaming
    kernel and more on its small tiles, residual adds in the epilogue, the attention on the paged cache in
    place.  Every fusion on against the plain quantized block (gather + torch attention), several steps, within
    the stated bf16 tolerance, caches included."""
    from khaosz_amd import fuse_shared_inputs

    dev, dt = "cuda:0", torch.bfloat16
    dim, Hq, Hkv, D, ffn, S, steps, page = 512, 4, 2, 128, 1408, 40, 3, 16
    torch.manual_seed(70 + B)
    plain = DecoderBlock(dim, Hq, ffn, Hkv)
    plain.reset_parameters()
    plain = plain.to(dev).to(dt)
    fused = DecoderBlock(dim, Hq, ffn, Hkv).to(dev).to(dt)
    fused.load_state_dict(plain.state_dict())
    assert quantize_model(plain) == 7 and quantize_model(fused) == 7
    fuse_shared_inputs(fused, norms=True, decode_attention=True, residuals=True)
    P = (S + steps + page - 1) // page
    n_pages = B * P + 3
    table = torch.randperm(n_pages)[:B * P].view(B, P).to(dev)
    ca, cb = PagedKV(n_pages, page, Hkv, D, dev, dt), PagedKV(n_pages, page, Hkv, D, dev, dt)
    tab = rotary_table(D, 128, device=dev)
    x = torch.randn(B, S + steps, dim, device=dev).to(dt)
    rel = lambda a, b: ((a.float() - b.float()).norm() / b.float().norm()).item()
    with torch.inference_mode():
        pa = plain(x[:, :S], _freqs(tab, B, 0, S), None, ca.bind(table, S))
        pb = fused(x[:, :S], _freqs(tab, B, 0, S), None, cb.bind(table, S))
        assert rel(pb, pa) < 1e-2
        for t in range(steps):
            pos = S + t
            ya = plain(x[:, pos:pos + 1], _freqs(tab, B, pos, 1), decode_mask(B, pos + 1, dev, dt), ca.bind(table, pos + 1))
            yb = fused(x[:, pos:pos + 1], _freqs(tab, B, pos, 1), None, cb.bind(table, pos + 1))
            assert yb.shape == (B, 1, dim) and rel(yb, ya) < 1e-2, (t, rel(yb, ya))
        # the norm folded into the quantiser skips a bf16 rounding, so codes (and with them k and v) move by
        # a quantisation step here and there: the caches agree as the outputs do
        assert rel(cb.k, ca.k) < 1e-2 and rel(cb.v, ca.v) < 1e-2


@pytest.mark.gpu
def test_config5_full_size_fused_block_against_the_unfused_block_and_an_oracle_composition(oracle):
    """Benchmark configuration 5 at its own size on the path the benchmark times: hidden 2048, 16 query /
    4 KV heads of 128, FFN 5632, every fusion on, 8 x 512 prefill through a shuffled table of 64-token pages,
    then decode steps of 8 tokens past 512 cached positions (position slices combined by the merge launch: at this size the output projection leaves that to it).
    (i) every step against the same weights in the unfused quantized block; (ii) one decode step against the
    decoder block (decoder_block.py:43-59) composed on the CPU from the oracle's functions: the q/k/v
    projection, the rotated queries and the cache contents bit for bit, everything behind the attention
    within the stated bf16 tolerance, and the MLP half bit for bit on the attention half's own output."""
    import numpy as np

    from khaosz_amd import fuse_shared_inputs

    def bits(t):
        return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16).copy()

    def from_bits(a):
        return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(torch.bfloat16)

    def add_bf16(a_bits, b_bits):  # the bits of a separate bf16 add
        return bits((from_bits(a_bits).float() + from_bits(b_bits).float()).to(torch.bfloat16))

    dev, dt = "cuda:0", torch.bfloat16
    dim, Hq, Hkv, D, ffn, B, S, steps, page = 2048, 16, 4, 128, 5632, 8, 512, 4, 64
    torch.manual_seed(55)
    plain = DecoderBlock(dim, Hq, ffn, Hkv)
    plain.reset_parameters()
    with torch.no_grad():
        plain.input_norm.weight.copy_(1 + 0.1 * torch.randn(dim))
        plain.post_attention_norm.weight.copy_(1 + 0.1 * torch.randn(dim))
    plain = plain.to(dev).to(dt)
    fused = DecoderBlock(dim, Hq, ffn, Hkv).to(dev).to(dt)
    fused.load_state_dict(plain.state_dict())
    assert quantize_model(plain) == 7 and quantize_model(fused) == 7
    fuse_shared_inputs(fused, norms=True, decode_attention=True, residuals=True)
    assert fused._norm_quant and fused._residual_adds and fused.attention._decode_attention

    P = (S + steps + page - 1) // page
    n_pages = B * P + 5
    table = torch.randperm(n_pages)[:B * P].view(B, P).to(dev)
    ca, cb = PagedKV(n_pages, page, Hkv, D, dev, dt), PagedKV(n_pages, page, Hkv, D, dev, dt)
    tab = rotary_table(D, 1024, device=dev)
    x = torch.randn(B, S + steps, dim, device=dev).to(dt)
    rel = lambda a, b: ((a.float() - b.float()).norm() / b.float().norm()).item()
    att, mlp = fused.attention, fused.mlp
    n1, n2 = fused.input_norm, fused.post_attention_norm
    with torch.inference_mode():
        pa = plain(x[:, :S], _freqs(tab, B, 0, S), None, ca.bind(table, S))
        pb = fused(x[:, :S], _freqs(tab, B, 0, S), None, cb.bind(table, S))
        assert rel(pb, pa) < 1e-2                      # stated bf16 tolerance
        assert rel(cb.k, ca.k) < 1e-2 and rel(cb.v, ca.v) < 1e-2
        for t in range(steps):
            pos = S + t
            xt, fr = x[:, pos:pos + 1], _freqs(tab, B, pos, 1)
            da = plain(xt, fr, decode_mask(B, pos + 1, dev, dt), ca.bind(table, pos + 1))
            if t == steps - 1:                         # state the oracle step starts from
                k0, v0 = bits(cb.k), bits(cb.v)
            db = fused(xt, fr, None, cb.bind(table, pos + 1))
            assert db.shape == (B, 1, dim) and rel(db, da) < 1e-2, (t, rel(db, da))
        # the last step once more in its two halves (an idempotent rewrite of the same cache slots)
        h_gpu = att(xt, fr, None, cb.bind(table, pos + 1), norm=(n1.weight, n1.norm_eps), residual=xt)
        out_gpu = mlp(h_gpu, norm=(n2.weight, n2.norm_eps), residual=h_gpu)
        assert torch.equal(out_gpu, db)
        qkv_gpu = att._qkv(xt, norm=(n1.weight, n1.norm_eps))

    # ---- the same step on the CPU, from the oracle's functions
    T = pos + 1
    xb = bits(xt.reshape(B, dim))
    qkv_w, qkv_s = att._qkv.qweight.cpu().numpy(), att._qkv.w_scale.cpu().numpy()
    xq, sx = oracle.c_rmsnorm_quant_i8(xb, bits(n1.weight), n1.norm_eps, bf16_bits=True)
    qkv = oracle.c_dequant_epilogue(oracle.c_gemm_i8_i32(xq, qkv_w), sx, qkv_s, bf16_out=True)
    assert np.array_equal(bits(qkv_gpu.reshape(B, -1)), qkv)                      # bit for bit
    fr_np = np.ascontiguousarray(torch.view_as_real(fr.reshape(B, D // 2)).cpu().numpy())
    q_rot = oracle.c_rope_kv_write(qkv, fr_np, table.cpu().numpy(), pos, k0, v0, Hq, Hkv)
    assert np.array_equal(bits(cb.k), k0) and np.array_equal(bits(cb.v), v0)      # the cache after the step, bit for bit
    attn = oracle.c_paged_attn_decode(q_rot, k0, v0, table.cpu().numpy(), T, D ** -0.5)
    o = oracle.c_linear_w8a8(attn.reshape(B, Hq * D), att.o_proj.qweight.cpu().numpy(), att.o_proj.w_scale.cpu().numpy(),
                             x_bf16_bits=True, bf16_out=True)
    h = add_bf16(o, xb)
    assert rel(h_gpu.reshape(B, dim).cpu(), from_bits(h)) < 1e-2                  # behind the attention: stated tolerance

    def mlp_half(h_bits):
        hq, hs = oracle.c_rmsnorm_quant_i8(h_bits, bits(n2.weight), n2.norm_eps, bf16_bits=True)
        ug = oracle.c_dequant_epilogue(oracle.c_gemm_i8_i32(hq, mlp._upgate.qweight.cpu().numpy()), hs,
                                       mlp._upgate.w_scale.cpu().numpy(), bf16_out=True)
        # a decode step: up, gate and the activation are one launch that rounds h to bf16, and `down` quantises
        # those bf16 rows itself (the prefill's activation kernel quantises h from fp32 instead)
        _, _, hf = oracle.c_swiglu_quant_i8(ug, bf16_bits=True, want_h=True)
        aq, asc = oracle.c_quant_rowwise_i8(oracle.np_f32_to_bf16_bits(hf), bf16_bits=True)
        d = oracle.c_dequant_epilogue(oracle.c_gemm_i8_i32(aq, mlp.down.qweight.cpu().numpy()), asc,
                                      mlp.down.w_scale.cpu().numpy(), bf16_out=True)
        return add_bf16(d, h_bits)

    assert rel(out_gpu.reshape(B, dim).cpu(), from_bits(mlp_half(h))) < 1e-2      # whole step, oracle end to end
    # the MLP half on the bits the GPU's attention half produced: norm + quantise, up/gate + SwiGLU, quantise,
    # down and the residual add, bit for bit
    assert np.array_equal(bits(out_gpu.reshape(B, dim)), mlp_half(bits(h_gpu.reshape(B, dim))))


@pytest.mark.gpu
def test_qk_norm_block_through_the_paged_cache_kernels_tracks_the_stock_path():
    """use_qk_norm with the paged-cache kernels: they normalise the rotated heads and cache the normalised
    key (attention.py:86-92).  Against the same quantized block on gather / repeat_kv / stock attention:
    prompt, a chunk on top of cached tokens, decode steps in one slice and in several; cache contents
    within one bf16 step, outputs within bf16 rounding."""
    from khaosz_amd import fuse_shared_inputs

    dev, dt = "cuda:0", torch.bfloat16
    for dim, heads, kv, S in ((512, 4, 2, 70), (512, 8, 2, 290)):       # head dimension 128 and 64
        torch.manual_seed(11)
        a = DecoderBlock(dim, heads, 1408, kv, use_qk_norm=True)
        a.reset_parameters()
        with torch.no_grad():
            a.attention.q_norm.weight.add_(0.3 * torch.randn_like(a.attention.q_norm.weight))
            a.attention.k_norm.weight.add_(0.3 * torch.randn_like(a.attention.k_norm.weight))
        a = a.to(dev).to(dt)
        b = DecoderBlock(dim, heads, 1408, kv, use_qk_norm=True).to(dev).to(dt)
        b.load_state_dict(a.state_dict())
        quantize_model(a), quantize_model(b)
        fuse_shared_inputs(a)
        fuse_shared_inputs(b, decode_attention=True)
        assert b.attention._decode_attention and not a.attention._decode_attention
        D = dim // heads
        B, steps, page = 3, 3, 16
        P = (S + steps + 5 + page - 1) // page
        tab = rotary_table(D, 512, device=dev)
        table = torch.randperm(B * P, device=dev).view(B, P)
        ca, cb = PagedKV(B * P, page, kv, D, dev, dt), PagedKV(B * P, page, kv, D, dev, dt)
        x = torch.randn(B, S + steps, dim, device=dev).to(dt)
        with torch.inference_mode():
            pa = a(x[:, :S], _freqs(tab, B, 0, S), None, ca.bind(table, S))
            pb = b(x[:, :S], _freqs(tab, B, 0, S), None, cb.bind(table, S))
            assert ((pa.float() - pb.float()).norm() / pa.float().norm()).item() < 1e-2
            assert torch.allclose(ca.k.float(), cb.k.float(), rtol=1e-2, atol=1e-2) and torch.equal(ca.v, cb.v)
            # the keys in the cache are unit-RMS times the gain: nothing like the un-normalised ones
            rms = cb.k[table[0, 0], 0, 0].float().div(b.attention.k_norm.weight.float()).pow(2).mean().sqrt().item()
            assert abs(rms - 1.0) < 2e-2
            for t in range(steps):
                pos = S + t
                mask = decode_mask(B, pos + 1, dev, dt)
                ya = a(x[:, pos:pos + 1], _freqs(tab, B, pos, 1), mask, ca.bind(table, pos + 1))
                yb = b(x[:, pos:pos + 1], _freqs(tab, B, pos, 1), None, cb.bind(table, pos + 1))
                rel = ((ya.float() - yb.float()).norm() / ya.float().norm()).item()
                assert rel < 1e-2, (dim, heads, t, rel)
            assert torch.allclose(ca.k.float(), cb.k.float(), rtol=1e-2, atol=1e-2) and torch.equal(ca.v, cb.v)
            more = torch.randn(B, 5, dim, device=dev).to(dt)           # a chunk on top of the cached tokens
            T = S + steps + 5
            cm = torch.zeros(B, 1, 5, T, device=dev, dtype=dt)
            cm[:, :, :, T - 5:] = torch.full((5, 5), float("-inf"), device=dev, dtype=dt).triu(1)
            ya = a(more, _freqs(tab, B, S + steps, 5), cm, ca.bind(table, T))
            yb = b(more, _freqs(tab, B, S + steps, 5), None, cb.bind(table, T))
            assert ((ya.float() - yb.float()).norm() / ya.float().norm()).item() < 1e-2
            assert torch.allclose(ca.k.float(), cb.k.float(), rtol=1e-2, atol=1e-2)
