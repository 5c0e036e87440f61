"""The reference's other callers of Linear -- multi-head latent attention (attention.py:140-156: q_proj,
kv_a_proj, kv_b_proj with K = kv_lora_rank, o_proj, gate) and DeepSeekMoE (mlp.py:48-91: a router with
N = n_routed_experts, experts fed the ragged 2-D gather x[token_idx]) -- through quantize_model and the
quantized path, bit for bit against the oracle.  The modules below carry the reference's child names and
are built from a stand-in for its Linear class that this package recognises by name only."""
import sys

import numpy as np
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

pytestmark = pytest.mark.gpu

from khaosz_amd.linear import Linear, QuantLinear, quantize_model  # noqa: E402

DEV = "cuda:0"


def _say(*a):
    print(*a, file=sys.stderr, flush=True)


def bf16_bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


class RefLinear(nn.Module):
    """linear.py:7-21 of the reference, under its name and module path, unrelated to this package's Linear."""

    def __init__(self, in_dim, out_dim, bias=False):
        super().__init__()
        self.weight = nn.Parameter(torch.randn(out_dim, in_dim) / in_dim ** 0.5)
        self.bias = nn.Parameter(torch.randn(out_dim) * 0.01) if bias else None

    def forward(self, x):
        return F.linear(x, self.weight, self.bias)


RefLinear.__name__ = RefLinear.__qualname__ = "Linear"
RefLinear.__module__ = "astrai.model.components.linear"


class RefMLP(nn.Module):  # mlp.py:17-27
    def __init__(self, dim, dim_ffn):
        super().__init__()
        self.up, self.gate, self.down = RefLinear(dim, dim_ffn), RefLinear(dim, dim_ffn), RefLinear(dim_ffn, dim)

    def forward(self, x):
        return self.down(F.silu(self.gate(x)) * self.up(x))


RefMLP.__name__ = RefMLP.__qualname__ = "MLP"
RefMLP.__module__ = "astrai.model.components.mlp"


class RefMoE(nn.Module):
    """The routed half of DeepSeekMoE (mlp.py:72-93): top-k of a softmax over the router's logits, each
    expert run on the rows routed to it."""

    def __init__(self, dim, dim_ffn, n_experts, k):
        super().__init__()
        self.k = k
        self.router = RefLinear(dim, n_experts)
        self.routed_experts = nn.ModuleList([RefMLP(dim, dim_ffn) for _ in range(n_experts)])
        self.seen = []  # rows each expert was handed in the last forward

    def forward(self, x):
        probs = torch.softmax(self.router(x).float(), dim=-1).to(x.dtype)
        w, idx = torch.topk(probs, self.k, dim=-1)
        w = w / w.sum(dim=-1, keepdim=True)
        out = torch.zeros_like(x)
        self.seen = []
        for e, expert in enumerate(self.routed_experts):
            tok, slot = (idx == e).nonzero(as_tuple=True)
            self.seen.append(int(tok.numel()))
            if tok.numel() == 0:
                continue
            out.index_add_(0, tok, expert(x[tok]) * w[tok, slot].unsqueeze(-1))
        return out


def _oracle_linear(oracle, q: QuantLinear, x: torch.Tensor) -> np.ndarray:
    """bf16 bit patterns the oracle gives for this module on these rows"""
    bias = None if q.bias is None else q.bias.detach().float().cpu().numpy()
    return oracle.c_linear_w8a8(bf16_bits(x), q.qweight.cpu().numpy(), q.w_scale.cpu().numpy(), bias,
                                x_bf16_bits=True, bf16_out=True)


@pytest.mark.parametrize("rows", [0, 1, 5, 16, 17, 33, 100, 259])
def test_expert_on_a_ragged_gather_of_rows(oracle, rows):
    """mlp.py:83-91: an expert's input is x[token_idx], a fresh 2-D tensor with any number of rows
    (none included, though the reference skips that case); every row count lands on the decode kernel,
    the tiled GEMM or nothing, and gives the oracle's bits."""
    _say("expert rows", rows)
    torch.manual_seed(rows)
    mlp = RefMLP(256, 704).to(DEV)
    assert quantize_model(mlp) == 3
    x = torch.randn(300, 256, device=DEV, dtype=torch.bfloat16)
    tok = torch.randperm(300, device=DEV)[:rows].sort().values
    xin = x[tok]
    with torch.inference_mode():
        for name in ("up", "gate"):
            y = getattr(mlp, name)(xin)
            assert y.shape == (rows, 704) and y.dtype == torch.bfloat16
            if rows:
                assert np.array_equal(bf16_bits(y), _oracle_linear(oracle, getattr(mlp, name), xin)), name
        h = F.silu(mlp.gate(xin)) * mlp.up(xin)
        y = mlp.down(h)
        assert y.shape == (rows, 256)
        if rows:
            assert np.array_equal(bf16_bits(y), _oracle_linear(oracle, mlp.down, h))
        assert mlp(xin).shape == (rows, 256)


@pytest.mark.parametrize("n_experts", [8, 64])
def test_router_sized_projection_and_a_whole_routed_layer(oracle, n_experts):
    """mlp.py:48: the router is a Linear with N = n_routed_experts.  It stays in floating point by default
    (its logits feed a top-k) and is quantized when named; quantized, its few output columns match the
    oracle for decode-sized and prefill-sized batches.  The routed layer with quantized experts follows
    the float layer within the quantisation noise, experts without a token included."""
    _say("router", n_experts)
    torch.manual_seed(n_experts)
    moe = RefMoE(256, 352, n_experts, 2).to(DEV).to(torch.bfloat16)
    x = torch.randn(40, 256, device=DEV, dtype=torch.bfloat16)
    with torch.inference_mode():
        ref = moe(x)
    assert quantize_model(moe) == 3 * n_experts and type(moe.router) is RefLinear
    with torch.inference_mode():
        got = moe(x)                       # same float router -> same routing, quantized experts
        assert sum(moe.seen) == 40 * 2 and (n_experts == 8 or 0 in moe.seen)
        assert (got.float() - ref.float()).norm() / ref.float().norm() < 5e-2
    assert quantize_model(moe, target_modules={"router"}) == 1 and isinstance(moe.router, QuantLinear)
    with torch.inference_mode():
        for rows in (1, 7, 16, 40):
            y = moe.router(x[:rows])
            assert y.shape == (rows, n_experts)
            assert np.array_equal(bf16_bits(y), _oracle_linear(oracle, moe.router, x[:rows])), rows


class RefMLAProjections(nn.Module):
    """The Linear calls of MLA.forward (attention.py:166-176, 209-212) with its child names; the attention
    between them is not restated."""

    def __init__(self, dim, n_heads, n_kv_heads, kv_lora_rank, head_dim):
        super().__init__()
        self.q_proj = RefLinear(dim, n_heads * head_dim)
        self.kv_a_proj = RefLinear(dim, kv_lora_rank)
        self.kv_b_proj = RefLinear(kv_lora_rank, n_kv_heads * 2 * head_dim)
        self.o_proj = RefLinear(dim, dim)
        self.gate = RefLinear(dim, dim)


@pytest.mark.parametrize("tokens", [(2, 1), (4, 4), (2, 48)])
def test_mla_projections_through_the_default_targets(oracle, tokens):
    """kv_a_proj (N = kv_lora_rank), kv_b_proj (K = kv_lora_rank, N = n_kv_heads x 2 x head_dim) and the
    others take the default target set; 3-D inputs [batch, seq, dim] at decode and prefill sizes."""
    _say("mla", tokens)
    torch.manual_seed(7)
    dim, kv_rank, head_dim = 512, 128, 96   # head_dim = nope 64 + rope 32
    m = RefMLAProjections(dim, 8, 2, kv_rank, head_dim).to(DEV)
    assert quantize_model(m) == 5
    B, S = tokens
    x = torch.randn(B, S, dim, device=DEV, dtype=torch.bfloat16)
    with torch.inference_mode():
        for name in ("q_proj", "kv_a_proj", "o_proj", "gate"):
            q = getattr(m, name)
            y = q(x)
            assert y.shape == (B, S, q.out_dim)
            assert np.array_equal(bf16_bits(y).reshape(B * S, -1), _oracle_linear(oracle, q, x.reshape(B * S, dim))), name
        c = m.kv_a_proj(x)
        kv = m.kv_b_proj(c)
        assert kv.shape == (B, S, 2 * 2 * head_dim)
        assert np.array_equal(bf16_bits(kv).reshape(B * S, -1), _oracle_linear(oracle, m.kv_b_proj, c.reshape(B * S, kv_rank)))


def test_reference_class_with_a_bias_and_this_packages_linear_quantize_alike(oracle):
    torch.manual_seed(3)
    ref = RefLinear(128, 80, bias=True).to(DEV)
    own = Linear(128, 80, bias=True).to(DEV)
    own.load_state_dict(ref.state_dict())
    holder = nn.ModuleDict({"up": ref, "down": own})
    assert quantize_model(holder) == 2
    x = torch.randn(9, 128, device=DEV, dtype=torch.bfloat16)
    with torch.inference_mode():
        a, b = holder["up"](x), holder["down"](x)
    assert torch.equal(a, b)
    assert np.array_equal(bf16_bits(a), _oracle_linear(oracle, holder["up"], x))


class RefGQAProjections(nn.Module):
    """The Linear calls of the reference's GQA.forward in its order (attention.py:83-85, 105-108), under its
    class name; what lies between them is replaced by a fixed mixing of q, k and v."""

    def __init__(self, dim, n_heads, n_kv_heads, gated):
        super().__init__()
        hd = dim // n_heads
        self.q_proj, self.k_proj, self.v_proj = RefLinear(dim, dim), RefLinear(dim, n_kv_heads * hd), RefLinear(dim, n_kv_heads * hd)
        self.o_proj = RefLinear(dim, dim)
        self.rep = n_heads // n_kv_heads
        if gated:
            self.gate = RefLinear(dim, dim)
        self.gated = gated

    def forward(self, x):
        B, S, _ = x.shape
        q = self.q_proj(x).reshape(B, S, -1, 32)
        k = self.k_proj(x).reshape(B, S, -1, 32)
        v = self.v_proj(x).reshape(B, S, -1, 32)
        out = (q + k.repeat_interleave(self.rep, 2) * v.repeat_interleave(self.rep, 2)).flatten(2)
        if self.gated:
            out = out * torch.sigmoid(self.gate(x))
        return self.o_proj(out)


RefGQAProjections.__name__ = RefGQAProjections.__qualname__ = "GQA"
RefGQAProjections.__module__ = "astrai.model.components.attention"


class RefMLA(RefMLAProjections):
    """MLA.forward's Linear calls in order (attention.py:166-176, 205-209): q_proj(x), kv_a_proj(x), a norm,
    kv_b_proj, the gate on x, o_proj."""

    def forward(self, x):
        B, S, _ = x.shape
        q = self.q_proj(x)
        q = q.view(B, S, 8, -1)                              # a view, as the reference takes it
        c = self.kv_a_proj(x)
        c = F.rms_norm(c, (c.shape[-1],))
        kv = self.kv_b_proj(c).view(B, S, 2, -1)
        mixed = q.flatten(2)[..., :x.shape[-1]] * kv.flatten(2).mean(-1, keepdim=True)
        return self.o_proj(mixed * torch.sigmoid(self.gate(x)))


RefMLA.__name__ = RefMLA.__qualname__ = "MLA"
RefMLA.__module__ = "astrai.model.components.attention"


def _count_launches(monkeypatch):
    from khaosz_amd import ops
    calls = []
    for name in ("gemv_w8a8_decode", "linear_w8a8", "quant_rowwise_i8"):
        real = getattr(ops, name)
        monkeypatch.setattr(ops, name, (lambda real, name: lambda *a, **k: (calls.append(name), real(*a, **k))[1])(real, name))
    return calls


@pytest.mark.parametrize("tokens", [(2, 1), (3, 4), (2, 48)])
def test_reference_modules_share_one_launch_behind_their_own_forward(monkeypatch, tokens):
    """fuse_shared_inputs on modules that carry the reference's class names (GQA, MLA, MLP and the experts of a
    routed layer): their forward is untouched, the projections of one input run as one concatenated launch
    (one activation quantisation), outputs and state-dict keys are what they were, bit for bit -- at decode
    sizes, where the GEMV quantises its rows itself, and at prefill sizes."""
    from khaosz_amd import fuse_shared_inputs
    _say("shared inputs of reference modules", tokens)
    torch.manual_seed(11)
    B, S = tokens
    dim = 256
    mods = {"gqa": RefGQAProjections(dim, 8, 2, gated=True), "gqa_plain": RefGQAProjections(dim, 8, 4, gated=False),
            "mla": RefMLA(dim, 8, 2, 128, 96), "mlp": RefMLP(dim, 704)}
    x = torch.randn(B, S, dim, device=DEV, dtype=torch.bfloat16)
    for name, m in mods.items():
        m = m.to(DEV)
        assert quantize_model(m) > 0
        keys = sorted(m.state_dict().keys())
        calls = _count_launches(monkeypatch)
        with torch.inference_mode():
            want = m(x)
        before = calls.count("gemv_w8a8_decode") + calls.count("linear_w8a8")
        assert fuse_shared_inputs(m) == 1, name
        assert sorted(m.state_dict().keys()) == keys
        del calls[:]
        with torch.inference_mode():
            got = m(x)
            again = m(x)                                     # nothing stale is served on a second pass
        after = (calls.count("gemv_w8a8_decode") + calls.count("linear_w8a8")) // 2
        saved = {"gqa": 3, "gqa_plain": 2, "mla": 2, "mlp": 1}[name]
        assert before - after == saved, (name, before, after)
        assert torch.equal(got, want) and torch.equal(again, want), name
        # a tensor modified in place between two calls is a new input (where torch tracks versions)
        y = x.clone()
        first = m.q_proj(y) if hasattr(m, "q_proj") else m.up(y)
        y.mul_(2.0)
        second = m.q_proj(y) if hasattr(m, "q_proj") else m.up(y)
        assert not torch.equal(first, second)
        monkeypatch.undo()


def test_routed_experts_share_up_and_gate(monkeypatch):
    """Every expert of a routed layer is an MLP of the reference (mlp.py:17-27, 53-55): up and gate of an expert
    read the same gathered rows x[token_idx] and become one launch; the layer's output keeps its bits."""
    from khaosz_amd import fuse_shared_inputs
    torch.manual_seed(5)
    moe = RefMoE(256, 352, 8, 2).to(DEV).to(torch.bfloat16)
    x = torch.randn(40, 256, device=DEV, dtype=torch.bfloat16)
    assert quantize_model(moe) == 24
    with torch.inference_mode():
        want = moe(x)
    assert fuse_shared_inputs(moe) == 8
    with torch.inference_mode():
        assert torch.equal(moe(x), want)
