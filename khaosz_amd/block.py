"""The callers of Linear inside one decoder block, restated so that the
quantized path can be exercised at the shapes a real model presents.

Structure follows the reference (pre-norm residual block with GQA and a SwiGLU
MLP), each piece citing the file it restates; only the seven projections are
this package's own arithmetic, everything else is the same stock torch call the
reference makes.  Two KV caches offer the two methods attention needs (``write`` / ``gather``,
the ``KvcacheView`` interface, astrai/inference/core/cache.py:277-290): a
contiguous per-sequence buffer, and a paged one with the storage layout and the
write / gather semantics of the reference's ``Storage`` (cache.py:187-274).
Page allocation, prefix sharing and eviction belong to the serving layer and are
not restated: the page table is handed in.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor

from . import ops
from .linear import Linear, QuantLinear


class RMSNorm(nn.Module):
    """``F.rms_norm`` with a learned gain (astrai/model/components/norm.py:7-15)."""

    def __init__(self, dim: int, norm_eps: float):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.norm_eps = norm_eps

    def forward(self, x: Tensor) -> Tensor:
        return F.rms_norm(x, (x.shape[-1],), self.weight, self.norm_eps)


def rotary_table(head_dim: int, max_len: int, base: float = 10000.0, device=None) -> Tensor:
    """complex64 ``[max_len, head_dim/2]`` with angle ``t * base**(-2i/d)``
    (astrai/model/components/rope.py:8-19: float64 angles, float32 cos/sin)."""
    inv = base ** (-torch.arange(0, head_dim, 2, dtype=torch.float64, device=device) / head_dim)
    ang = torch.outer(torch.arange(max_len, dtype=torch.float64, device=device), inv).float()
    return torch.polar(torch.ones_like(ang), ang)


def apply_rotary(x: Tensor, freqs: Tensor) -> Tensor:
    """Rotate interleaved pairs ``(x[2i], x[2i+1])`` of ``x [B, S, H, D]`` by ``freqs [B, S, D/2]``
    in float32 and cast back (rope.py:26-33)."""
    xc = torch.view_as_complex(x.float().reshape(*x.shape[:-1], -1, 2))
    out = torch.view_as_real(xc * freqs.unsqueeze(2)).flatten(-2)
    return out.to(x.dtype)


class ContiguousKV:
    """KV cache for one block: ``[B, max_len, Hkv, D]``; ``total_len`` is the length after the
    tokens being written, as in ``KvcacheView`` (cache.py:282-290)."""

    def __init__(self, batch: int, max_len: int, n_kv_heads: int, head_dim: int, device, dtype):
        self.k = torch.zeros((batch, max_len, n_kv_heads, head_dim), device=device, dtype=dtype)
        self.v = torch.zeros_like(self.k)
        self.total_len = 0

    def bind(self, total_len: int) -> "ContiguousKV":
        self.total_len = total_len
        return self

    def write(self, layer_id: int, k: Tensor, v: Tensor) -> None:
        start = self.total_len - k.size(1)
        self.k[:, start:self.total_len] = k
        self.v[:, start:self.total_len] = v

    def gather(self, layer_id: int) -> Tuple[Tensor, Tensor]:
        return self.k[:, :self.total_len], self.v[:, :self.total_len]


class PagedKV:
    """Paged KV cache for ``n_layers`` blocks (one by default): pages
    ``[n_layers, n_pages, page_size, Hkv, D]`` (cache.py:187-214) and a page table
    ``[B, pages_per_sequence]`` of physical page ids, -1 for a logical page that is not
    mapped (cache.py:187-274).  ``write`` places the new tokens at logical positions
    ``total_len - S .. total_len`` page by page; rows whose page is unmapped are skipped.
    ``gather`` materialises ``[B, total_len, Hkv, D]`` through the table, zeros where unmapped.
    Which table entries are mapped is decided on a host copy of the table made at bind time,
    so neither method synchronises with the device (the reference tests the device tensor,
    ``cache.py:233,262``) and both can be captured in a HIP graph.  That host copy is made when a
    table tensor is first bound: a table that was changed in place (a page mapped as a sequence grew)
    must be bound again with ``refresh=True`` -- or be a new tensor, as the reference's
    ``make_table_tensor`` produces for every step.
    ``seq_lens`` (int64 ``[B]`` on the device, optional): the positions each sequence may attend to
    in a single-token step whose sequences sit at different positions; the attention kernels apply it as
    the reference's position mask (transformer.py:40-46)."""

    def __init__(self, n_pages: int, page_size: int, n_kv_heads: int, head_dim: int, device, dtype,
                 n_layers: int = 1):
        self.page_size = page_size
        self.k_layers = torch.zeros((n_layers, n_pages, page_size, n_kv_heads, head_dim), device=device, dtype=dtype)
        self.v_layers = torch.zeros_like(self.k_layers)
        self.page_table: Optional[Tensor] = None
        self._attn_ws: Optional[Tensor] = None
        self._mapped = None      # host bool [B, P]
        self._safe = None        # device table with -1 replaced by 0
        self._invalid = None     # device bool [B, P * page_size] or None when everything is mapped
        self.total_len = 0
        self.seq_lens: Optional[Tensor] = None

    def bind(self, page_table: Optional[Tensor] = None, total_len: int = 0, seq_lens: Optional[Tensor] = None,
             refresh: bool = False) -> "PagedKV":
        if page_table is not None and (refresh or page_table is not self.page_table):
            host = page_table.detach().cpu()
            self.page_table = page_table
            self._mapped = host >= 0
            self._safe = page_table.clamp(min=0)
            self._invalid = None
            if not bool(self._mapped.all()):
                inv = (~self._mapped).unsqueeze(-1).expand(-1, -1, self.page_size).flatten(1, 2)
                self._invalid = inv.to(page_table.device)
        if self.page_table is None:
            raise ValueError("bind() needs a page table")
        self.total_len = total_len
        self.seq_lens = seq_lens
        return self

    def attn_workspace(self, n_heads: int) -> Optional[Tensor]:
        """Scratch for the decode attention kernel's partial results, sized once for the longest
        sequence the bound page table can hold and shared by all layers (they run one after the other)."""
        B, P = self.page_table.shape
        need = ops.paged_attn_partials_bytes(B, n_heads, P * self.page_size)
        if self._attn_ws is None or self._attn_ws.numel() * 4 < need:
            self._attn_ws = torch.empty(need // 4, dtype=torch.float32, device=self.k_layers.device)
        return self._attn_ws

    @property
    def k(self) -> Tensor:
        """Layer 0's key pages (the whole cache of a single block)."""
        return self.k_layers[0]

    @property
    def v(self) -> Tensor:
        return self.v_layers[0]

    @property
    def all_mapped(self) -> bool:
        """Every entry of the bound page table names a page."""
        return self._invalid is None

    def write(self, layer_id: int, k: Tensor, v: Tensor) -> None:
        S = k.size(1)
        if S == 0:
            return
        start, ps = self.total_len - S, self.page_size
        if start < 0 or (self.total_len + ps - 1) // ps > self.page_table.size(1):
            raise ValueError("tokens fall outside the page table")
        kc, vc = self.k_layers[layer_id], self.v_layers[layer_id]
        done = 0
        for pi in range(start // ps, (self.total_len - 1) // ps + 1):
            lo = max(pi * ps, start)
            hi = min((pi + 1) * ps, self.total_len)
            off, n = lo - pi * ps, hi - lo
            rows = self._mapped[:, pi]
            if bool(rows.all()):
                phys = self._safe[:, pi]
                kc[phys, off:off + n] = k[:, done:done + n]
                vc[phys, off:off + n] = v[:, done:done + n]
            elif bool(rows.any()):
                sel = rows.nonzero().flatten().to(k.device)
                phys = self._safe[sel, pi]
                kc[phys, off:off + n] = k[sel, done:done + n]
                vc[phys, off:off + n] = v[sel, done:done + n]
            done += n

    def gather(self, layer_id: int) -> Tuple[Tensor, Tensor]:
        k = self.k_layers[layer_id][self._safe].flatten(1, 2)
        v = self.v_layers[layer_id][self._safe].flatten(1, 2)
        if self._invalid is not None:
            m = self._invalid[:, :, None, None]
            k, v = k.masked_fill(m, 0.0), v.masked_fill(m, 0.0)
        return k[:, :self.total_len], v[:, :self.total_len]


class GQA(nn.Module):
    """Grouped-query attention (astrai/model/components/attention.py:32-109), with its two
    options: RMSNorm over the head dimension of q and k after the rotation (``use_qk_norm``,
    attention.py:62-64,88-89) and a sigmoid output gate computed from the block input by a fifth
    Linear (``use_gated_attention``, attention.py:66-67,105-106).  Benchmark configuration 5
    leaves both off.  With qk-norm the paged-cache kernels normalise the rotated heads themselves and
    cache the normalised key, as the reference does."""

    def __init__(self, dim: int, n_heads: int, n_kv_heads: int, layer_id: int = 0, use_qk_norm: bool = False,
                 norm_eps: float = 1e-5, use_gated_attention: bool = False):
        super().__init__()
        if dim % n_heads or n_heads % n_kv_heads:
            raise ValueError("dim must divide into heads and heads into kv heads")
        self.head_dim = dim // n_heads
        self.n_heads, self.n_kv_heads, self.layer_id = n_heads, n_kv_heads, layer_id
        self.use_qk_norm, self.use_gated_attention = use_qk_norm, use_gated_attention
        self.q_proj = Linear(dim, n_heads * self.head_dim)
        self.k_proj = Linear(dim, n_kv_heads * self.head_dim)
        self.v_proj = Linear(dim, n_kv_heads * self.head_dim)
        self.o_proj = Linear(dim, dim)
        if use_qk_norm:
            self.q_norm = RMSNorm(self.head_dim, norm_eps)
            self.k_norm = RMSNorm(self.head_dim, norm_eps)
        if use_gated_attention:
            self.gate = Linear(dim, dim)
        self._qkv: Optional[QuantLinear] = None  # not a registered child: the state dict keeps q/k/v keys
        self._decode_attention = False

    def fuse_projections(self) -> bool:
        """q, k and v read the same input (attention.py:83-85): once they are quantized, run them
        as one ``[Hq*D + 2*Hkv*D, dim]`` projection -- one activation quantisation, one launch."""
        if self._qkv is None and all(isinstance(m, QuantLinear) for m in (self.q_proj, self.k_proj, self.v_proj)):
            object.__setattr__(self, "_qkv", QuantLinear.concat([self.q_proj, self.k_proj, self.v_proj]))
            return True
        return False

    def fuse_decode_attention(self) -> bool:
        """Use the paged-cache kernels.  A step with one new token per sequence rotates q/k,
        writes k/v into their page slot and attends over the pages in place, all in one launch
        (``ops.rope_paged_attn_decode``), instead of the gather / repeat_kv / generic attention
        sequence; it assumes what the serving loop's decode step has: no padding inside the
        cached length (the additive mask is all zeros).  Several new tokens (prefill) get the
        rotation and the page writes as one launch (``ops.rope_kv_write``) in front of the stock
        attention, which then reads the new keys directly and shares KV heads without
        repeating them.  Needs the fused q/k/v projection, bf16, head dimension 64 or 128 and
        1, 2, 3, 4, 6 or 8 query heads per KV head.
        Outputs agree within bf16 rounding."""
        if (self._qkv is not None and self.head_dim in (64, 128)
                and self.n_heads // self.n_kv_heads in (1, 2, 3, 4, 6, 8)):
            self._decode_attention = True
        return self._decode_attention

    def _qk_norm(self) -> Optional[ops.QkNorm]:
        """The two head norms for the paged-cache kernels (which compute in bf16 activations)."""
        if not self.use_qk_norm:
            return None
        return ops.QkNorm(self.q_norm.weight.detach().to(torch.bfloat16), self.k_norm.weight.detach().to(torch.bfloat16),
                          self.q_norm.norm_eps)

    def _gated(self, out: Tensor, x: Tensor, norm, codes=None) -> Tensor:
        """``out * sigmoid(gate(x))`` (attention.py:105-106); ``x`` is the attention input, still to
        be normalised when ``norm`` is given, or replaced by its quantised form ``codes``."""
        if not self.use_gated_attention:
            return out
        if codes is not None:
            if not isinstance(self.gate, QuantLinear):
                raise ValueError("a pre-quantised input needs a quantized gate projection")
            g = self.gate.forward_codes(codes[0], codes[1], x.dtype)
        elif norm is None:
            g = self.gate(x)
        elif isinstance(self.gate, QuantLinear):
            g = self.gate(x, norm=norm)
        else:
            g = self.gate(F.rms_norm(x, (x.shape[-1],), norm[0], norm[1]))
        return out * torch.sigmoid(g).view(out.shape)

    def _out(self, out: Tensor, residual: Optional[Tensor]) -> Tensor:
        """o_proj, plus the residual stream when the caller hands it over."""
        if residual is None:
            return self.o_proj(out)
        if isinstance(self.o_proj, QuantLinear):
            return self.o_proj(out, residual=residual)
        return self.o_proj(out) + residual

    def _project_qkv(self, x: Tensor, codes, norm) -> Tensor:
        if codes is not None:
            return self._qkv.forward_codes(codes[0], codes[1], x.dtype).view(*x.shape[:-1], -1)
        return self._qkv(x) if norm is None else self._qkv(x, norm=norm)

    def forward(self, x: Tensor, rotary_emb: Tensor, attn_mask: Optional[Tensor] = None,
                cache=None, codes: Optional[Tuple[Tensor, Tensor]] = None,
                residual: Optional[Tensor] = None, norm=None) -> Tensor:
        """``codes``: the already normalised and quantised input ``(xq [B*S, dim], sx [B*S])`` from a
        fused norm; ``x`` then only gives the shape and dtype.  ``norm = (gain, eps)``: ``x`` is the
        un-normalised stream and the norm runs inside the fused q/k/v projection.  ``residual``:
        added to the output (in o_proj's epilogue when it is quantized)."""
        B, S, _ = x.shape
        if norm is not None and self._qkv is None:
            x, norm = F.rms_norm(x, (x.shape[-1],), norm[0], norm[1]), None
        # The paged decode kernels know two masks: none, and per-sequence lengths (``cache.seq_lens``).  Any
        # mask TENSOR -- padding, or a caller's own -- goes to the stock attention below: the kernels would
        # ignore it.  (A step whose sequences all sit at the same position needs no mask tensor at all; for
        # different positions the caller binds ``seq_lens`` instead, as ``AutoRegressiveLM.forward`` does.)
        if (self._decode_attention and S == 1 and attn_mask is None and isinstance(cache, PagedKV) and x.is_cuda
                and x.dtype == torch.bfloat16):
            qkv = self._project_qkv(x, codes, norm)
            # the output projection combines the attention's position slices itself when the step is small
            # enough for its in-kernel quantiser: one launch less
            split = (isinstance(self.o_proj, QuantLinear) and not self.use_gated_attention
                     and ops.attn_gemv_fusable(B, self.n_heads, self.head_dim, cache.total_len))
            out = ops.rope_paged_attn_decode(qkv.view(B, -1), rotary_emb.reshape(B, -1), cache.page_table,
                                             cache.total_len, cache.k_layers[self.layer_id],
                                             cache.v_layers[self.layer_id], self.n_heads, self.n_kv_heads,
                                             workspace=cache.attn_workspace(self.n_heads), partials=split,
                                             seq_lens=cache.seq_lens, qk_norm=self._qk_norm())
            if split:
                return self.o_proj.forward_attn(out, x.dtype, residual).view(B, 1, -1)
            return self._out(self._gated(out.view(B, 1, -1), x, norm, codes), residual)
        if (self._decode_attention and isinstance(cache, PagedKV) and x.is_cuda and x.dtype == torch.bfloat16
                and S <= cache.total_len):
            # several new tokens (prefill): rotation and the page writes as one launch.  Without a mask tensor the
            # attention is causal by position: a prompt on an empty, fully mapped cache runs the kernel that
            # reads the new keys and values directly (v in place from qkv); a chunk on top of cached tokens,
            # or a table with unmapped pages, the one that reads everything through the page table.  A mask
            # tensor (padding) goes to the stock attention.
            nq, nkv = self.n_heads * self.head_dim, self.n_kv_heads * self.head_dim
            qkv = self._project_qkv(x, codes, norm)
            start = cache.total_len - S
            direct = start == 0 and cache.all_mapped
            kc, vc = cache.k_layers[self.layer_id], cache.v_layers[self.layer_id]
            if attn_mask is None and not direct:
                q = ops.rope_kv_write(qkv, rotary_emb, cache.page_table, start, kc, vc, self.n_heads, self.n_kv_heads,
                                      qk_norm=self._qk_norm())
                out = ops.prefill_attn_paged(q, kc, vc, cache.page_table, start)
                return self._out(self._gated(out.view(B, S, -1), x, norm, codes), residual)
            q, k = ops.rope_kv_write(qkv, rotary_emb, cache.page_table, start, kc, vc, self.n_heads, self.n_kv_heads,
                                     return_k=True, qk_norm=self._qk_norm())
            if direct:
                v = qkv[..., nq + nkv:].view(B, S, self.n_kv_heads, self.head_dim)
                if attn_mask is None:
                    return self._out(self._gated(ops.prefill_attn_causal(q, k, v).view(B, S, -1), x, norm, codes), residual)
            else:
                k, v = cache.gather(self.layer_id)
            out = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), attn_mask,
                                                 enable_gqa=self.n_heads != self.n_kv_heads)
            return self._out(self._gated(out.transpose(1, 2).reshape(B, S, -1), x, norm, codes), residual)
        if self._qkv is not None:
            nq, nkv = self.n_heads * self.head_dim, self.n_kv_heads * self.head_dim
            qkv = self._project_qkv(x, codes, norm)
            q, k, v = qkv.split((nq, nkv, nkv), dim=-1)
        else:
            q, k, v = self.q_proj(x), self.k_proj(x), self.v_proj(x)
        q = q.reshape(B, S, self.n_heads, self.head_dim)
        k = k.reshape(B, S, self.n_kv_heads, self.head_dim)
        v = v.reshape(B, S, self.n_kv_heads, self.head_dim)
        q, k = apply_rotary(q, rotary_emb), apply_rotary(k, rotary_emb)
        if self.use_qk_norm:  # after the rotation, as the reference does (attention.py:86-89)
            q, k = self.q_norm(q), self.k_norm(k)
        if cache is not None:
            cache.write(self.layer_id, k, v)
            k, v = cache.gather(self.layer_id)
        rep = self.n_heads // self.n_kv_heads
        if rep > 1:  # attention.py:15-23
            k = k.repeat_interleave(rep, dim=2)
            v = v.repeat_interleave(rep, dim=2)
        out = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), attn_mask,
                                             is_causal=attn_mask is None)
        return self._out(self._gated(out.transpose(1, 2).reshape(B, S, -1), x, norm, codes), residual)


class MLP(nn.Module):
    """``down(up(x) * silu(gate(x)))`` (astrai/model/components/mlp.py:16-27)."""

    def __init__(self, dim: int, dim_ffn: int):
        super().__init__()
        self.up = Linear(dim, dim_ffn)
        self.gate = Linear(dim, dim_ffn)
        self.down = Linear(dim_ffn, dim)
        self._upgate: Optional[QuantLinear] = None
        self._swiglu_quant = False  # set by DecoderBlock.fuse_norm_quant(): not bit-identical, opt-in

    def fuse_projections(self) -> bool:
        """up and gate read the same input (mlp.py:25): one ``[2*dim_ffn, dim]`` projection."""
        if self._upgate is None and isinstance(self.up, QuantLinear) and isinstance(self.gate, QuantLinear):
            object.__setattr__(self, "_upgate", QuantLinear.concat([self.up, self.gate]))
            return True
        return False

    def forward(self, x: Tensor, codes: Optional[Tuple[Tensor, Tensor]] = None,
                residual: Optional[Tensor] = None, norm=None) -> Tensor:
        """``codes`` / ``norm``: as for the attention block (the input of up and gate)."""
        if norm is not None and self._upgate is None:
            x, norm = F.rms_norm(x, (x.shape[-1],), norm[0], norm[1]), None
        if residual is not None and not isinstance(self.down, QuantLinear):
            return self.forward(x, codes, norm=norm) + residual
        kw = {} if residual is None else {"residual": residual}
        if self._upgate is not None:
            if (self._swiglu_quant and codes is None and isinstance(self.down, QuantLinear)
                    and ops.gemv_swiglu_ok(x, self._upgate.qweight.shape[0] // 2)):
                # decode step: up, gate and the activation in one launch (the [M, 2F] projections are never
                # written), then `down`, which quantises the few rows of h itself
                ug = self._upgate
                h = ops.gemv_w8a8_decode_swiglu(x, ug.qweight, ug.w_scale, ug.bias, out_dtype=x.dtype, norm=norm)
                return self.down(h.view(*x.shape[:-1], -1), **kw)
            if codes is not None:
                ug = self._upgate.forward_codes(codes[0], codes[1], x.dtype).view(*x.shape[:-1], -1)
            else:
                ug = self._upgate(x) if norm is None else self._upgate(x, norm=norm)
            if (self._swiglu_quant and isinstance(self.down, QuantLinear) and ug.is_cuda
                    and ug.shape[-1] // 2 <= ops.SWIGLU_QUANT_MAX_F.get(ug.dtype, 0)):
                # activation, product and the down projection's quantisation in one launch
                hq, hs = ops.swiglu_quant_rowwise_i8(ug)
                return self.down.forward_codes(hq, hs, x.dtype, **kw).view(*x.shape[:-1], -1)
            up, gate = ug.chunk(2, dim=-1)
            return self.down(up * F.silu(gate), **kw)
        return self.down(self.up(x) * F.silu(self.gate(x)), **kw)


class DecoderBlock(nn.Module):
    """``x += attn(norm(x)); x += mlp(norm(x))`` (astrai/model/components/decoder_block.py:12-59)."""

    def __init__(self, dim: int, n_heads: int, dim_ffn: int, n_kv_heads: int, norm_eps: float = 1e-5,
                 layer_id: int = 0, use_qk_norm: bool = False, use_gated_attention: bool = False):
        super().__init__()
        self.attention = GQA(dim, n_heads, n_kv_heads, layer_id, use_qk_norm, norm_eps, use_gated_attention)
        self.input_norm = RMSNorm(dim, norm_eps)
        self.post_attention_norm = RMSNorm(dim, norm_eps)
        self.mlp = MLP(dim, dim_ffn)
        self._norm_quant = False
        self._residual_adds = False

    def reset_parameters(self) -> None:
        for m in self.modules():
            if isinstance(m, Linear):
                m.reset_parameters()

    def fuse_norm_quant(self) -> bool:
        """Both norms feed fused quantized projections only (q/k/v, up/gate): compute norm and
        per-token quantisation in one launch and never write the normalised activations.  The
        bf16 rounding of the norm output disappears, so outputs move by less than the
        quantisation noise (not bit-identical to the unfused block)."""
        if self.attention._qkv is not None and self.mlp._upgate is not None:
            self._norm_quant = True
            self.mlp._swiglu_quant = True  # likewise: silu * up and the quantisation for `down` in one launch
        return self._norm_quant

    def fuse_residual_adds(self) -> bool:
        """Hand the residual stream to o_proj and down, which add it in their epilogue when they
        are quantized (bit-identical to the separate add, one pass over the activations less)."""
        self._residual_adds = True
        return True

    def forward(self, x: Tensor, rotary_emb: Tensor, attention_mask: Optional[Tensor] = None,
                cache=None) -> Tensor:
        if self._residual_adds:  # each branch's last projection adds the stream it is given
            kw = lambda r: {"residual": r}
            add = lambda y, r: y
        else:
            kw = lambda r: {}
            add = lambda y, r: y + r
        if (self._norm_quant and x.is_cuda and x.dtype == self.input_norm.weight.dtype
                and x.shape[-1] <= ops.RMSNORM_QUANT_MAX_K.get(x.dtype, 0)):
            n1, n2 = self.input_norm, self.post_attention_norm
            x = add(self.attention(x, rotary_emb, attention_mask, cache, norm=(n1.weight, n1.norm_eps), **kw(x)), x)
            return add(self.mlp(x, norm=(n2.weight, n2.norm_eps), **kw(x)), x)
        x = add(self.attention(self.input_norm(x), rotary_emb, attention_mask, cache, **kw(x)), x)
        return add(self.mlp(self.post_attention_norm(x), **kw(x)), x)


def decode_mask(batch: int, total_len: int, device, dtype) -> Tensor:
    """Additive mask ``[B, 1, 1, T]`` of a single new token attending to everything cached
    (what astrai/model/transformer.py:17-46 builds for a decode step without padding)."""
    return torch.zeros((batch, 1, 1, total_len), device=device, dtype=dtype)
