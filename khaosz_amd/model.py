"""The whole decoder-only model around the blocks, restated so that the quantized
path can be measured end to end the way the reference measures itself
(scripts/tools/benchmark.py:21-249 on astrai/model/transformer.py:50-151):
token embedding, ``n_layers`` pre-norm blocks sharing one rotary table and one
paged KV cache, a final RMSNorm and the vocabulary projection.

Only what the benchmark's configurations use is here (grouped-query attention
with its qk-norm and output-gate options, SwiGLU MLP, optional tied embedding;
no MoE / MLA).  The attention mask follows ``process_attention_mask``
(transformer.py:17-46) for the two cases the benchmark runs -- a prompt from
position 0 (causal, no mask tensor) and one new token per sequence (a mask of
zeros) -- without its device-to-host reads, so a step can be captured in a HIP
graph.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor

from .block import DecoderBlock, PagedKV, RMSNorm, rotary_table
from .linear import Linear


@dataclass
class LMConfig:
    """The fields of ``AutoRegressiveLMConfig`` (astrai/config/model_config.py:41-60) this model reads."""

    vocab_size: int = 10000
    dim: int = 1536
    n_layers: int = 24
    n_heads: int = 24
    n_kv_heads: int = 4
    dim_ffn: int = 6912
    max_len: int = 2048
    norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    tie_weight: bool = False
    use_qk_norm: bool = False
    use_gated_attention: bool = False


class Embedding(nn.Module):
    """``F.embedding`` over a learned table (astrai/model/components/embedding.py:7-17)."""

    def __init__(self, vocab_size: int, dim: int):
        super().__init__()
        self.weight = nn.Parameter(torch.empty((vocab_size, dim)))

    def reset_parameters(self) -> None:
        nn.init.normal_(self.weight, mean=0.0, std=0.02)

    def forward(self, ids: Tensor) -> Tensor:
        return F.embedding(ids, self.weight)


class AutoRegressiveLM(nn.Module):
    """Same attribute names and state-dict keys as the reference model
    (``embed_tokens``, ``layers.N.*``, ``norm``, ``lm_head``), so ``quantize_model`` and
    ``fuse_shared_inputs`` find their targets and a reference checkpoint's keys line up."""

    def __init__(self, config: LMConfig):
        super().__init__()
        self.config = config
        head_dim = config.dim // config.n_heads
        # complex64 [max_len, head_dim / 2]; a plain attribute, not a buffer: ``model.to(bfloat16)`` must not
        # round it (the reference's buffer is rounded by that cast, rope.py:57-60,70 -- not repeated here)
        self._freqs = rotary_table(head_dim, config.max_len, config.rope_theta)
        self.embed_tokens = Embedding(config.vocab_size, config.dim)
        self.layers = nn.ModuleList([
            DecoderBlock(config.dim, config.n_heads, config.dim_ffn, config.n_kv_heads, config.norm_eps, layer_id=i,
                         use_qk_norm=config.use_qk_norm, use_gated_attention=config.use_gated_attention)
            for i in range(config.n_layers)])
        self.norm = RMSNorm(config.dim, config.norm_eps)
        self.lm_head = Linear(config.dim, config.vocab_size)
        if config.tie_weight:
            self.lm_head.weight = self.embed_tokens.weight
        for m in self.modules():
            if m is not self and hasattr(m, "reset_parameters") and isinstance(m, (Linear, Embedding)):
                m.reset_parameters()

    def new_cache(self, n_pages: int, page_size: int, device=None, dtype=None) -> PagedKV:
        """A paged KV cache with one set of pages per layer (``KVCache``'s storage, cache.py:187-214)."""
        c = self.config
        p = self.embed_tokens.weight
        return PagedKV(n_pages, page_size, c.n_kv_heads, c.dim // c.n_heads, device or p.device, dtype or p.dtype,
                       n_layers=c.n_layers)

    def forward(self, input_ids: Tensor, input_mask: Optional[Tensor] = None, paged_cache: Optional[PagedKV] = None,
                position_ids: Optional[Tensor] = None, start_pos: Optional[int] = None) -> Dict[str, Tensor]:
        """``start_pos``: position of the first input token when every sequence is at the same one
        (what the benchmark runs); it replaces ``position_ids`` and keeps the step free of
        device-to-host reads.  With ``position_ids`` given instead, the mask is built as the
        reference builds it."""
        if input_ids.dim() != 2:
            raise ValueError("input_ids must be [B, S]")
        B, S = input_ids.shape
        x = self.embed_tokens(input_ids)
        if self._freqs.device != x.device:
            self._freqs = self._freqs.to(x.device)
        if start_pos is None and position_ids is None:
            start_pos = 0
        if start_pos is not None:
            if start_pos + S > self._freqs.shape[0]:
                raise ValueError(f"positions up to {start_pos + S} exceed max_len {self._freqs.shape[0]}")
            rotary = self._freqs[start_pos:start_pos + S].unsqueeze(0).expand(B, -1, -1)
            if input_mask is not None:
                raise ValueError("padding masks need position_ids")
            # a prompt from position 0 is causal without a mask tensor; later tokens attend to all
            # cached positions and causally among themselves
            mask = None
            # with the paged-cache kernels in every layer neither a single-token step nor a chunk on top of
            # cached tokens takes a mask tensor: causality is by position inside the kernels
            fused_step = (isinstance(paged_cache, PagedKV) and x.is_cuda and x.dtype == torch.bfloat16
                          and all(getattr(layer.attention, "_decode_attention", False) for layer in self.layers))
            if start_pos > 0 and not fused_step:
                T = start_pos + S
                mask = torch.zeros((B, 1, S, T), device=x.device, dtype=x.dtype)
                if S > 1:
                    mask[:, :, :, start_pos:] = torch.full((S, S), -torch.finfo(x.dtype).max / 2, device=x.device,
                                                           dtype=x.dtype).triu(1)
        else:
            rotary = self._freqs[position_ids]
            fused_step = (S == 1 and input_mask is None and isinstance(paged_cache, PagedKV) and x.is_cuda
                          and x.dtype == torch.bfloat16
                          and all(getattr(layer.attention, "_decode_attention", False) for layer in self.layers))
            if fused_step:
                # a decode step of sequences at possibly different positions (executor.py:59-94): the reference's
                # mask lets sequence b attend to positions <= position_ids[b]; the paged kernels take that as
                # per-sequence lengths, without a mask tensor and without reading the positions back to the host
                mask = None
                paged_cache.seq_lens = (position_ids[:, 0] + 1).to(torch.int64).contiguous()
            else:
                mask = _attention_mask(x, position_ids, input_mask)
        if start_pos is not None and isinstance(paged_cache, PagedKV):
            paged_cache.seq_lens = None  # lengths of an earlier mixed-position step do not apply to this call
        try:
            for layer in self.layers:
                x = layer(x, rotary, mask, paged_cache)
        finally:
            # the per-sequence lengths belong to this step only: a later call on the same cache object (a block or
            # an attention module used directly, another forward) must not find them
            if isinstance(paged_cache, PagedKV):
                paged_cache.seq_lens = None
        hidden = self.norm(x)
        return {"logits": self.lm_head(hidden), "hidden_states": hidden}


def _attention_mask(x: Tensor, position_ids: Tensor, input_mask: Optional[Tensor]) -> Optional[Tensor]:
    """``process_attention_mask(..., is_causal=True)`` (transformer.py:17-46), reads of the device included."""
    if input_mask is not None and input_mask.dim() > 2:
        return input_mask
    B, S = x.shape[:2]
    T = int(position_ids.max().item()) + 1
    if input_mask is None:
        if int(position_ids.min().item()) == 0:
            return None
        pad = torch.ones(B, T, dtype=torch.bool, device=x.device)
    else:
        pad = input_mask[:, :T].to(device=x.device, dtype=torch.bool)
    attend = pad.view(B, 1, T).expand(B, S, T).clone()
    attend &= position_ids.unsqueeze(-1) >= torch.arange(T, device=x.device)
    return torch.full((B, 1, S, T), -torch.finfo(x.dtype).max / 2, dtype=x.dtype,
                      device=x.device).masked_fill_(attend.unsqueeze(1), 0.0)
