"""Host-side mirror of the reference's Linear module and its quantized drop-ins.

``Linear`` keeps the reference's surface (astrai/model/components/linear.py:7-21):
``Linear(in_dim, out_dim, bias=False)``, a ``weight [out_dim, in_dim]`` parameter,
``bias [out_dim]`` or ``None``, ``forward(x[..., in_dim]) -> [..., out_dim]``.

``QuantLinear`` and ``Fp8Linear`` subclass it, so ``isinstance(m, Linear)`` -- the
test the reference uses to discover layers (astrai/model/components/lora.py:64,87)
-- still holds, and they are swapped in with ``setattr(parent, child, new)`` the
way ``inject_lora`` does (lora.py:74-106).  Their forward runs entirely in the HIP
library; there is no CPU or eager fallback.
"""
from __future__ import annotations

import logging
import math
from typing import Iterable, Optional, Sequence, Set, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor

from . import ops

logger = logging.getLogger(__name__)


class Linear(nn.Module):
    """Float Linear with the reference's constructor, attributes and forward."""

    def __init__(self, in_dim: int, out_dim: int, bias: bool = False):
        super().__init__()
        self.weight = nn.Parameter(torch.empty((out_dim, in_dim)))
        self.bias = nn.Parameter(torch.zeros(out_dim)) if bias else None

    @property
    def in_dim(self) -> int:
        return self.weight.shape[1]

    @property
    def out_dim(self) -> int:
        return self.weight.shape[0]

    def reset_parameters(self) -> None:
        # same distributions as linear.py:13-18: U(-1/sqrt(in), 1/sqrt(in)) for both
        bound = 1.0 / math.sqrt(self.weight.shape[1])
        nn.init.kaiming_uniform_(self.weight, a=math.sqrt(5))
        if self.bias is not None:
            nn.init.uniform_(self.bias, -bound, bound)

    def forward(self, x: Tensor) -> Tensor:
        return F.linear(x, self.weight, self.bias)


class _PerStream:
    """Scratch tensors a module keeps per (device, stream): the decode workspace, the one-launch quantiser's state.
    Bounded: the most recently used ``keep`` streams stay, older entries are dropped (a module called from ever
    new side or capture streams would otherwise grow by a workspace per stream for the life of the model).
    Keys are raw stream handles, which the runtime may hand out again for a new stream: harmless for a stateless
    workspace, and for the quantiser's state too, because what it needs is only that calls sharing it do not
    overlap in time -- which launches on one stream never do -- and every call leaves it in the state the next
    one accepts."""

    def __init__(self, keep: int = 8):
        self._keep, self._items = keep, {}

    def get(self, device, make, fits=lambda t: True):
        key = (device, torch.cuda.current_stream(device).cuda_stream)
        t = self._items.pop(key, None)
        if t is None or not fits(t):
            t = make()
        self._items[key] = t  # most recently used last
        while len(self._items) > self._keep:
            self._items.pop(next(iter(self._items)))
        return t

    def __len__(self):
        return len(self._items)


def _no_grad_guard(x: Tensor) -> None:
    if torch.is_grad_enabled() and x.requires_grad:
        raise RuntimeError("the quantized Linear is forward-only; call it under torch.no_grad()/inference_mode()")


class _SharedInput:
    """Sibling projections that a module's forward applies to ONE input tensor, run as one concatenated
    projection (``QuantLinear.concat``: one activation quantisation, one launch, bit-identical columns)
    without touching that forward: the first sibling called with a tensor computes all columns, every
    sibling returns its column slice.  The input is recognised by identity (and, where torch tracks one,
    by its version counter), and both it and the result are dropped as soon as every sibling has taken
    its slice, so nothing outlives the forward that used it.  Not for concurrent calls of one module from
    several threads.  For modules whose forward is known to hand
    the same, unmodified tensor to all siblings (the reference's GQA, MLA and MLP: attention.py:83-85,
    105-106, 166-170, 205-206; mlp.py:25)."""

    def __init__(self, fused: "QuantLinear", bounds: Sequence[Tuple[int, int]]):
        self.fused, self.bounds = fused, list(bounds)
        self._x = self._y = None
        self._version = None
        self._served: set = set()

    @staticmethod
    def _version_of(x: Tensor):
        try:
            return x._version
        except RuntimeError:  # inference tensors carry no version counter
            return None

    def output(self, x: Tensor, index: int) -> Tensor:
        if self._x is not x or self._version != self._version_of(x) or index in self._served:
            self._y = self.fused(x)
            self._x, self._version, self._served = x, self._version_of(x), set()
        lo, hi = self.bounds[index]
        y = self._y[..., lo:hi]
        self._served.add(index)
        if len(self._served) == len(self.bounds):
            self._x = self._y = None
            self._served = set()
        return y


class QuantLinear(Linear):
    """W8A8 Linear: per-channel int8 weight, per-token int8 activation.

    Buffers: ``qweight int8 [out, in]``, ``w_scale float32 [out]``; ``bias`` stays a
    parameter (or None).  ``weight`` reads back the dequantized float weight for
    callers that inspect it (lora.py:34-38, transformer.py:95-96).  A float
    ``<prefix>weight`` entry in a state dict is quantized on load, so float
    checkpoints with the reference's key names (tests/module/test_lora.py:201-208)
    still load.
    """

    DECODE_MAX_ROWS = 16

    def __init__(self, in_dim: int, out_dim: int, bias: bool = False, device=None):
        nn.Module.__init__(self)
        self.register_buffer("qweight", torch.zeros((out_dim, in_dim), dtype=torch.int8, device=device))
        self.register_buffer("w_scale", torch.ones((out_dim,), dtype=torch.float32, device=device))
        self.bias = nn.Parameter(torch.zeros(out_dim, device=device), requires_grad=False) if bias else None
        # decode workspaces (activation codes between the row quantiser and the GEMV), one per (device, stream):
        # the same module called from two streams or threads must not share one
        self._workspaces = _PerStream()
        self._shared: Optional[Tuple[_SharedInput, int]] = None  # set by share_inputs(): (group, index in it)

    # -- construction -----------------------------------------------------
    @classmethod
    def from_linear(cls, base: nn.Module) -> "QuantLinear":
        """Quantize ``base.weight`` per output channel on the GPU it lives on."""
        w = base.weight.detach()
        if not w.is_cuda:
            raise RuntimeError("QuantLinear.from_linear needs the weight on the GPU (the quantizer is a HIP kernel)")
        out_dim, in_dim = w.shape
        q = cls(in_dim, out_dim, bias=base.bias is not None, device=w.device)
        q.load_float_weight(w)
        if base.bias is not None:
            q.bias = nn.Parameter(base.bias.detach().clone(), requires_grad=False)
        return q

    @classmethod
    def concat(cls, parts: Sequence["QuantLinear"]) -> "QuantLinear":
        """One module computing ``cat([p(x) for p in parts], -1)`` for projections that read the
        same input (q/k/v: attention.py:83-85; up/gate: mlp.py:25): the activation is quantised
        once and the weights are streamed by one launch.  Per-channel weight scales and per-token
        activation scales make every output element the same arithmetic as in its own module, so
        the result is bit-identical.  Afterwards the parts' ``qweight`` / ``w_scale`` (and bias)
        are row slices of the fused buffers: no second copy of the weights is kept."""
        parts = list(parts)
        if not parts or any(not isinstance(p, QuantLinear) for p in parts):
            raise ValueError("concat needs QuantLinear modules")
        if len({p.in_dim for p in parts}) != 1 or len({p.bias is None for p in parts}) != 1:
            raise ValueError("parts must share in_dim and all have, or all lack, a bias")
        dev = parts[0].qweight.device
        fused = cls(parts[0].in_dim, sum(p.out_dim for p in parts), bias=parts[0].bias is not None, device=dev)
        fused.qweight = torch.cat([p.qweight for p in parts], dim=0)
        fused.w_scale = torch.cat([p.w_scale for p in parts], dim=0)
        if fused.bias is not None:
            fused.bias = nn.Parameter(torch.cat([p.bias.detach() for p in parts], dim=0), requires_grad=False)
        row = 0
        for p in parts:
            n = p.out_dim
            p.qweight = fused.qweight[row:row + n]
            p.w_scale = fused.w_scale[row:row + n]
            if p.bias is not None:
                p.bias = nn.Parameter(fused.bias.detach()[row:row + n], requires_grad=False)
            row += n
        return fused

    def load_float_weight(self, w: Tensor) -> None:
        if tuple(w.shape) != tuple(self.qweight.shape):
            raise ValueError(f"weight shape {tuple(w.shape)} does not match {tuple(self.qweight.shape)}")
        if w.dtype not in (torch.float32, torch.bfloat16):
            w = w.float()
        codes, scale = ops.quant_rowwise_i8(w.to(self.qweight.device))
        self.qweight.copy_(codes)
        self.w_scale.copy_(scale)

    # -- the reference's attribute surface ----------------------------------
    @property
    def weight(self) -> Tensor:
        return self.qweight.float() * self.w_scale[:, None]

    @property
    def in_dim(self) -> int:
        return self.qweight.shape[1]

    @property
    def out_dim(self) -> int:
        return self.qweight.shape[0]

    def reset_parameters(self) -> None:
        raise RuntimeError("QuantLinear holds quantized weights; initialise a float Linear and convert it")

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                              error_msgs):
        key = prefix + "weight"
        if key in state_dict and (prefix + "qweight") not in state_dict:
            w = state_dict.pop(key)
            try:
                self.load_float_weight(w)
            except (ValueError, RuntimeError) as e:
                error_msgs.append(f"{key}: {e}")
            state_dict[prefix + "qweight"] = self.qweight
            state_dict[prefix + "w_scale"] = self.w_scale
        super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                                      error_msgs)

    # -- forward ----------------------------------------------------------------
    def forward(self, x: Tensor, residual: Optional[Tensor] = None, norm=None) -> Tensor:
        """``residual`` (shape and dtype of the output): returns ``linear(x) + residual`` with the add
        done in the kernel's epilogue, bit-identical to adding the two tensors afterwards.
        ``norm = (gain [in_dim], eps)``: returns ``linear(rms_norm(x) * gain)`` with the norm fused
        into the activation quantisation (the normalised activations are never written; see
        ``ops.rmsnorm_quant_rowwise_i8``)."""
        _no_grad_guard(x)
        if self._shared is not None and residual is None and norm is None:
            return self._shared[0].output(x, self._shared[1])
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1])
        M = x2.shape[0]
        if x2.shape[1] != self.qweight.shape[1]:
            raise ValueError(f"expected last dim {self.qweight.shape[1]}, got {x2.shape[1]}")
        if x2.dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"activation dtype {x2.dtype} is not supported (float32 or bfloat16)")
        if M <= self.DECODE_MAX_ROWS:
            ops._need_gpu(x, self.qweight)
            need = 16 * self.qweight.shape[1] + 512
            ws = self._workspaces.get(x.device, lambda: torch.empty((need,), dtype=torch.uint8, device=x.device),
                                      lambda t: t.numel() >= need)
            y = ops.gemv_w8a8_decode(x2, self.qweight, self.w_scale, self.bias, out_dtype=x.dtype, workspace=ws,
                                     residual=residual, norm=norm)
        else:
            xq, sx = ops.quant_rowwise_i8(x2) if norm is None else ops.rmsnorm_quant_rowwise_i8(x2, norm[0], norm[1])
            y = ops.linear_w8a8(xq, sx, self.qweight, self.w_scale, self.bias, out_dtype=x.dtype, residual=residual)
        return y.reshape(*lead, self.qweight.shape[0])

    def forward_codes(self, xq: Tensor, sx: Tensor, out_dtype: torch.dtype,
                      residual: Optional[Tensor] = None) -> Tensor:
        """The same projection for an input that is already quantised (``xq int8 [M, K]``,
        ``sx float32 [M]``): what a producer that fuses the quantisation hands over, or what
        several projections of one input share.  Returns ``[M, out_dim]``."""
        if xq.dim() != 2 or xq.shape[1] != self.qweight.shape[1]:
            raise ValueError(f"expected codes [M, {self.qweight.shape[1]}], got {tuple(xq.shape)}")
        if xq.shape[0] <= self.DECODE_MAX_ROWS:
            return ops.gemv_w8a8_codes(xq, sx, self.qweight, self.w_scale, self.bias, out_dtype=out_dtype,
                                       residual=residual)
        return ops.linear_w8a8(xq, sx, self.qweight, self.w_scale, self.bias, out_dtype=out_dtype, residual=residual)

    def forward_attn(self, parts: "ops.AttnPartials", out_dtype: torch.dtype = torch.bfloat16,
                     residual: Optional[Tensor] = None) -> Tensor:
        """The projection applied to a decode step's attention output that is still in slices
        (``ops.rope_paged_attn_decode(..., partials=True)``): combined, quantised and multiplied in
        one launch.  Returns ``[B, out_dim]``, the bits of ``forward`` on the merged output."""
        return ops.gemv_w8a8_attn(parts, self.qweight, self.w_scale, self.bias, out_dtype=out_dtype, residual=residual)

    def extra_repr(self) -> str:
        return f"in_dim={self.in_dim}, out_dim={self.out_dim}, bias={self.bias is not None}, w8a8"


class Fp8Linear(Linear):
    """FP8 (OCP e4m3fn) Linear with per-tensor scales and fp32 accumulation."""

    def __init__(self, in_dim: int, out_dim: int, bias: bool = False, device=None):
        nn.Module.__init__(self)
        self.register_buffer("qweight", torch.zeros((out_dim, in_dim), dtype=torch.uint8, device=device))
        self.register_buffer("w_scale", torch.ones((1,), dtype=torch.float32, device=device))
        self.bias = nn.Parameter(torch.zeros(out_dim, device=device), requires_grad=False) if bias else None
        self._workspaces = _PerStream()    # decode workspaces, one per (device, stream), as in QuantLinear
        self._quant_states = _PerStream()  # the one-launch activation quantiser's state, one per (device, stream)

    DECODE_MAX_ROWS = 16

    @classmethod
    def from_linear(cls, base: nn.Module) -> "Fp8Linear":
        w = base.weight.detach()
        if not w.is_cuda:
            raise RuntimeError("Fp8Linear.from_linear needs the weight on the GPU (the quantizer is a HIP kernel)")
        q = cls(w.shape[1], w.shape[0], bias=base.bias is not None, device=w.device)
        if w.dtype not in (torch.float32, torch.bfloat16):
            w = w.float()
        codes, scale = ops.quant_tensor_fp8(w)
        q.qweight.copy_(codes)
        q.w_scale.copy_(scale)
        if base.bias is not None:
            q.bias = nn.Parameter(base.bias.detach().clone(), requires_grad=False)
        return q

    @property
    def weight(self) -> Tensor:
        return self.qweight.view(torch.float8_e4m3fn).float() * self.w_scale

    @property
    def in_dim(self) -> int:
        return self.qweight.shape[1]

    @property
    def out_dim(self) -> int:
        return self.qweight.shape[0]

    def reset_parameters(self) -> None:
        raise RuntimeError("Fp8Linear holds quantized weights; initialise a float Linear and convert it")

    def forward(self, x: Tensor, residual: Optional[Tensor] = None) -> Tensor:
        """``residual`` (shape and dtype of the output): added in the kernel's epilogue, the bits of a separate add."""
        _no_grad_guard(x)
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1])
        if x2.shape[1] != self.qweight.shape[1]:
            raise ValueError(f"expected last dim {self.qweight.shape[1]}, got {x2.shape[1]}")
        if x2.shape[0] <= self.DECODE_MAX_ROWS:  # decode step: the weight-streaming GEMV
            ops._need_gpu(x, self.qweight)
            need = 16 * self.qweight.shape[1] + 2048
            ws = self._workspaces.get(x.device, lambda: torch.empty((need,), dtype=torch.uint8, device=x.device),
                                      lambda t: t.numel() >= need)
            y = ops.gemv_fp8_decode(x2, self.qweight, self.w_scale, self.bias, out_dtype=x.dtype, workspace=ws,
                                    residual=residual)
        else:
            ops._need_gpu(x, self.qweight)
            state = self._quant_states.get(x.device, lambda: ops.fp8_onepass_state(x.device))
            xq, sx = ops.quant_tensor_fp8(x2, state=state)  # one launch for large inputs
            y = ops.linear_fp8(xq, sx, self.qweight, self.w_scale, self.bias, out_dtype=x.dtype, residual=residual)
        return y.reshape(*lead, self.qweight.shape[0])


# Child names quantized by default: the projections of GQA (attention.py:57-67, `gate` is its optional output
# gate), of MLA (attention.py:140-156: q_proj, kv_a_proj, kv_b_proj, o_proj, gate) and of every MLP, the experts of
# DeepSeekMoE included (mlp.py:20-22,48-55).  Left in floating point unless named explicitly: `lm_head` (it may
# alias the embedding, transformer.py:95-96) and DeepSeekMoE's `router` (mlp.py:48): its few outputs feed a top-k,
# where int8 noise on near-equal logits changes which experts run, for under 0.1 % of a layer's weight bytes.
TARGET_MODULES_ATTN = {"q_proj", "k_proj", "v_proj", "o_proj", "kv_a_proj", "kv_b_proj"}
TARGET_MODULES_FFN = {"up", "gate", "down"}


def share_inputs(parent: nn.Module, names: Sequence[str]) -> bool:
    """Run the quantized children ``names`` of ``parent`` -- projections its forward applies to one and
    the same tensor -- as one concatenated projection behind their own ``forward`` (see ``_SharedInput``);
    ``parent``'s code and state-dict keys stay as they are.  Returns False (and changes nothing) unless at
    least two of the named children exist and all of those are ``QuantLinear`` with one input width and
    alike in having a bias."""
    parts = [getattr(parent, n, None) for n in names]
    parts = [p for p in parts if p is not None]
    if len(parts) < 2 or any(not isinstance(p, QuantLinear) or p._shared is not None for p in parts):
        return False
    if len({p.in_dim for p in parts}) != 1 or len({p.bias is None for p in parts}) != 1:
        return False
    bounds, row = [], 0
    for p in parts:
        bounds.append((row, row + p.out_dim))
        row += p.out_dim
    group = _SharedInput(QuantLinear.concat(parts), bounds)
    for i, p in enumerate(parts):
        p._shared = (group, i)
    return True


# Modules of the reference whose forward hands one tensor to several projections, by class (module path, name)
# -- matched by name so that this package never imports the reference: GQA (attention.py:83-85; the output gate
# reads the same x, attention.py:105-106), MLA (attention.py:166-170, 205-206) and MLP, the experts of DeepSeekMoE
# included (mlp.py:25).
REFERENCE_SHARED_INPUTS = {
    ("astrai.model.components.attention", "GQA"): ("q_proj", "k_proj", "v_proj", "gate"),
    ("astrai.model.components.attention", "MLA"): ("q_proj", "kv_a_proj", "gate"),
    ("astrai.model.components.mlp", "MLP"): ("up", "gate"),
}


def fuse_shared_inputs(model: nn.Module, norms: bool = False, decode_attention: bool = False,
                       residuals: bool = False) -> int:
    """Call ``fuse_projections()`` on every module that offers it (attention and MLP blocks whose
    projections read one input); returns how many fused modules were built.  Run it after
    ``quantize_model`` and after loading weights: the fused module owns the weight storage from
    then on.  Outputs stay bit-identical.  Modules of the reference itself (its GQA, MLA and MLP classes,
    recognised by name) get the same single launch behind their own unchanged forward (``share_inputs``).
    ``norms=True`` additionally lets blocks compute
    RMSNorm and the quantisation of its output in one launch (``fuse_norm_quant()``), which
    drops the bf16 rounding of the normalised activations: not bit-identical, inside the
    quantisation noise.  ``decode_attention=True`` lets attention modules with a fused q/k/v
    projection run single-token steps on a paged cache through the in-place attention kernels
    (``fuse_decode_attention()``).  ``residuals=True`` lets blocks hand the residual stream to the
    quantized projection that ends each branch (``fuse_residual_adds()``): the add happens in that
    kernel's epilogue, bit-identical to the separate add."""
    n = 0
    for m in model.modules():
        f = getattr(m, "fuse_projections", None)
        if callable(f):
            n += int(f())
            continue
        names = REFERENCE_SHARED_INPUTS.get((type(m).__module__, type(m).__name__))
        if names is not None:  # the reference's own module: its forward is untouched
            # (the output gate joins the group only if it matches the others in having a bias)
            n += int(share_inputs(m, names) or share_inputs(m, [x for x in names if x != "gate" or "up" in names]))
    if norms:
        for m in model.modules():
            f = getattr(m, "fuse_norm_quant", None)
            if callable(f):
                f()
    if decode_attention:
        for m in model.modules():
            f = getattr(m, "fuse_decode_attention", None)
            if callable(f):
                f()
    if residuals:
        for m in model.modules():
            f = getattr(m, "fuse_residual_adds", None)
            if callable(f):
                f()
    return n


def _is_float_linear(m: nn.Module, extra: Iterable[type]) -> bool:
    if isinstance(m, (QuantLinear, Fp8Linear)):
        return False
    if isinstance(m, Linear) or isinstance(m, tuple(extra)):
        return True
    # the reference's own class, matched by identity of name and module so that
    # this package never has to import it
    t = type(m)
    return t.__name__ == "Linear" and t.__module__ == "astrai.model.components.linear"


def quantize_model(model: nn.Module, target_modules: Optional[Set[str]] = None, mode: str = "int8",
                   linear_types: Iterable[type] = ()) -> int:
    """Replace float Linear children by quantized ones, in place.

    Walks ``named_modules`` and swaps by ``setattr`` exactly as ``inject_lora``
    does (lora.py:85-94).  ``target_modules`` is a set of child names (default:
    the attention and MLP projections); ``lm_head`` is never in the default set
    because it may alias the embedding (astrai/model/transformer.py:95-96).
    Returns the number of layers replaced.
    """
    if mode not in ("int8", "fp8"):
        raise ValueError(f"mode must be 'int8' or 'fp8', got {mode!r}")
    if target_modules is None:
        target_modules = TARGET_MODULES_ATTN | TARGET_MODULES_FFN
    cls = QuantLinear if mode == "int8" else Fp8Linear
    replaced = 0
    seen = []
    for name, module in list(model.named_modules()):
        if not _is_float_linear(module, linear_types):
            continue
        parent_name, _, child_name = name.rpartition(".")
        seen.append(child_name)
        if child_name not in target_modules:
            continue
        if module.weight.shape[1] % 16:
            # the kernels walk the reduction in 16-byte vectors; such a layer (the reference's dim-8 test
            # models) stays in floating point rather than failing at its first call
            logger.warning("Linear %s left in floating point: in_dim %d is not a multiple of 16", name,
                           module.weight.shape[1])
            continue
        parent = model.get_submodule(parent_name) if parent_name else model
        setattr(parent, child_name, cls.from_linear(module))
        replaced += 1
    if replaced == 0:
        logger.warning("No Linear layers quantized. Available Linear child names: %s; target_modules: %s",
                       sorted(set(seen)), sorted(target_modules))
    else:
        logger.info("Quantized %d Linear layers (%s)", replaced, mode)
    return replaced
