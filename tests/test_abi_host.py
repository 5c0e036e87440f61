"""CPU-side checks: the C-ABI library loads, exports every symbol the header
declares, rejects bad arguments before touching a GPU, and the host module keeps
the reference's Linear surface (astrai/model/components/linear.py:7-21) and swap
invariants (tests/module/test_lora.py in the reference)."""
import os
import re

import pytest
import torch
import torch.nn as nn

import khaosz_amd
from khaosz_amd import _abi, ops
from khaosz_amd.linear import Fp8Linear, Linear, QuantLinear, quantize_model

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "astrai_q.h")).read()
    declared = set(re.findall(r"\b(aq_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_abi.SYMBOLS), declared ^ set(_abi.SYMBOLS)
    lib = _abi.load()
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.aq_version() == 100


def test_lab_library_holds_the_product_and_the_lab_symbols():
    """The probes and the tile-forcing hook live in a second library built from the same objects:
    the product library exports none of them."""
    lab_header = open(os.path.join(ROOT, "khaosz_amd", "csrc", "aq_lab.h")).read()
    declared = set(re.findall(r"\b(aq_lab_[a-z0-9_]+)\s*\(", lab_header))
    assert declared == set(_abi.LAB_SYMBOLS), declared ^ set(_abi.LAB_SYMBOLS)
    lab, lib = _abi.load_lab(), _abi.load()
    for name in declared:
        assert hasattr(lab, name), name
        assert not hasattr(lib, name), f"{name} leaked into the product library"
    for name in _abi.SYMBOLS:
        assert hasattr(lab, name), name
    assert lab.aq_lab_set_gemm_tile(3) == -2 and lab.aq_lab_set_gemm_tile(0) == 0


def test_argument_validation_happens_before_any_launch():
    lib = _abi.load()
    P = 1 << 20  # a 16-byte aligned fake pointer; never dereferenced on these paths
    assert lib.aq_quant_rowwise_i8(P, 0, 4, 17, 17, P, P, None) == -2      # K % 16
    assert lib.aq_quant_rowwise_i8(P, 7, 4, 16, 16, P, P, None) == -3      # dtype
    assert lib.aq_quant_rowwise_i8(None, 0, 4, 16, 16, P, P, None) == -1   # null
    assert lib.aq_quant_rowwise_i8(P + 4, 0, 4, 16, 16, P, P, None) == -4  # alignment
    assert lib.aq_quant_rowwise_i8(P, 0, 4, 32, 16, P, P, None) == -2      # ldx < K
    assert lib.aq_quant_rowwise_i8(P, 0, 0, 16, 16, P, P, None) == 0       # empty is fine
    assert lib.aq_gemm_i8_i32(P, P, P, 4, 4, 24, None) == -2
    assert lib.aq_gemm_i8_i32(P, P, P, 0, 4, 32, None) == 0
    assert lib.aq_gemm_i8_i32(P, None, P, 4, 4, 32, None) == -1
    assert lib.aq_linear_w8a8(P, P, P, P, None, 0, P, 5, 4, 4, 32, None) == -3
    assert lib.aq_linear_w8a8(P, None, P, P, None, 0, P, 1, 4, 4, 32, None) == -1
    assert lib.aq_linear_fp8(P, P, P, P, P, 9, 4, 4, 32, None) == -3
    assert lib.aq_linear_fp8_residual(P, P, P, P, P, 7, None, P, 1, 4, 4, 32, None) == -3       # bias dtype
    assert lib.aq_linear_fp8_residual(P, P, P, P, None, 0, P + 2, P, 1, 4, 4, 32, None) == -4   # residual alignment
    assert lib.aq_gemv_w8a8_decode(P, 1, P, P, None, 0, P, 1, 17, 8, 32, P, 1 << 20, None) == -2  # M > 16
    assert lib.aq_gemv_w8a8_decode(P, 1, P, P, None, 0, P, 1, 4, 8, 32, P, 8, None) == -5         # workspace
    assert lib.aq_gemv_w8a8_decode(P, 1, P, P, None, 0, P + 2, 1, 4, 8, 32, P, 1 << 20, None) == -4  # y alignment
    assert lib.aq_gemv_w8a8_codes(P, P, P, P + 1, None, 0, P, 1, 4, 8, 32, None) == -4            # scale alignment
    assert lib.aq_linear_w8a8(P, P, P, P, None, 0, P, 1, 4, 1 << 21, 32, None) == -6              # N beyond the epilogue's offsets
    assert lib.aq_gemv_w8a8_workspace_bytes(16, 2048) >= 16 * 2048 + 64
    assert b"multiple of 16" in lib.aq_error_string(-2)
    with pytest.raises(ValueError):
        _abi.check(-2, "x")
    with pytest.raises(RuntimeError):
        _abi.check(-1, "x")


def test_ops_refuse_cpu_tensors_loudly():
    x = torch.randn(4, 32)
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.quant_rowwise_i8(x)
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.gemm_i8_i32(torch.zeros(4, 32, dtype=torch.int8), torch.zeros(4, 32, dtype=torch.int8))
    ql = QuantLinear(32, 16)
    with pytest.raises(RuntimeError, match="GPU only"):
        ql(x)
    lin = Linear(32, 16)
    lin.reset_parameters()
    with pytest.raises(RuntimeError, match="GPU"):
        QuantLinear.from_linear(lin)


def test_linear_keeps_the_reference_surface():
    torch.manual_seed(0)
    lin = Linear(24, 8)
    assert lin.bias is None and tuple(lin.weight.shape) == (8, 24)
    lin.reset_parameters()
    assert lin.weight.abs().max() <= 1 / 24 ** 0.5 + 1e-6
    x = torch.randn(2, 5, 24)
    assert torch.equal(lin(x), torch.nn.functional.linear(x, lin.weight))
    lb = Linear(24, 8, bias=True)
    lb.reset_parameters()
    assert set(lb.state_dict()) == {"weight", "bias"}
    assert torch.allclose(lb(x), x @ lb.weight.T + lb.bias, atol=1e-6)


def test_quant_linear_is_a_linear_with_quantized_state():
    q = QuantLinear(32, 16, bias=True)
    assert isinstance(q, Linear) and isinstance(q, nn.Module)
    assert set(q.state_dict()) == {"qweight", "w_scale", "bias"}
    assert q.qweight.dtype == torch.int8 and q.w_scale.dtype == torch.float32
    q.qweight.fill_(3)
    q.w_scale.fill_(0.5)
    assert torch.equal(q.weight, torch.full((16, 32), 1.5))
    assert q.in_dim == 32 and q.out_dim == 16
    f = Fp8Linear(32, 16)
    assert isinstance(f, Linear) and set(f.state_dict()) == {"qweight", "w_scale"}
    fb = Fp8Linear(32, 16, bias=True)
    assert set(fb.state_dict()) == {"qweight", "w_scale", "bias"} and tuple(fb.bias.shape) == (16,)
    with pytest.raises(RuntimeError):
        q.reset_parameters()


class _Block(nn.Module):
    def __init__(self):
        super().__init__()
        self.q_proj = Linear(32, 32)
        self.up = Linear(32, 64)
        self.lm_head = Linear(32, 100)
        self.other = nn.Linear(32, 32)


def test_quantize_model_walks_like_inject_lora_and_skips_untargeted(monkeypatch):
    # from_linear needs a GPU; stand in a recorder so the walk itself is tested on CPU
    made = []

    def fake(cls, base):
        made.append(base)
        return QuantLinear(base.weight.shape[1], base.weight.shape[0], bias=base.bias is not None)

    monkeypatch.setattr(QuantLinear, "from_linear", classmethod(fake))
    m = nn.Sequential(_Block(), _Block())
    n = quantize_model(m)
    assert n == 4 and len(made) == 4
    assert isinstance(m[0].q_proj, QuantLinear) and isinstance(m[1].up, QuantLinear)
    assert type(m[0].lm_head) is Linear and type(m[0].other) is nn.Linear
    keys = set(m.state_dict())
    assert "0.q_proj.qweight" in keys and "0.q_proj.w_scale" in keys and "0.lm_head.weight" in keys
    assert quantize_model(m) == 0  # idempotent: quantized layers are not float Linears
    with pytest.raises(ValueError):
        quantize_model(m, mode="int4")


def _reference_linear_class():
    """A class that looks, to code that never imports the reference, exactly like the reference's
    own Linear (astrai/model/components/linear.py:7-21): same name, same module path, same attributes
    and forward -- and no relation to this package's Linear."""

    class RefLinear(nn.Module):
        def __init__(self, in_dim, out_dim, bias=False):
            super().__init__()
            self.weight = nn.Parameter(torch.randn(out_dim, in_dim) * 0.05)
            self.bias = nn.Parameter(torch.zeros(out_dim)) if bias else None

        def forward(self, x):
            return nn.functional.linear(x, self.weight, self.bias)

    RefLinear.__name__ = RefLinear.__qualname__ = "Linear"
    RefLinear.__module__ = "astrai.model.components.linear"
    return RefLinear


def test_the_reference_class_is_recognised_by_name_without_importing_it(monkeypatch):
    from khaosz_amd.linear import _is_float_linear

    Ref = _reference_linear_class()
    assert not issubclass(Ref, Linear)
    assert _is_float_linear(Ref(16, 8), ())
    # the same class under another module path, or another name, is somebody else's layer
    Other = _reference_linear_class()
    Other.__module__ = "somewhere.else"
    assert not _is_float_linear(Other(16, 8), ())
    assert _is_float_linear(Other(16, 8), (Other,))  # unless the caller names its type
    Renamed = _reference_linear_class()
    Renamed.__name__ = "Dense"
    assert not _is_float_linear(Renamed(16, 8), ())
    assert not _is_float_linear(nn.Linear(16, 8), ())

    made = []

    def fake(cls, base):
        made.append(base)
        return QuantLinear(base.weight.shape[1], base.weight.shape[0], bias=base.bias is not None)

    monkeypatch.setattr(QuantLinear, "from_linear", classmethod(fake))

    class MLABlock(nn.Module):  # child names of the reference's MLA and DeepSeekMoE (attention.py:140-156, mlp.py:48-55)
        def __init__(self):
            super().__init__()
            self.q_proj, self.kv_a_proj, self.kv_b_proj, self.o_proj = Ref(32, 48), Ref(32, 16), Ref(16, 96), Ref(32, 32)
            self.router = Ref(32, 8)
            self.routed_experts = nn.ModuleList([_RefMLP(Ref) for _ in range(2)])

    class _Holder(nn.Module):
        def __init__(self):
            super().__init__()
            self.attn = MLABlock()
            self.up = Ref(8, 32)   # the reference's dim-8 test models: in_dim not a multiple of 16

    m = _Holder()
    n = quantize_model(m)
    # q/kv_a/kv_b/o + 2 experts x (up, gate, down); router stays float by default, `up` with in_dim 8 is skipped
    assert n == 4 + 6 and len(made) == n
    assert type(m.attn.router) is Ref and type(m.up) is Ref
    assert isinstance(m.attn.kv_a_proj, QuantLinear) and isinstance(m.attn.routed_experts[1].down, QuantLinear)
    assert quantize_model(m, target_modules={"router"}) == 1 and isinstance(m.attn.router, QuantLinear)


class _RefMLP(nn.Module):
    def __init__(self, L):
        super().__init__()
        self.up, self.gate, self.down = L(32, 64), L(32, 64), L(64, 32)


def test_package_exports():
    assert {"Linear", "QuantLinear", "Fp8Linear", "quantize_model"} <= set(dir(khaosz_amd))


def test_gemm_tile_choice_for_the_benchmark_shapes_and_a_few_hundred_rows():
    """The tile shape is picked on the host from M, N and the number of compute units alone.  Pinned here for
    256 compute units: the benchmark configurations keep the wide tiles (one round of 256 tiles of 256 x 128
    for the prefill configuration, 256 tiles of 128 x 128 for the FP8 one), a few hundred rows get the small
    tiles that still give every compute unit at most one tile, and a launch of many rounds never takes a small
    tile."""
    lab = _abi.load_lab()
    pick = lambda M, N: lab.aq_lab_choose_gemm_tile(M, N, 256)
    assert pick(4096, 2048) == 256          # configuration 3: 256 tiles of 256 x 128, one round
    assert pick(2048, 2048) == 128          # configuration 4: 256 tiles of 128 x 128
    assert pick(8192, 8192) == 256
    assert pick(4096, 3072) == 256 and pick(4096, 11264) == 256   # block prefill: q/k/v, up/gate
    assert pick(2048, 13824) == 256         # model prefill, up/gate
    assert pick(64, 8192) == 33 and pick(48, 2048) == 33          # 64 x 32: 256 and 64 tiles
    assert pick(128, 8192) == 65            # 64 x 64: 256 tiles (64 x 32 would need two rounds)
    assert pick(256, 8192) == 64            # 128 x 64
    assert pick(128, 11264) == 64 and pick(64, 11264) == 65
    assert pick(384, 8192) == 128 and pick(512, 8192) == 128
    assert pick(768, 8192) == 256 and pick(1024, 8192) == 256
    assert pick(512, 2048) == 65 and pick(1024, 2048) == 64 and pick(256, 2048) == 33
    for M, N in ((8192, 8192), (100000, 4096), (1 << 20, 1 << 20)):
        assert pick(M, N) in (128, 256)
    assert lab.aq_lab_choose_gemm_tile(0, 8, 256) == -2 and lab.aq_lab_choose_gemm_tile(8, 8, 0) == -2


def test_quant_tensor_fp8_refuses_a_workspace_smaller_than_its_slots():
    """aq_quant_tensor_fp8 writes AQ_FP8_AMAX_WS_BYTES of partial maxima: a smaller workspace is refused before
    anything is launched (argument checks only: runs without a GPU)."""
    lib = _abi.load()
    dummy = 4096  # never dereferenced: the size check comes first
    assert lib.aq_quant_tensor_fp8(dummy, 1, 64, dummy, dummy, dummy, 4, None) == -5
    assert lib.aq_quant_tensor_fp8(dummy, 1, 64, dummy, dummy, dummy, _abi.AQ_FP8_AMAX_WS_BYTES - 1, None) == -5
    assert b"workspace" in lib.aq_error_string(-5).lower()
