"""MI355X-native quantized-Linear path behind the reference's Linear module."""
from .linear import Fp8Linear, Linear, QuantLinear, fuse_shared_inputs, quantize_model, share_inputs  # noqa: F401
from .model import AutoRegressiveLM, LMConfig  # noqa: F401

__version__ = "0.1.0"
