from . import llama  # noqa: F401  (registers the architecture)
from .builder import DecoderModel, build_model, expected_tensors

__all__ = ["DecoderModel", "build_model", "expected_tensors"]
