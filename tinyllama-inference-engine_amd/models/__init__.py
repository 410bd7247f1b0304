from . import fadutar, llama, narolorn, raketar, tugalix  # noqa: F401  (each registers its architecture)
from .builder import DecoderModel, build_model, expected_tensors

__all__ = ["DecoderModel", "build_model", "expected_tensors"]
