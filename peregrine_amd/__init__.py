"""peregrine_amd -- peregrine's quantized-inference operators on AMD MI355X.

The package is a thin host-side mirror of the reference crate's operator API
(`peregrine::quant`, `peregrine::gguf` dequant + matmul, the MoE expert FFN)
over the C ABI of ``libperegrine_hip.so`` (hand-written HIP kernels for gfx950).
There is no CPU fallback: importing the operator modules without the built
library raises, and every call needs a GPU.
"""
from . import _ffi  # noqa: F401  (fails loudly if the library is missing)
from .context import Context, default_context
from . import quant, gguf, moe, llama, mxfp4, huffman

__all__ = ["Context", "default_context", "quant", "gguf", "moe", "llama", "mxfp4", "huffman"]
