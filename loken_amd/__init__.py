"""MI355X (gfx950) GGUF block-quantized matmul: decode mat-vec, prefill tiled matmul and the
expert-grouped MoE variant, behind a C ABI (``include/loken_gfx950.h``).

``loken_amd.lib`` loads the shared library; ``loken_amd.ops`` is the thin host layer that takes
torch device tensors (memory and streams only) and calls the C ABI.
"""
from . import lib, synth  # noqa: F401

__all__ = ["lib", "synth"]
