"""MI355X (gfx950) kernels for the per-rank hot path of RAI-SCC/jigsaw.

The package mirrors the reference's operator-level callables (the ones stored on
``ConvNdConfig`` / ``RingAttentionConfig`` / ``RollConfig`` and the LayerNorm
autograd function) and routes each of them to hand-written HIP kernels in
``lib/libjigsaw_hip.so`` through a C ABI (``include/jigsaw_hip.h``). There is no
CPU fallback: using an operator without the built library raises.
"""

from ._lib import LibraryMissing, abi_version, lib_path, load  # noqa: F401

__all__ = ["LibraryMissing", "abi_version", "lib_path", "load"]
