"""MI355X (gfx950) int8 transformer-layer forward path behind LightSeq's interfaces.

The compute lives in ``lib/liblightseq_hip.so`` (hand-written HIP kernels + a C ABI,
see ``include/lightseq_hip.h``); this package is the thin Python host side: a ctypes
loader (``lightseq_amd.lib``), launcher wrappers that take torch tensors
(``lightseq_amd.kernels``) and the ``lightseq.inference``-style model classes
(``lightseq_amd.inference``).  There is no CPU fallback: without the built library
every entry point raises.
"""
__version__ = "0.1.0"
