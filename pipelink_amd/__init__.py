"""MI355X-native build of PipeLink's routed-expert MXFP8 FFN hot path.

Device code: hand-written HIP stages under ``stages/`` (gfx950).  Host side: a C-ABI
library (``libplk_hip.so``, sources in ``csrc/``) driven through ``ctypes`` by
``pipelink_amd.host``; PyTorch only supplies device tensors and streams.
"""
__version__ = "0.1.0"
