"""MI355X-native (gfx950) kernels behind SpGT's operator and module API.

Sub-packages mirror the reference layout:
  spgt_amd.extension.bind.galerkin_attention / datamove  - operator API
  spgt_amd.network.sp_layer / sp_model                   - accelerated modules
The HIP kernels live in csrc/ and are reached through the C ABI of
libspgt_hip.so (include/spgt_hip.h).
"""
from ._lib import LIB_PATH, SpgtError, load  # noqa: F401

__all__ = ["LIB_PATH", "SpgtError", "load"]
