"""MI355X-native WKV operators for Vision-RWKV behind the reference's operator interface.

    from vision_rwkv_amd import RUN_CUDA            # Bi-WKV  (VRWKV)
"""
from ._lib import VrwkvError, LIB_PATH, build, lib
from .ops import WKV, RUN_CUDA, bi_wkv_forward

__all__ = ["WKV", "RUN_CUDA", "bi_wkv_forward", "VrwkvError", "LIB_PATH", "build", "lib"]
