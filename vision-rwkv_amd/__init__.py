"""MI355X-native WKV operators for Vision-RWKV behind the reference's operator interface.

    from vision_rwkv_amd import RUN_CUDA            # Bi-WKV  (VRWKV)
    from vision_rwkv_amd import RUN_CUDA_RWKV6      # wkv6    (VRWKV6)
"""
from ._lib import VrwkvError, LIB_PATH, build, lib, option, get_option, set_option
from .ops import WKV, RUN_CUDA, bi_wkv_forward, bi_wkv_backward, WKV_6, RUN_CUDA_RWKV6, wkv6_forward, wkv6_backward, HEAD_SIZE, q_shift, q_shift_mix, q_shift_mix_autograd, row_fuse, row_fuse_tensor_ops, maa_mix, groupnorm_gate

from . import ext
from .backbone import VRWKV, vrwkv_l
from .backbone6 import VRWKV6, vrwkv6_b, q_shift_multihead

__all__ = ["WKV", "RUN_CUDA", "bi_wkv_forward", "bi_wkv_backward", "WKV_6", "RUN_CUDA_RWKV6", "wkv6_forward", "wkv6_backward", "HEAD_SIZE", "q_shift", "q_shift_mix", "q_shift_mix_autograd", "row_fuse", "row_fuse_tensor_ops", "maa_mix", "groupnorm_gate", "VRWKV", "vrwkv_l", "VRWKV6", "vrwkv6_b", "q_shift_multihead", "ext", "VrwkvError", "LIB_PATH", "build", "lib", "option", "get_option", "set_option"]
