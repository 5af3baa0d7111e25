// Bi-WKV forward kernels for __hip_bfloat16 I/O.
#include "biwkv_fwd_impl.h"
namespace vrwkv {
namespace biwkv_fwd_detail {
template int biwkv_fwd_launch_io<__hip_bfloat16>(const Plan&, const float*, const float*, const void*, const void*, const void*, void*, float*, int, int, int, hipStream_t);
}
}
#ifdef VRWKV_STAMPS
VRWKV_DEFINE_STAMP_SETTER(bf16)
#endif
