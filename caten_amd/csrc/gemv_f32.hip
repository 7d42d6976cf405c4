// k_gemv instantiations for CTHIP_F32 weights (see gemv_kernels.h).
#include "gemv_kernels.h"

namespace cthip {
extern const GemvVariant kGemvF32[] = {
    GEMV_SHAPES_F32(V)
};
extern const int kGemvF32Count = (int)(sizeof(kGemvF32) / sizeof(kGemvF32[0]));
}  // namespace cthip
