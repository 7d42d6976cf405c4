// k_gemv instantiations for CTHIP_F32 weights (see gemv_kernels.h).
#include "gemv_kernels.h"

namespace cthip {
extern const GemvVariant kGemvF32[] = {
    V(CTHIP_F32, 16, 4), V(CTHIP_F32, 64, 1), V(CTHIP_F32, 64, 2), V(CTHIP_F32, 64, 3), V(CTHIP_F32, 64, 4), V(CTHIP_F32, 64, 6), V(CTHIP_F32, 64, 8), V(CTHIP_F32, 64, 12), V(CTHIP_F32, 64, 16), V(CTHIP_F32, 64, 24),
};
extern const int kGemvF32Count = (int)(sizeof(kGemvF32) / sizeof(kGemvF32[0]));
}  // namespace cthip
