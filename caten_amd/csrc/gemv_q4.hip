// k_gemv instantiations for CTHIP_Q4_0 weights (see gemv_kernels.h).
#include "gemv_kernels.h"

namespace cthip {
extern const GemvVariant kGemvQ4[] = {
    V(CTHIP_Q4_0, 16, 1), V(CTHIP_Q4_0, 16, 2), V(CTHIP_Q4_0, 32, 2), V(CTHIP_Q4_0, 64, 1), V(CTHIP_Q4_0, 64, 2), V(CTHIP_Q4_0, 64, 3), V(CTHIP_Q4_0, 64, 4),
};
extern const int kGemvQ4Count = (int)(sizeof(kGemvQ4) / sizeof(kGemvQ4[0]));
}  // namespace cthip
