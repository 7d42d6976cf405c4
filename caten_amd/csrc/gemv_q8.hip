// k_gemv instantiations for CTHIP_Q8_0 weights (see gemv_kernels.h).
#include "gemv_kernels.h"

namespace cthip {
extern const GemvVariant kGemvQ8[] = {
    V(CTHIP_Q8_0, 16, 1), V(CTHIP_Q8_0, 16, 2), V(CTHIP_Q8_0, 16, 3), V(CTHIP_Q8_0, 16, 4), V(CTHIP_Q8_0, 32, 3), V(CTHIP_Q8_0, 32, 4), V(CTHIP_Q8_0, 64, 3), V(CTHIP_Q8_0, 64, 4), V(CTHIP_Q8_0, 64, 6), V(CTHIP_Q8_0, 64, 8),
};
extern const int kGemvQ8Count = (int)(sizeof(kGemvQ8) / sizeof(kGemvQ8[0]));
}  // namespace cthip
