// k_gemv instantiations for CTHIP_Q4_0 weights (see gemv_kernels.h).
#include "gemv_kernels.h"

namespace cthip {
extern const GemvVariant kGemvQ4[] = {
    GEMV_SHAPES_Q4(V)
};
extern const int kGemvQ4Count = (int)(sizeof(kGemvQ4) / sizeof(kGemvQ4[0]));
}  // namespace cthip
