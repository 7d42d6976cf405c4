// k_gemv instantiations for CTHIP_Q8_0 weights (see gemv_kernels.h).
#include "gemv_kernels.h"

namespace cthip {
extern const GemvVariant kGemvQ8[] = {
    GEMV_SHAPES_Q8(V)
};
extern const int kGemvQ8Count = (int)(sizeof(kGemvQ8) / sizeof(kGemvQ8[0]));
}  // namespace cthip
