// k_gemm64_f64.hip -- instantiates the 64x64-tile variants of the large-tile contraction kernel for f64.
#include "gemm128.hpp"

namespace tfh {
void launch_gemm64x64_f64(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st) {
    gemm::launch_gemm64x64_any<double, false>(g, grid, akf, bkf, st);
}
}  // namespace tfh
