// k_gemm64_f32.hip -- instantiates the 64x64-tile variants of the large-tile contraction kernel for f32.
#include "gemm128.hpp"

namespace tfh {
void launch_gemm64x64_f32(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st) {
    gemm::launch_gemm64x64_any<float, false>(g, grid, akf, bkf, st);
}
}  // namespace tfh
