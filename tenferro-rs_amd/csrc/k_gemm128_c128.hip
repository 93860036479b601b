// k_gemm128_c128.hip -- instantiates the 128x128 and 128x64 contraction kernels for c128 (four operand layouts).
#include "gemm128.hpp"

namespace tfh {
void launch_gemm128_c128(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st) {
    gemm::launch_gemm128_any<double, true>(g, grid, akf, bkf, st);
}
void launch_gemm128x64_c128(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st) {
    gemm::launch_gemm128x64_any<double, true>(g, grid, akf, bkf, st);
}
void launch_gemm128_grouped_c128(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st) {
    gemm::launch_gemm128_grouped_any<double, true>(g, grid, akf, bkf, st);
}
}  // namespace tfh
