// k_gemm128_f32.hip -- instantiates the 128x128 and 128x64 contraction kernels for f32 (four operand layouts).
#include "gemm128.hpp"

namespace tfh {
void launch_gemm128_f32(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st) {
    gemm::launch_gemm128_any<float, false>(g, grid, akf, bkf, st);
}
void launch_gemm128x64_f32(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st) {
    gemm::launch_gemm128x64_any<float, false>(g, grid, akf, bkf, st);
}
void launch_gemm128_grouped_f32(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st) {
    gemm::launch_gemm128_grouped_any<float, false>(g, grid, akf, bkf, st);
}
}  // namespace tfh
