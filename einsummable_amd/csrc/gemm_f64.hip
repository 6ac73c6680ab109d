// f64 instantiations of the MFMA GEMM kernels (v_mfma_f64_16x16x4_f64).
#include "gemm_dma_kernel.h"
#include "gemm_kernel.h"

namespace es
{
namespace gemm
{

void launch_gemm_f64(int, int, gemm_args_t const& a, hipStream_t stream)
{
    using T = double;
    if (a.tiles_m == 0) return;
    // Operands on a vector path (along k, or along their own m / n mode) and K in whole
    // 128-byte slices: slices straight from global memory into LDS, as for f16 and f32, four
    // stages deep (the kernel holds 128 accumulator and 166 other registers: one workgroup
    // per compute unit whatever the LDS would allow).
    if (gemm_dma_wide_eligible<T>(a, 4) && a.a_mode <= 1 && a.b_mode <= 1 && a.splits <= 1) {
        auto go = [&](auto am, auto bm) {
            constexpr int AM = decltype(am)::value, BM_ = decltype(bm)::value;
            launch_gemm_dma_kernel_mode<T, 128, 128, 4, AM, BM_, 128>(a, stream);
        };
        using zero = std::integral_constant<int, 0>;
        using one = std::integral_constant<int, 1>;
        if (a.a_mode == 0) {
            a.b_mode == 0 ? go(zero{}, zero{}) : go(zero{}, one{});
        } else {
            a.b_mode == 0 ? go(one{}, zero{}) : go(one{}, one{});
        }
        return;
    }
    launch_gemm_kernel<T, 128, 128, -1, -1>(with_tile(a, 128, 128), stream);
}

}  // namespace gemm
}  // namespace es
