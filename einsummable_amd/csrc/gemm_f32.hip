// fp32 instantiations of the MFMA GEMM kernel.
#include "gemm_dma_kernel.h"
#include "gemm_kernel.h"

namespace es
{
namespace gemm
{

void launch_gemm_f32(int bm, int bn, gemm_args_t const& a, hipStream_t stream)
{
    using T = float;
    if (a.tiles_m == 0) return;
    if (gemm_dma_eligible<T>(a)) {
        if (bm == 256 && bn == 256) return launch_gemm_dma_kernel<T, 256, 256, 4>(a, stream);
        if (bm == 256 && bn == 128) return launch_gemm_dma_kernel<T, 256, 128, 4>(a, stream);
        if (bm == 128 && bn == 256) return launch_gemm_dma_kernel<T, 128, 256, 4>(a, stream);
        if (bm == 128 && bn == 128 && a.wide_slices && a.a_mode == 0 &&
            gemm_dma_wide_eligible<T>(a, uint32_t(a.wide_slices))) {
            if (a.b_mode == 0) {
                if (a.wide_slices == 2) launch_gemm_dma_kernel_mode<T, 128, 128, 2, 0, 0, 128>(a, stream);
                else if (a.wide_slices == 3) launch_gemm_dma_kernel_mode<T, 128, 128, 3, 0, 0, 128>(a, stream);
                else launch_gemm_dma_kernel_mode<T, 128, 128, 4, 0, 0, 128>(a, stream);
            } else {
                if (a.wide_slices == 2) launch_gemm_dma_kernel_mode<T, 128, 128, 2, 0, 1, 128>(a, stream);
                else if (a.wide_slices == 3) launch_gemm_dma_kernel_mode<T, 128, 128, 3, 0, 1, 128>(a, stream);
                else launch_gemm_dma_kernel_mode<T, 128, 128, 4, 0, 1, 128>(a, stream);
            }
            if (a.splits > 1) launch_gemm_fold<T>(a, stream);
            return;
        }
        if (bm == 128 && bn == 128) return launch_gemm_dma_kernel<T, 128, 128, 4>(a, stream);
    }
    if (bm == 256 && bn == 256 && launch_gemm_fast<T, 256, 256>(a, stream)) return;
    gemm_args_t const b = with_tile(a, 128, 128);
    if (launch_gemm_fast<T, 128, 128>(b, stream)) return;
    launch_gemm_kernel<T, 128, 128, -1, -1>(b, stream);
}

}  // namespace gemm
}  // namespace es
