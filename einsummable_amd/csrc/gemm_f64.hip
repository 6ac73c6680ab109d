// f64 instantiation of the MFMA GEMM kernel (general load paths only).
#include "gemm_kernel.h"

namespace es
{
namespace gemm
{

void launch_gemm_f64(int, int, gemm_args_t const& a, hipStream_t stream)
{
    if (a.tiles_m == 0) return;
    launch_gemm_kernel<double, 128, 128, -1, -1>(with_tile(a, 128, 128), stream);
}

}  // namespace gemm
}  // namespace es
