// f64 instantiation of the MFMA GEMM kernel (general load paths only).
#include "gemm_kernel.h"

namespace es
{
namespace gemm
{

void launch_gemm_f64(int, int, gemm_args_t const& a, hipStream_t stream)
{
    if (a.tiles_m == 0) return;
    launch_gemm_kernel<double, 128, 128, -1, -1>(a, stream);
}

bool gemm_has_tile(int elem_size, int bm, int bn)
{
    if (bm == 128 && bn == 128) return true;
    return elem_size < 8 && bm == 256 && bn == 256;
}

}  // namespace gemm
}  // namespace es
