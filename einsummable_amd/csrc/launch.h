// Host-callable launchers of the statically compiled HIP kernels.
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstdint>

namespace es
{

// A touch normalised to four dimensions (leading dimensions of size 1 are padded in):
// element strides of the three outer dimensions, base element offsets, and the innermost
// dimension counted in vectors of `vec` elements.
struct touch_launch_t {
    uint64_t size[3];     // outer extents
    uint64_t str_inn[3];  // element strides of the outer dimensions in the input tensor
    uint64_t str_out[3];
    uint64_t base_inn, base_out;
    uint64_t vec_per_row;
    uint64_t n_vec;  // size[0]*size[1]*size[2]*vec_per_row
    int      vec;    // elements per vector: 16 / elem_size, or 1
    bool     small;  // n_vec and every extent fit 32 bits
};

// op: 0 copy, 1 add, 2 mul, 3 min, 4 max.  dtype_code: 0 f16, 1 f32, 2 f64, 3 c64.
void launch_touch(touch_launch_t const& a, int elem_size, int dtype_code, int op,
                  hipStream_t stream, void* out, void const* inn);

void launch_fill_constant(int elem_size, uint64_t bits, uint64_t nelem, hipStream_t stream,
                          void* out);

void launch_fill_lowertri(int elem_size, uint64_t lower_bits, uint64_t upper_bits, uint64_t nrow,
                          uint64_t ncol, int64_t start, hipStream_t stream, void* out);

}  // namespace es
