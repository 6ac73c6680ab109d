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
    int      outer;  // outer dimensions with more than one entry (0: the region is one row,
                     // 1: rows of one outer dimension, slot 2; else the general decomposition)
};

// op: 0 copy, 1 add, 2 mul, 3 min, 4 max.  dtype_code: 0 f16, 1 f32, 2 f64, 3 c64.
void launch_touch(touch_launch_t const& a, int elem_size, int dtype_code, int op,
                  hipStream_t stream, void* out, void const* inn);

// A group of touches into one output tensor, applied in list order by a single launch: every
// thread owns one output vector and folds the touches that cover it, so overlapping windows
// see exactly the sequential result.  All items are normalised to four dimensions.
struct touch_item_t {
    void const* inn;
    uint64_t    base_inn;    // element offset of the window's origin in the input
    uint64_t    str_inn[3];  // element strides of the three outer dimensions of the input
    uint32_t    lo[4];       // window origin in the output
    uint32_t    size[4];     // window extents
    int         op;          // 0 copy, 1 add, 2 mul, 3 min, 4 max
    int         vec_inn;     // level kernel: the input can be read as 16-byte vectors that
                             // line up with the output's vectors
    int         vec_rows;    // owner kernel: every input row starts on a 16-byte boundary ...
    int         shift;       // ... and the window lies this many elements off the output's
                             // vector grid
};

constexpr int TOUCH_BATCH_MAX = 32;  // items per level launch (kernel-argument budget)

// A list of touches for the owner-computes kernel, packed into the kernel arguments: every
// workgroup (one wavefront) owns 64 consecutive output vectors of one row of the windows'
// bounding box and folds, in list order, the items whose windows reach it.  Items of a list
// whose touches have at most two dimensions are stored with two (12 words, leading extents
// are 1 in every item), others with four (16 words): 64 or 60 touches travel in one launch.
// Words of an item, ND = 2 or 4: input pointer (2), base_inn (2), lo[ND], size[ND],
// str_inn[ND - 1] (elements, < 2^32), op | vec_rows << 8 | shift << 16.
constexpr int TOUCH_LIST_WORDS = 960;
constexpr int TOUCH_LIST_BLOCK_HOST = 64;  // output vectors per workgroup of the owner kernel

struct touch_list_t {
    uint32_t n;
    uint32_t rank;            // 1..4: of the touches; > 2 selects the four-dimensional items
    uint32_t vec;             // elements per output vector
    uint32_t chunks_per_row;  // workgroups per row of the bounding box
    uint32_t eager;           // the windows cover at least half of the bounding box
    uint32_t uniform_op;      // 0, or 1 + the op that all items share, all taking whole vectors
    uint32_t box_lo[4];       // bounding box of the windows, four normalised dimensions
    uint32_t box_size[4];     // inner extent in elements, a multiple of vec
    uint64_t out_str[3];      // element strides of the output's outer dimensions
    uint32_t w[TOUCH_LIST_WORDS];
};

inline int touch_list_item_words(int rank) { return rank > 2 ? 16 : 12; }

inline int touch_list_capacity(int rank)
{
    int const fit = TOUCH_LIST_WORDS / touch_list_item_words(rank);
    return fit < 64 ? fit : 64;  // the kernel finds its items with one 64-lane ballot
}

void launch_touch_list(touch_list_t const& b, int elem_size, int dtype_code, bool any_castable,
                       hipStream_t stream, void* out);

// A set of touches into one output tensor whose windows are pairwise disjoint: one launch,
// blockIdx.y selects the touch, every touch streams through its own window.  Output vectors
// that a window covers only in part are written element by element, so that windows sharing
// a vector never write each other's elements.
struct touch_level_t {
    int          n;
    int          vec;         // elements per output vector
    uint64_t     out_str[3];  // element strides of the output's outer dimensions
    uint64_t     max_vec;     // largest number of vectors any item covers
    touch_item_t items[TOUCH_BATCH_MAX];
};

void launch_touch_level(touch_level_t const& b, int elem_size, int dtype_code, bool any_castable,
                        hipStream_t stream, void* out);

void launch_fill_constant(int elem_size, uint64_t bits, uint64_t nelem, hipStream_t stream,
                          void* out);

void launch_fill_lowertri(int elem_size, uint64_t lower_bits, uint64_t upper_bits, uint64_t nrow,
                          uint64_t ncol, int64_t start, hipStream_t stream, void* out);

}  // namespace es
