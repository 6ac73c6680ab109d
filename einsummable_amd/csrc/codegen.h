// scalarop code generator: lowers an einsummable whose join is an arbitrary scalarop tree
// (elementwise, broadcast elementwise, and elementwise-then-reduce with a castable) to HIP
// source specialised for its structure, compiles it for gfx950 with the runtime compiler and
// launches it.  This replaces the reference's one-cuTENSOR-call-per-scalarop-node lowering
// (src/einsummable/simplescalarop.cc:432-489, src/engine/gpu/gpu_kernel_manager.cc:1951-2079)
// and its hand-matched special kernels (src/engine/gpu/cuda_kernels.cu:651-944) with a single
// fused pass over HBM per einsummable.
#pragma once
#include "ir.h"

#include <string>
#include <vector>

namespace es
{

enum class cg_kind { elementwise, reduce_row, reduce_col, row_chain };

// Everything needed to launch a generated kernel: the source, its entry point, the launch
// geometry and the packed argument block minus the pointers.
struct cg_kernel_t {
    cg_kind     kind;
    std::string source;
    std::string entry;
    int         n_inns = 0;
    bool        idx64 = false;
    int         vec = 1;                 // elements per vector access
    bool        row_pairs = false;       // elementwise: a thread moves two neighbouring input rows
    unsigned    block = 256;
    uint64_t    grid = 0;
    std::vector<uint64_t> params;        // written after the pointers as idx_t values
    // byte alignment every pointer must satisfy for this variant
    std::vector<int> out_inn_align;      // [0] = out, [1+k] = input k
    // Two-pass reductions: `splits` > 1 slices of the aggregated range run side by side
    // (grid z) and leave partial results in the workspace, which `entry2` then folds.
    int         splits = 1;
    std::string entry2;
    uint64_t    grid2 = 0;               // workgroups of `entry2`; 0: the same as `grid`
    uint64_t    ws_bytes = 0;
};

// Generate the kernel for a (merged) einsummable.  `max_vec` caps the vector width (1 forces
// the scalar variant used when a buffer is not 16-byte aligned).
cg_kernel_t generate_kernel(einsummable_t const& e, int max_vec = 16);

// A chain of nodes over the rows of one tensor whose intermediate results never leave the
// registers: reductions over a row (the innermost mode), pointwise steps on the per-row
// values, and a last elementwise node that writes the tensor -- softmax (row max, sum of
// exp(x - max), exp(x - max) / sum), normalisations.  Each row is held by a team of lanes,
// read once and written once; every stage computes what its own kernel would have computed,
// in the same order and with the same roundings (a stage's result passes through its output
// dtype before the next stage uses it), so the last node's output is bit for bit what the
// nodes give one after the other.  The reference runs such chains node by node
// (src/engine/gpu/gpu_kernel_manager.cc:326-430 are its hand-matched pieces of softmax).
struct cg_chain_t {
    std::vector<uint64_t> shape;  // join shape of every stage; the last mode is the row
    struct ext_t {
        dtype_t          dtype;
        std::vector<int> modes;  // increasing; with the last mode: a tensor read by vectors,
                                 // without: one value per row (or per kernel)
    };
    std::vector<ext_t> exts;  // the chain's inputs, in the order of the kernel's pointers
    struct stage_t {
        scalarop_t                join;
        std::optional<castable_t> castable;  // set: a reduction over the row
        std::vector<int>          args;      // per hole: k >= 0 external k, -1 - t: stage t's result
    };
    // reductions and pointwise steps on per-row values in any order, then the elementwise node
    std::vector<stage_t> stages;
};

// Throws ir_error when the chain has no such kernel (rows too long for the registers, inputs
// that are gathered, a stage the row reduction would have split ...).
cg_kernel_t generate_row_chain(cg_chain_t const& c, int max_vec = 16);

// Elements of a row per lane and step in the generated row reductions, by the smallest element
// among output and inputs: two reductions that agree in it (and in the row's length) add a
// row's elements in the same order.
int row_reduction_lane_elems(int smallest_elem_bytes);

// Whether generate_kernel makes a row reduction of e (some input holds the innermost mode).
bool is_row_reduction(einsummable_t const& e);

// Compile `source` for `arch` (e.g. "gfx950"); returns the code object.  Throws km_error.
std::vector<char> compile_hip_source(std::string const& source, std::string const& name,
                                     std::string const& arch);

// The code object of a generated source: read from the on-disk cache (ES_KM_CACHE_DIR, default
// ~/.cache/es_km; "off" disables) or compiled and written there.  *from_disk reports a hit.
std::vector<char> code_object_for(std::string const& source, bool* from_disk);

}  // namespace es
