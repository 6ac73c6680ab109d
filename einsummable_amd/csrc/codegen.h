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

enum class cg_kind { elementwise, reduce_row, reduce_col };

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
