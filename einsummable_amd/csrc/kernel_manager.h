// The kernel manager: plans one kernel per (merged) einsummable at build() and launches it on
// raw device buffers at operator().  Same surface and error behaviour as the reference's
// kernel_manager_t (src/engine/gpu/gpu_kernel_manager.h:274-321): build returns nullopt for
// an unsupported einsummable and never throws for that reason; calling an un-built
// einsummable, passing the wrong number of inputs or an undersized workspace throws
// (gpu_kernel_manager.cc:1103-1107, 1126, 1260, 1586, 1968).
#pragma once
#include "ir.h"

#include <hip/hip_runtime_api.h>

#include <memory>
#include <optional>
#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

namespace es
{

enum class km_status : int {
    invalid = -1,
    not_built = -2,
    workspace = -3,
    inputs = -4,
    device = -5
};

struct km_error : std::runtime_error {
    km_error(km_status s, std::string const& what) : std::runtime_error(what), status(s) {}
    km_status status;
};

// One planned kernel.  run() only enqueues work on `stream`.
struct plan_t {
    virtual ~plan_t() = default;
    virtual void run(hipStream_t stream, void* out, void const* const* inns, void* workspace,
                     uint64_t workspace_bytes) const = 0;
    uint64_t    workspace_bytes = 0;
    int         n_inns = 0;
    std::string description;
    // How many runs of this plan on different buffers one launch can take (1: none), and
    // that launch: outs[g], and inns[g * n_inns + k] for run g.  Same results as the runs
    // one after the other.
    // the HIP source of a generated kernel (its vector variant), empty for the others
    virtual std::string source() const { return std::string(); }
    virtual int  max_group() const { return 1; }
    virtual void run_group(hipStream_t, int /*runs*/, void* const* /*outs*/,
                           void const* const* /*inns*/) const
    {
        throw km_error(km_status::invalid, "this kernel does not take several runs at once");
    }
    // Plans whose generated kernels were planned without being compiled (plan_codegen with
    // `defer`) add themselves: finish_codegen_plans compiles and loads them together.
    virtual void deferred(std::vector<plan_t*>&) {}
};

class kernel_manager_t
{
public:
    explicit kernel_manager_t(int device);
    ~kernel_manager_t();

    std::optional<uint64_t> build(einsummable_t const& e);
    // build() for a list: the generated kernels of the einsummables not yet planned are
    // compiled together, as one program (runtime compilation is nearly all of a cold build,
    // and nearly all of it is the compiler's fixed cost per program).  Same results and same
    // error contract as build() called for each in turn; like build(), not to be called
    // concurrently.
    std::vector<std::optional<uint64_t>> build_many(std::vector<einsummable_t> const& es);
    // Whether build() would succeed, without compiling anything: the plan is made (a generated
    // kernel as source only) and kept for the build() or build_many() that follows, which
    // compiles it -- build_many() with all the others as one program.
    bool                    buildable(einsummable_t const& e);
    uint64_t                workspace_size(einsummable_t const& e) const;
    std::string             describe(einsummable_t const& e) const;

    void operator()(einsummable_t const& e, hipStream_t stream, void* out,
                    std::vector<void const*> const&             inns,
                    std::optional<std::tuple<void*, uint64_t>> workspace = std::nullopt) const;

    void operator()(touch_t const& touch, hipStream_t stream, void* out, void const* inn) const;

    // All touches write the same output tensor; the result equals applying them one after
    // the other in list order, in one launch per 32 touches.
    void touch_batch(std::vector<touch_t> const& touches, hipStream_t stream, void* out,
                     std::vector<void const*> const& inns) const;

    void constant_fill(dtype_t dtype, uint64_t value_bits, uint64_t nelem, hipStream_t stream,
                       void* out) const;
    void lowerTri_fill(dtype_t dtype, uint64_t lower_bits, uint64_t upper_bits, uint64_t nrow,
                       uint64_t ncol, int64_t start, hipStream_t stream, void* out) const;

    // Lookup by a caller-made key (the C ABI keys on the raw descriptor text so that the hot
    // path does not re-parse the scalarop).
    plan_t const* find_raw(std::string const& raw_key) const;
    void          alias_raw(std::string const& raw_key, einsummable_t const& e);
    void          run_plan(plan_t const& p, hipStream_t stream, void* out,
                           void const* const* inns, int n_inns, void* workspace,
                           uint64_t workspace_bytes) const;

    // the plan build() made for this einsummable, or null (for callers that launch the
    // same node many times and do not want the lookup on their hot path)
    plan_t const* plan_of(einsummable_t const& e) const { return find(e.merge_adjacent_dims()); }

    int device() const { return device_; }

private:
    plan_t const* find(einsummable_t const& merged) const;
    // the planners in their order; null when none takes it.  Touches no member.
    std::shared_ptr<plan_t> make_plan(einsummable_t const& merged, bool defer = false) const;

    int                                                      device_;
    std::unordered_map<std::string, std::shared_ptr<plan_t>> plans_;      // by merged key
    std::unordered_map<std::string, std::shared_ptr<plan_t>> planned_;    // by buildable(): not compiled yet
    std::unordered_map<std::string, std::shared_ptr<plan_t>> raw_plans_;  // by caller key
};

// Planners (one translation unit each).  Each returns nullptr when the einsummable is not
// of its kind; `e` has already been through merge_adjacent_dims.
std::shared_ptr<plan_t> plan_contraction(einsummable_t const& e, int device);
std::shared_ptr<plan_t> plan_complex_contraction(einsummable_t const& e, int device);
std::shared_ptr<plan_t> plan_transpose(einsummable_t const& e, int device);
// `defer`: generate the kernels' source only; finish_codegen_plans compiles and loads
std::shared_ptr<plan_t> plan_codegen(einsummable_t const& e, int device, bool defer = false);
// The kernel of a chain of nodes over rows (codegen.h: cg_chain_t), compiled and loaded on
// `device` (a negative device: generated only, for inspection; `defer`: compiled and loaded by
// finish_codegen_plans, with the other kernels of its list).  run() takes the last node's
// output and the chain's inputs.  Throws ir_error when the chain has no such kernel.
struct cg_chain_t;
std::shared_ptr<plan_t> plan_row_chain(cg_chain_t const& c, int device, bool defer = false);
// Compiles the generated kernels of all these plans as ONE runtime-compiled program (the
// compiler's fixed cost per program is most of the time of a small kernel, and it compiles
// one program at a time whatever the number of calling threads: the 25 distinct generated
// kernels of a LLaMA layer take 9.3 s one by one and 0.8 s as one program on the same
// machine) and loads the module on `device`.
void finish_codegen_plans(std::vector<plan_t*> const& plans, int device);

}  // namespace es
