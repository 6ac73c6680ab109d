// The exec-node layer over the kernel manager: a dependency graph of apply (einsummable /
// touch), fill, copy, evict / load and dummy nodes addressed by offsets into one device
// arena, run on one GPU.
//
// It plays the part of the reference's GPU exec graph for these node kinds
// (src/engine/exec_graph.h:17-80; gpu_einsummable_t, gpu_touch_t, gpu_constant_t,
// gpu_lowerTri_t, gpu_copy_t, gpu_evict_t, gpu_load_t, dummy_t in src/engine/gpu/exec_nodes.h and
// src/engine/gpu/exec_graph.cc:258-404, 600-690).  The reference drives its graph from a host
// event loop: every node takes a stream from a pool, launches, and reports back through
// cudaStreamAddCallback, after which the loop releases the node's dependents
// (src/engine/exec_state.cc).  That is one host round trip per node.  Here the order is fixed
// once, at finalize(): nodes are placed on a small pool of streams and every dependency that
// crosses streams becomes an event wait on the device, so run() is a burst of launches with
// no host synchronisation at all.  (A single-stream placement can also be captured into a
// HIP graph; capturing the fork / join of pool streams crashed the ROCm 7.2 runtime and is
// not supported.)
//
// Touch groups keep the reference's meaning (src/engine/managers.cc:3-21,
// gpu/exec_graph.cc:354-378): touches of one group are serialised, and the first of a group
// to run has its castable cleared (it initialises the output).  With a fixed order "first to
// run" is the first one inserted.  A touch without a group is a plain copy
// (gpu/exec_graph.cc:176-181).
#pragma once
#include "kernel_manager.h"

#include <cstdint>
#include <string>
#include <utility>
#include <vector>

namespace es
{

struct mem_t {
    uint64_t offset;
    uint64_t size;
};

class apply_graph_t
{
public:
    // `km` may be null: the graph can then be planned and inspected but not run
    explicit apply_graph_t(kernel_manager_t* km);
    ~apply_graph_t();
    apply_graph_t(apply_graph_t const&) = delete;
    apply_graph_t& operator=(apply_graph_t const&) = delete;

    // mems[0] is the output, the rest are the inputs in order (memgraph.h:252-263).
    // `deps` are ids of nodes that must complete first.  Each returns the new node's id.
    int add_einsummable(einsummable_t const& e, std::vector<mem_t> const& mems,
                        std::vector<int> const& deps);
    int add_touch(touch_t const& t, int group, std::vector<mem_t> const& mems,
                  std::vector<int> const& deps);
    int add_constant_fill(dtype_t dtype, uint64_t value_bits, uint64_t nelem, mem_t out,
                          std::vector<int> const& deps);
    int add_lowertri_fill(dtype_t dtype, uint64_t lower_bits, uint64_t upper_bits, uint64_t nrow,
                          uint64_t ncol, int64_t start, mem_t out, std::vector<int> const& deps);
    int add_copy(mem_t dst, mem_t src, std::vector<int> const& deps);
    // A node that launches nothing and only carries dependencies: what the reference makes
    // of inputmem / inputsto / partialize / alloc / del nodes and of nodes that live on
    // another device (gpu/exec_graph.cc:94-97).  `range` is kept for inspection only and
    // takes no part in add_memory_dependencies.
    // `is_del`: the dummy stands for the deletion of `range` (what a caller's own dels and the
    // memgraph's del nodes are); the other ranged dummies (inputmem, alloc, partialize) only
    // name a range and never let optimize() drop what is stored there
    int add_dummy(mem_t range, std::vector<int> const& deps, bool is_del = true);
    // Host storage (gpu_evict_t / gpu_load_t, gpu/exec_graph.cc:466-577; the reference's
    // storage is host memory too, src/engine/gpu/storage_manager.h).  evict copies an arena
    // range into the storage slot `storage_id`, load copies the slot back.  Slots are pinned
    // host buffers allocated at finalize, one per id, sized for the largest user; the
    // copies are asynchronous on the node's stream like every other node.
    int add_evict(mem_t src, int storage_id, std::vector<int> const& deps);
    int add_load(int storage_id, mem_t dst, std::vector<int> const& deps);
    // declares a slot that the caller fills before run (an inputsto node)
    void declare_storage(int storage_id, uint64_t size);
    // after finalize: host-side access to a slot (the caller orders these against run)
    void storage_write(int storage_id, void const* src, uint64_t size);
    void storage_read(int storage_id, void* dst, uint64_t size) const;

    // Adds, between every pair of nodes in insertion order, the dependency their memory
    // ranges imply (read after write, write after write, write after read).
    void add_memory_dependencies();

    // Removes round trips through memory that the node list spells out but the results do not
    // need, without changing one bit of what stays in memory.  The output S of a node u need
    // not be stored when u alone writes it, it is deleted after its readers -- a dummy that
    // covers S and depends on the last of them is read as S's del node (memgraph.h: del_t) --
    // and nothing before the last reader rewrites what u reads:
    //  - the one reader is a touch that copies S whole (the formation / partialize copy that
    //    follows every contraction and reduction, taskgraph.cc:3047-3061): u writes the
    //    copy's output itself;
    //  - every reader is an elementwise einsummable, or a reduction of one input, that takes S
    //    position by position, and u is elementwise: each reader becomes one einsummable
    //    whose join is its own with u's put in place of the hole (scalarop_t::compose keeps
    //    the rounding a store and a load make).  With several readers u is computed once
    //    per reader, which is taken while u's inputs are smaller than the traffic S caused.
    // A merged node stands at its reader's place and u becomes a dummy, so ids, and
    // dependencies on either, stay valid.  Einsummables the kernel manager cannot build stay as they are.
    // Before finalize; returns the number of nodes absorbed.  The reference has no such pass
    // at this level: its graphs reach the engine with these nodes in them.
    //
    // And a chain over rows becomes one launch: row reductions (and pointwise steps on their
    // per-row results) whose outputs only feed each other and one last elementwise node over
    // the same rows -- softmax as row max, sum of exp(x - max), exp(x - max) / sum; a
    // normalisation as sum of squares, power, scale -- with intermediate results that are
    // deleted afterwards.  The last node then reads each row once, keeps it in registers
    // through every stage and writes it once (codegen.h: cg_chain_t); its output has the bits
    // the nodes give one after the other.  The absorbed nodes become dummies.  Counted in the
    // return value; ES_KM_ROW_CHAINS=0 switches it off.
    int optimize();

    // Builds every einsummable on the kernel manager (throws km_error when one has no
    // kernel), fixes the launch order and places the nodes on `n_streams` streams.
    void finalize(int n_streams);

    // Enqueues the whole graph.  Work is ordered after what `main` holds at the call and
    // `main` is ordered after all of it on return; nothing synchronises with the host.
    void run(hipStream_t main, void* arena) const;

    // One node at a time, for a host event loop that keeps the dependencies itself (the
    // reference's exec_state_t, src/engine/exec_state.cc:197-219): enqueues node `id` on
    // `stream` -- no waits, no events; the caller launches a node when everything it depends
    // on has reported back -- and, behind it on the same stream, a host function that calls
    // `callback(user)` when the node's work is done (gpu_einsummable_t::launch and
    // gpu_touch_t::launch, src/engine/gpu/exec_graph.cc:277-335, 354-404, with
    // cudaStreamAddCallback).  The callback runs on a thread of the HIP runtime and must not
    // call the HIP API.  `workspace`: at least node_workspace(id) bytes, the caller's (from
    // its pool); unused by nodes that need none.  `first_in_group`: for a grouped touch, 1
    // clears the castable (the first touch of a group to run initialises the output,
    // managers.cc:3-21), 0 keeps it, -1 takes what insertion order said.  After finalize.
    void launch_node(int id, hipStream_t stream, void* arena, void* workspace,
                     uint64_t workspace_bytes, int first_in_group, void (*callback)(void*),
                     void* user) const;
    uint64_t node_workspace(int id) const;
    int      group_of(int id) const { return nodes_[id].group; }

    // "<kind> <range>..." -- the output first, "offset:size" each -- and for an einsummable
    // its key (shape, castable, modes, join text) after " | "; for inspection and tests
    std::string describe(int id) const;
    // The HIP source of the kernel the code generator makes for node `id` -- an einsummable
    // it would take (what optimize() merged included) or a chain over rows -- empty for any
    // other node.  Works without a kernel manager and before finalize: an aid for tests.
    std::string generated_source(int id) const;

    int n_nodes() const { return int(nodes_.size()); }
    // smallest arena that holds every range a node touches
    uint64_t arena_bytes() const;
    // 0 einsummable, 1 touch, 2 constant fill, 3 lowertri fill, 4 copy, 5 dummy, 6 evict,
    // 7 load, 8 chain over rows (made by optimize)
    int                       kind_of(int id) const { return int(nodes_[id].kind); }
    std::vector<mem_t> const& mems_of(int id) const { return nodes_[id].mems; }
    // after finalize: launch position, stream and dependencies (own + implied) of a node
    int                     position_of(int id) const { return nodes_[id].position; }
    int                     stream_of(int id) const { return nodes_[id].stream; }
    std::vector<int> const& deps_of(int id) const { return nodes_[id].deps; }
    // number of event waits run() enqueues (dependencies that cross streams)
    int n_cross_stream_waits() const { return n_waits_; }
    // number of kernel / copy launches one run() makes (a run of grouped touches counts once)
    int n_launches() const;

private:
    enum class kind_t { einsummable, touch, constant, lowertri, copy, dummy, evict, load, chain };
    struct node_t {
        kind_t             kind;
        einsummable_t      e;
        touch_t            touch;
        std::optional<castable_t> group_castable;  // as given, before the first member's is cleared
        int                group = -1;
        dtype_t            dtype = dtype_t::f32;
        uint64_t           bits0 = 0, bits1 = 0, n0 = 0, n1 = 0;
        int64_t            start = 0;
        int                storage_id = -1;
        bool               is_del = false;  // dummies: the range is deleted here
        std::vector<mem_t> mems;
        std::vector<int>   deps;
        std::vector<int>   waits;  // dependencies on other streams, reduced
        int                position = -1;
        int                stream = -1;
        bool               record = false;  // some dependent waits for this node's event
        // Touches of one group that follow each other in launch order and write the same
        // output run as one launch (kernel_manager_t::touch_batch), at the first one's
        // place: `batch_head` is that node's id (-1: launched on its own), and the head
        // holds the ids of all of them.  Likewise independent einsummables of one key that
        // follow each other, when their kernel takes several runs at once
        // (plan_t::run_group: the q, k and v projections of a layer).
        int                batch_head = -1;
        std::vector<int>   batch;
        // chain over rows: its kernel (null without a kernel manager) and how many nodes it
        // stands for; `e` is the last node's einsummable, mems the output and the chain's inputs
        std::shared_ptr<plan_t> chain_plan;
        int                     chain_stages = 0;
    };

    int  insert(node_t&& n, std::vector<int> const& deps);
    bool absorb_into_readers(int u);
    int  fuse_row_chain(int v);
    void launch(node_t const& n, hipStream_t stream, char* arena) const;

    kernel_manager_t*        km_;
    std::vector<node_t>      nodes_;
    std::vector<int>         order_;
    std::vector<hipStream_t> streams_;
    std::vector<hipEvent_t>  events_;  // one per node that records
    std::vector<int>         event_of_;
    // scratch for kernels that need it: one buffer per stream (a stream runs its nodes one
    // after the other), sized for the stream's hungriest node; the reference takes these
    // from a pool per launch (src/engine/gpu/workspace.cc:48-91)
    std::vector<void*>       workspace_;
    std::vector<uint64_t>    workspace_bytes_;
    struct slot_t {
        uint64_t size = 0;
        void*    host = nullptr;  // pinned
    };
    std::vector<std::pair<int, slot_t>> slots_;  // by storage id
    slot_t*       slot(int storage_id);
    slot_t const* slot(int storage_id) const;
    hipEvent_t               fork_ = nullptr;
    std::vector<hipEvent_t>  joins_;
    // per stream: holds a node at all; its last node is not yet waited for by a node of the
    // first stream (only then run() ends with a join of that stream)
    std::vector<char>        stream_used_, stream_joins_;
    int                      n_waits_ = 0;
    bool                     finalized_ = false;
};

}  // namespace es
