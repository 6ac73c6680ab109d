/*
 * es_km.h -- C ABI of the MI355X (gfx950) kernel manager for einsummable apply nodes.
 *
 * This is the drop-in boundary for the GPU apply path of dcbdan/einsummable: every entry
 * point replaces one member of the reference's `kernel_manager_t`
 * (src/engine/gpu/gpu_kernel_manager.h:274-321).  The reference has no FFI layer; its exec
 * nodes call the C++ class directly (src/engine/gpu/exec_graph.cc:135, 316, 384, 623, 675).
 * A maintainer binds this library by giving `kernel_manager_t` the members shown in
 * `es_km.hpp` (a header-only C++ class over this ABI with the reference's member names).
 *
 * Conventions
 *  - Descriptors travel in the reference's own text forms: a scalarop is the text written by
 *    `operator<<(ostream&, scalarop_t)` (src/einsummable/scalarop.cc:2881-3011), e.g.
 *    "*[hole|f16@0,hole|f16@1]"; a castable is one of '+' 'x' 'v' '^'
 *    (scalarop.cc:3078-3093) or 0 for none; dtypes are the enum values below
 *    (scalarop.h:10).
 *  - An einsummable is (join_shape[join_rank], inns, out_rank, join text, castable) exactly
 *    as the fields of `einsummable_t` (src/einsummable/einsummable.h:8-20).  `inns` is
 *    flattened: input k holds modes inns_flat[inns_offsets[k] .. inns_offsets[k+1]).
 *  - All device pointers are owned by the caller (sub-ranges of its arena); the library
 *    never allocates or frees tensor memory.  Every launch is asynchronous on the given
 *    stream (`hipStream_t` passed as void*); nothing synchronises.
 *  - Return codes: 0 success, ES_KM_UNSUPPORTED (1) where the reference returns nullopt,
 *    negative where the reference throws std::runtime_error.  The message of the last
 *    failure on a handle is available from es_km_last_error.
 */
#ifndef ES_KM_H
#define ES_KM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ES_KM_F16 = 0, ES_KM_F32 = 1, ES_KM_F64 = 2, ES_KM_C64 = 3 };

enum {
    ES_KM_OK = 0,
    ES_KM_UNSUPPORTED = 1,       /* build: no kernel for this einsummable (reference: nullopt)  */
    ES_KM_ERR_INVALID = -1,      /* malformed descriptor (reference: constructor throws)        */
    ES_KM_ERR_NOT_BUILT = -2,    /* execute / workspace_size before build                       */
    ES_KM_ERR_WORKSPACE = -3,    /* workspace missing or smaller than build() reported          */
    ES_KM_ERR_INPUTS = -4,       /* wrong number of input pointers                              */
    ES_KM_ERR_DEVICE = -5        /* HIP runtime or runtime-compiler failure                     */
};

typedef struct es_km es_km_t;

/* kernel_manager_t(int device)                          gpu_kernel_manager.h:275
 * Returns NULL when the device cannot be selected (see es_km_last_error(NULL)). */
es_km_t* es_km_create(int device);
void     es_km_destroy(es_km_t* km);

/* Message of the most recent failure on this handle (on this thread for km == NULL). */
const char* es_km_last_error(es_km_t* km);

/* optional<workspace_info_t> build(einsummable_t const&)        gpu_kernel_manager.h:302
 * Plans (and, for elementwise / reduction forms, runtime-compiles) the kernel for one
 * einsummable and memoises it under the einsummable's value, after merge_adjacent_dims
 * (gpu_kernel_manager.cc:590-600).  *workspace_bytes receives the scratch size execute needs. */
int es_km_build(es_km_t* km, const uint64_t* join_shape, int join_rank, const int* inns_flat,
                const int* inns_offsets, int n_inns, int out_rank, const char* join_text,
                char castable, uint64_t* workspace_bytes);

/* workspace_info_t workspace_size(einsummable_t const&) const   gpu_kernel_manager.h:304 */
int es_km_workspace_size(es_km_t* km, const uint64_t* join_shape, int join_rank,
                         const int* inns_flat, const int* inns_offsets, int n_inns, int out_rank,
                         const char* join_text, char castable, uint64_t* workspace_bytes);

/* void operator()(einsummable_t const&, cudaStream_t, void* out, vector<void const*> inns,
 *                 optional<tuple<void*, uint64_t>> workspace) const
 *                                                               gpu_kernel_manager.h:308-312
 * workspace may be NULL when build reported 0 bytes. */
int es_km_execute(es_km_t* km, const uint64_t* join_shape, int join_rank, const int* inns_flat,
                  const int* inns_offsets, int n_inns, int out_rank, const char* join_text,
                  char castable, void* stream, void* out, const void* const* inns,
                  int n_inn_ptrs, void* workspace, uint64_t workspace_bytes);

/* es_km_execute with the workspace supplied by the library: it allocates nothing.  No
 * counterpart in the reference, whose callers take workspaces from a pool of device
 * allocations (src/engine/gpu/workspace.cc:48-91).  It is for callers that cannot allocate
 * when they execute: code under HIP graph capture, tight serving loops, harnesses that forbid
 * allocation.  The workspace is ES_KM_STATIC_WORKSPACE_BYTES of device memory that belongs to
 * the library's code object on each device (held until the process ends); an einsummable
 * whose build reported more fails with ES_KM_ERR_WORKSPACE, one that reported 0 runs as with
 * es_km_execute.  Every call on a device uses the same memory and leaves its partial results
 * there: calls that may overlap in time on one device (different streams, different threads)
 * race; order them, or give all but one a workspace of their own through es_km_execute.
 * Results are bit-identical to es_km_execute. */
#define ES_KM_STATIC_WORKSPACE_BYTES (64ull << 20)
int es_km_execute_static_workspace(es_km_t* km, const uint64_t* join_shape, int join_rank,
                                   const int* inns_flat, const int* inns_offsets, int n_inns,
                                   int out_rank, const char* join_text, char castable,
                                   void* stream, void* out, const void* const* inns,
                                   int n_inn_ptrs);

/* Name of the kernel family chosen by build for this einsummable, e.g. "elementwise",
 * "reduce_row", "contraction_mfma_f16" (diagnostics; no counterpart in the reference apart
 * from its force_debug printouts, gpu_kernel_manager.cc:1008-1034). */
int es_km_describe(es_km_t* km, const uint64_t* join_shape, int join_rank, const int* inns_flat,
                   const int* inns_offsets, int n_inns, int out_rank, const char* join_text,
                   char castable, char* out, size_t cap);

/* void operator()(touch_t const&, cudaStream_t, void* out, void const* inn) const
 *                                                               gpu_kernel_manager.h:306
 * touchdims = rank x {d_inn, d_out, offset_inn, offset_out, size} (touch.h:8-13).
 * simplify() is applied inside, as build_touch does (src/engine/gpu/kernels.cc:150-152);
 * more than four dimensions after simplify is an error. */
int es_km_touch(es_km_t* km, const uint64_t* touchdims, int rank, char castable, int dtype,
                void* stream, void* out, const void* inn);

/* A group of touches into ONE output tensor in one call (one launch for up to 64 touches): the
 * result is bit-identical to calling es_km_touch on each, in list order, including where
 * windows overlap.  touchdims holds the selections back to back (ranks[i] x 5 values each),
 * castables[i] is '+','x','v','^' or 0, inns[i] the input of touch i.  All touches share the
 * dtype, the rank and the output extents.  No counterpart in the reference, whose engine
 * issues the touches of a group one by one (src/engine/gpu/exec_graph.cc:354-404); offered
 * because a partialize unit's inputs all hit the same output region
 * (src/einsummable/taskgraph.cc:3224-3266) and each launch otherwise costs more than the
 * copy it performs. */
int es_km_touch_batch(es_km_t* km, int n_touches, const uint64_t* touchdims, const int* ranks,
                      const char* castables, int dtype, void* stream, void* out,
                      const void* const* inns);

/* void constant_fill(fill_t::constant_t const&, cudaStream_t, void* out) const
 *                                                               gpu_kernel_manager.h:321
 * value_bits: the scalar's bytes, little-endian, in the low bytes of a uint64
 * (scalar_t::data, scalarop.h:70-71); nelem = product of the fill's shape. */
int es_km_fill_constant(es_km_t* km, int dtype, uint64_t value_bits, uint64_t nelem, void* stream,
                        void* out);

/* void lowerTri_fill(fill_t::lowertri_t const&, cudaStream_t, void* out) const
 *                                                               gpu_kernel_manager.h:320
 * out[i, j] = (i - start >= j) ? lower : upper with signed i - start (fill.h:14-24). */
int es_km_fill_lowertri(es_km_t* km, int dtype, uint64_t lower_bits, uint64_t upper_bits,
                        uint64_t nrow, uint64_t ncol, int64_t start, void* stream, void* out);

/* Diagnostics without a device: generate (and, with compile != 0, runtime-compile for
 * gfx950) the kernel source the scalarop code generator emits for an elementwise or
 * elementwise-then-reduce einsummable.  No counterpart in the reference (its closest
 * relative is scalarop_t::to_cppstr, src/einsummable/scalarop.cc:1495-1555). */
int es_km_codegen_source(const uint64_t* join_shape, int join_rank, const int* inns_flat,
                         const int* inns_offsets, int n_inns, int out_rank, const char* join_text,
                         char castable, int compile, char* out, size_t cap);

/* Host-logic diagnostics without a device (used by the CPU test-suite).
 * es_km_scalarop_roundtrip: parse a scalarop text with the library's parser and print it
 *   back (operator>> / operator<< of scalar_ns::node_t, scalarop.cc:2881-3060), reporting
 *   the output dtype and the number of holes.
 * es_km_merge_adjacent_dims: einsummable_t::merge_adjacent_dims (einsummable.cc:166-218)
 *   followed by str() (einsummable.cc:483-501); returns the new join rank (>= 1) or a
 *   negative error.  Output arrays must hold join_rank / the input's mode count entries. */
int es_km_scalarop_roundtrip(const char* text, char* out, size_t cap, int* out_dtype,
                             int* n_inputs);
/* es_km_scalarop_simplify: parse, replace the n_vars named variables by constants
 *   (scalarop_t::replace_variables; n_vars may be 0), bring the expression to the reference's
 *   canonical form (node_t::simplify, scalarop.cc:1233-1416, applied by every scalarop_t
 *   constructor, :1942-1948) and print it.  What es_km_graph_load_memgraph does to a join
 *   that carries variables (gpu/exec_graph.cc:106-108). */
int es_km_scalarop_simplify(const char* text, const char* const* var_names,
                            const double* var_values, int n_vars, char* out, size_t cap);
int es_km_merge_adjacent_dims(const uint64_t* join_shape, int join_rank, const int* inns_flat,
                              const int* inns_offsets, int n_inns, int out_rank,
                              const char* join_text, char castable, uint64_t* new_join_shape,
                              int* new_inns_flat, int* new_inns_offsets, int* new_out_rank,
                              char* str_out, size_t str_cap);

/* Measurement aid (no counterpart in the reference): fp16 matrix-core throughput in TFLOP/s
 * with register-resident operands -- `blocks` workgroups of 4 wavefronts each issue
 * 8 * iters v_mfma_f32_32x32x16_f16.  operands: 8 KiB on the device (their bit patterns set
 * the power draw, hence the clock); scratch: blocks * 1 KiB on the device.  Synchronises the
 * stream.  Negative on error. */
double es_km_probe_mfma_f16(es_km_t* km, const void* operands, void* scratch, int blocks, int iters,
                            void* stream);

/* ---------------------------------------------------------------------------------------
 * Exec-node layer: a dependency graph of apply / fill / copy nodes over ONE device arena.
 *
 * Replaces, for one GPU, the reference's GPU exec graph and its node types
 *   exec_graph_t::insert / node_t                   src/engine/exec_graph.h:53-80
 *   gpu_einsummable_t::launch                       src/engine/gpu/exec_graph.cc:276-332
 *   gpu_touch_t::launch (group semantics)           src/engine/gpu/exec_graph.cc:354-404
 *   gpu_constant_t / gpu_lowerTri_t / gpu_copy_t    src/engine/gpu/exec_nodes.h:112-160
 *   streampool_manager_t, group_manager_t           src/engine/gpu/stream_pool.cc,
 *                                                   src/engine/managers.cc:3-21
 * Memory ranges are (offset, size) into the arena passed to run (mem_t, memgraph.h:44-60;
 * mems[0] is the output, memgraph.h:252-263).  A node may only depend on nodes added before
 * it: insertion order is the launch order.  Where the reference reports every node's
 * completion to a host event loop through a stream callback, finalize fixes the order and
 * the stream of every node once and run enqueues everything, cross-stream dependencies as
 * event waits on the device; nothing synchronises with the host.  A graph finalized on one
 * stream may be captured into a HIP graph; do not capture a multi-stream run (the fork /
 * join of pool streams inside a capture crashed the HIP runtime of ROCm 7.2).
 * `add_*` return the node id (>= 0) or a negative error code.
 * Touches: group < 0 makes the touch a copy (exec_graph.cc:176-181); touches of one group
 * run in insertion order and the first has its castable cleared (exec_graph.cc:368-378).
 * es_km_graph_create(NULL) gives a graph that can be planned and inspected but not run. */
typedef struct es_km_graph es_km_graph_t;

es_km_graph_t* es_km_graph_create(es_km_t* km);
void           es_km_graph_destroy(es_km_graph_t* g);

int es_km_graph_add_einsummable(es_km_graph_t* g, const uint64_t* join_shape, int join_rank,
                                const int* inns_flat, const int* inns_offsets, int n_inns,
                                int out_rank, const char* join_text, char castable,
                                const uint64_t* mem_offsets, const uint64_t* mem_sizes, int n_mems,
                                const int* deps, int n_deps);
int es_km_graph_add_touch(es_km_graph_t* g, const uint64_t* touchdims, int rank, char castable,
                          int dtype, int group, const uint64_t* mem_offsets,
                          const uint64_t* mem_sizes, const int* deps, int n_deps);
int es_km_graph_add_fill_constant(es_km_graph_t* g, int dtype, uint64_t value_bits,
                                  uint64_t nelem, uint64_t offset, uint64_t size, const int* deps,
                                  int n_deps);
int es_km_graph_add_fill_lowertri(es_km_graph_t* g, int dtype, uint64_t lower_bits,
                                  uint64_t upper_bits, uint64_t nrow, uint64_t ncol, int64_t start,
                                  uint64_t offset, uint64_t size, const int* deps, int n_deps);
int es_km_graph_add_copy(es_km_graph_t* g, uint64_t dst_offset, uint64_t src_offset, uint64_t size,
                         const int* deps, int n_deps);

/* Adds the dependencies the nodes' memory ranges imply (read after write, write after
 * write, write after read), for callers that hold no explicit edge list. */
int es_km_graph_add_memory_dependencies(es_km_graph_t* g);

/* Optional, before finalize: removes round trips through memory that change no stored bit.
 * A touch that copies a whole range which one einsummable wrote and nobody else reads (the
 * formation copy behind every contraction and reduction, src/einsummable/taskgraph.cc:
 * 3047-3061) is dropped and the einsummable writes the copy's output.  An elementwise
 * einsummable whose output is read only by elementwise einsummables (or reductions of one
 * input) that take it position by position is computed by each of those readers instead: a
 * reader becomes one einsummable with both joins, the inner value rounded as the store
 * between them rounded it.  With several readers that is taken while the producer's inputs are
 * smaller than the traffic its output caused; a sum is only merged when its order of addition
 * stays what it was.  Both need the range's del node (memgraph.h: del_t) in the graph, as a
 * dummy that covers the range and depends on its last reader: without it the range counts as
 * a result and stays.  Last, a chain over rows -- row reductions, pointwise steps on their
 * per-row results and the elementwise node that uses them, over the same rows, with every
 * intermediate result deleted afterwards (softmax: row max, sum of exp(x - max), the
 * quotient) -- becomes one launch that reads each row once and writes it once; the last
 * node's output keeps its bits (ES_KM_ROW_CHAINS=0 in the environment leaves chains alone).
 * A conversion to f32 whose output a complex node reads as c64, and a conversion to f16 of
 * what a complex node wrote (rotary embeddings: to_f32, product on the buffer seen as c64,
 * to_f16), go into the complex node, which then reads and writes pairs of f16.
 * Node ids stay valid: an absorbed node becomes a dummy.  *n_absorbed
 * (may be null) receives how many were absorbed.  No counterpart in the reference, whose
 * engine launches the nodes as the memgraph lists them. */
int es_km_graph_optimize(es_km_graph_t* g, int* n_absorbed);

/* Builds every einsummable (an unsupported one is an error here), places the nodes on
 * n_streams (1..16) streams.  The graph is immutable afterwards. */
int es_km_graph_finalize(es_km_graph_t* g, int n_streams);

/* Enqueues the whole graph: ordered after what `stream` holds at the call, and `stream` is
 * ordered after all of it on return.  Calls on one graph must not overlap in time. */
int es_km_graph_run(es_km_graph_t* g, void* stream, void* arena);

/* After finalize: launch position, stream index and dependencies of a node (deps receives
 * at most cap ids, *n_deps the full count); number of event waits one run enqueues. */
int es_km_graph_node_info(es_km_graph_t* g, int id, int* position, int* stream, int* deps, int cap,
                          int* n_deps);
int es_km_graph_cross_stream_waits(es_km_graph_t* g);
/* Any time: a node as text, "<kind> <offset>:<size> ..." (the output range first) and, for an
 * einsummable, " | [join shape]castable modes->out rank | join" (the join in the text form of
 * scalarop's operator<<, src/einsummable/scalarop.cc:2881-3011).  Writes at most cap-1
 * characters and a terminator; returns the full length, negative for a bad id. */
int64_t es_km_graph_node_describe(es_km_graph_t* g, int id, char* out, uint64_t cap);
/* Test aid, like es_km_codegen_source: the HIP source of the generated kernel of a node (an
 * elementwise or reduction einsummable, what es_km_graph_optimize merged included, or a chain
 * over rows), empty for any other node; with `compile` it is also compiled for gfx950 (no
 * device needed).  Returns the full length, negative on an error (a failed compile:
 * ES_KM_ERR_DEVICE, text in es_km_last_error of the graph's manager, or of NULL).  No
 * counterpart in the reference. */
int64_t es_km_graph_node_source(es_km_graph_t* g, int id, int compile, char* out, uint64_t cap);
/* After finalize: launches one run makes.  Touches of one group that follow each other in
 * insertion order and write the same output range count once: they run as one
 * es_km_touch_batch launch, with the bytes of one launch per touch
 * (src/engine/gpu/exec_graph.cc:354-404 issues them one by one). */
int es_km_graph_launches(es_km_graph_t* g);

/* One node at a time, for a host event loop that keeps the dependencies itself.
 *   gpu_einsummable_t::launch(resources, callback)   src/engine/gpu/exec_graph.cc:277-335
 *   gpu_touch_t::launch (first-in-group decided by the group manager at run time)
 *                                                    src/engine/gpu/exec_graph.cc:354-404,
 *                                                    src/engine/managers.cc:3-21
 *   gpu_constant_t / gpu_lowerTri_t / gpu_copy_t / gpu_evict_t / gpu_load_t ::launch
 *                                                    src/engine/gpu/exec_graph.cc:600-690, 482-577
 * Enqueues node `id` of a finalized graph on `stream` -- no waits and no events: the caller
 * launches a node once every node it depends on (es_km_graph_node_info) has called back --
 * followed on the same stream by a host function (hipLaunchHostFunc; the reference uses
 * cudaStreamAddCallback) that calls callback(user) when the node's work is done.  The
 * callback runs on a thread of the HIP runtime and must not call the HIP API; NULL asks for
 * none.  workspace: at least es_km_graph_node_workspace(id) bytes, from the caller's pool,
 * ignored by nodes that need none.  first_in_group, for a touch in a group: 1 clears its
 * castable (the first touch of a group to run initialises the output), 0 keeps the castable
 * it was added with, -1 takes what insertion order said (the first member inserted). */
typedef void (*es_km_callback_t)(void* user);
int es_km_graph_launch_node(es_km_graph_t* g, int id, void* stream, void* arena, void* workspace,
                            uint64_t workspace_bytes, int first_in_group,
                            es_km_callback_t callback, void* user);
int es_km_graph_node_workspace(es_km_graph_t* g, int id, uint64_t* workspace_bytes);
int es_km_graph_node_group(es_km_graph_t* g, int id);   /* the touch's group, or -1 */

/* The resource pools such an event loop draws from.
 *   gpu_workspace_manager_t: the first free block that is large enough, else a new device
 *     allocation; released blocks are kept for reuse and freed with the pool
 *                                                    src/engine/gpu/workspace.cc:48-91
 *   streampool_t / streampool_manager_t: a fixed set of streams, try-acquire hands out a
 *     free one or nothing                            src/engine/gpu/stream_pool.cc:8-75
 * Both are safe to use from several threads. */
typedef struct es_km_workspace_pool es_km_workspace_pool_t;
typedef struct es_km_stream_pool    es_km_stream_pool_t;
es_km_workspace_pool_t* es_km_workspace_pool_create(int device);
void                    es_km_workspace_pool_destroy(es_km_workspace_pool_t* p);
/* NULL on failure (es_km_last_error(NULL)); *got_bytes receives the block's real size */
void* es_km_workspace_pool_acquire(es_km_workspace_pool_t* p, uint64_t bytes, uint64_t* got_bytes);
int   es_km_workspace_pool_release(es_km_workspace_pool_t* p, void* block);
int   es_km_workspace_pool_blocks(es_km_workspace_pool_t* p);
es_km_stream_pool_t* es_km_stream_pool_create(int device, int n_streams);
void                 es_km_stream_pool_destroy(es_km_stream_pool_t* p);
void* es_km_stream_pool_try_acquire(es_km_stream_pool_t* p);   /* a hipStream_t, or NULL */
int   es_km_stream_pool_release(es_km_stream_pool_t* p, void* stream);

/* Nodes that launch nothing and only carry dependencies (dummy_t, which the reference makes
 * of inputmem / inputsto / partialize / alloc / del nodes, src/engine/gpu/exec_graph.cc:94-97).
 * The range is kept for inspection and takes no part in add_memory_dependencies. */
int es_km_graph_add_dummy(es_km_graph_t* g, uint64_t offset, uint64_t size, const int* deps,
                          int n_deps);
/* add_dummy with a non-empty range is how a caller spells a del (memgraph.h: del_t): it is
 * what lets es_km_graph_optimize drop the range.  add_placeholder names a range without
 * deleting it -- what the memgraph loader makes of inputmem / alloc / partialize nodes, whose
 * ranges hold or will hold data (gpu/exec_graph.cc:94-97 makes dummy_t of all of them alike;
 * only this library's optimize() needs to tell them apart). */
int es_km_graph_add_placeholder(es_km_graph_t* g, uint64_t offset, uint64_t size, const int* deps,
                                int n_deps);

/* Host storage: gpu_evict_t::launch / gpu_load_t::launch, src/engine/gpu/exec_graph.cc:482-577
 * (memgraph_t::evict_t / load_t, src/einsummable/memgraph.h:306-325).  evict copies an arena
 * range to the storage slot `storage_id`, load copies the slot to an arena range; both are
 * asynchronous copies on the node's stream.  A slot is a pinned host buffer the graph
 * allocates at finalize, sized for its largest user (the reference allocates one per evict
 * and frees it after the load, storage_manager.h).  declare_storage announces a slot the
 * caller fills itself (an inputsto node, memgraph.h:222-228); storage_write / storage_read
 * are host copies, valid after finalize, which the caller orders against run. */
int es_km_graph_add_evict(es_km_graph_t* g, uint64_t offset, uint64_t size, int storage_id,
                          const int* deps, int n_deps);
int es_km_graph_add_load(es_km_graph_t* g, int storage_id, uint64_t offset, uint64_t size,
                         const int* deps, int n_deps);
int es_km_graph_declare_storage(es_km_graph_t* g, int storage_id, uint64_t size);
int es_km_graph_storage_write(es_km_graph_t* g, int storage_id, const void* src, uint64_t size);
int es_km_graph_storage_read(es_km_graph_t* g, int storage_id, void* dst, uint64_t size);

/* memgraph_t::from_wire (src/einsummable/memgraph.cc:381-480) followed by what
 * exec_graph_t::make_gpu_exec_graph does with the result (src/engine/gpu/exec_graph.cc:26-245):
 * `bytes` is a serialized MemGraph message (src/proto/einsummable.proto:233-238, as written by
 * memgraph_t::to_wire, memgraph.cc:258-379); every node of it becomes one node of the empty
 * graph `g`, with the same id, for compute location `loc`:
 *   inputmem, inputsto, partialize, alloc, del, nodes of other locations -> dummy
 *   apply -> einsummable (scalar variables named in var_names replaced by var_values first,
 *            exec_graph.cc:108-110) or touch with its group
 *   constant -> constant / lowertri fill;  copy, move within `loc` -> copy
 *   evict, load -> host storage;  inputsto read here -> declared storage slot
 * A move between two locations is an error (one process drives one device).  A lowertri
 * fill has nrow and ncol exchanged, as the reference's reader leaves them
 * (src/einsummable/fill.cc:137-143).  Returns the number of nodes or a negative error;
 * finalize and run the graph as usual. */
int es_km_graph_load_memgraph(es_km_graph_t* g, const void* bytes, uint64_t size, int loc,
                              const char* const* var_names, const double* var_values, int n_vars);

/* Inspection: node count, the smallest arena holding every range, and a node's kind
 * (0 einsummable, 1 touch, 2 constant fill, 3 lowertri fill, 4 copy, 5 dummy, 6 evict,
 * 7 load, 8 a chain over rows that es_km_graph_optimize made) and ranges (for a dummy made of
 * an inputmem: where the caller puts that input). */
int      es_km_graph_num_nodes(es_km_graph_t* g);
uint64_t es_km_graph_arena_bytes(es_km_graph_t* g);
int es_km_graph_node_mems(es_km_graph_t* g, int id, int* kind, uint64_t* offsets, uint64_t* sizes,
                          int cap, int* n_mems);

/* Diagnostics without a device: decodes a serialized MemGraph and writes one line per node
 * with every decoded field into `out` (at most cap bytes, NUL-terminated).  Returns the
 * full length of the text or a negative error (message via es_km_last_error(NULL)). */
int64_t es_km_memgraph_describe(const void* bytes, uint64_t size, char* out, uint64_t cap);

#ifdef __cplusplus
}
#endif
#endif
