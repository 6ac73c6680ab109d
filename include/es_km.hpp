// es_km.hpp -- header-only C++ face of the C ABI in es_km.h with the member names, argument
// meaning and error behaviour of the reference's kernel_manager_t
// (src/engine/gpu/gpu_kernel_manager.h:274-321):
//
//   optional<workspace_info_t> build(einsummable_t const&)   nullopt when unsupported
//   workspace_info_t workspace_size(einsummable_t const&)    throws if not built
//   operator()(einsummable_t, stream, out, inns, workspace)  throws std::runtime_error on a
//                                                            missing build, a wrong input
//                                                            count or a short workspace
//   operator()(touch_t, stream, out, inn)
//   constant_fill / lowerTri_fill
//
// The descriptor structs carry the same fields as the reference's einsummable_t
// (src/einsummable/einsummable.h:8-20), touch_t (touch.h:8-29) and fill_t (fill.h:11-30); the
// join travels as the text `operator<<(ostream&, scalarop_t)` writes.  Inside the reference
// tree the adapter is three lines per call: flatten `inns`, print `join` and the castable
// with write_with_ss, forward to the C entry point.
#pragma once
#include "es_km.h"

#include <complex>
#include <cstring>
#include <map>
#include <optional>
#include <stdexcept>
#include <string>
#include <tuple>
#include <vector>

namespace eskm
{

enum class dtype_t { f16 = ES_KM_F16, f32 = ES_KM_F32, f64 = ES_KM_F64, c64 = ES_KM_C64 };
enum class castable_t { add, mul, min, max };

inline char castable_char(std::optional<castable_t> const& c)
{
    if (!c) return 0;
    switch (c.value()) {
        case castable_t::add:
            return '+';
        case castable_t::mul:
            return 'x';
        case castable_t::min:
            return 'v';
        case castable_t::max:
            return '^';
    }
    return 0;
}

// scalar_t (src/einsummable/scalarop.h:24-75): a dtype and eight raw bytes
struct scalar_t {
    dtype_t dtype = dtype_t::f32;
    uint8_t data[8] = {0, 0, 0, 0, 0, 0, 0, 0};

    scalar_t() = default;
    explicit scalar_t(float v) : dtype(dtype_t::f32) { std::memcpy(data, &v, 4); }
    explicit scalar_t(double v) : dtype(dtype_t::f64) { std::memcpy(data, &v, 8); }
    explicit scalar_t(std::complex<float> v) : dtype(dtype_t::c64) { std::memcpy(data, &v, 8); }
    static scalar_t from_f16_bits(uint16_t bits)
    {
        scalar_t s;
        s.dtype = dtype_t::f16;
        std::memcpy(s.data, &bits, 2);
        return s;
    }
    uint64_t bits() const
    {
        uint64_t b;
        std::memcpy(&b, data, 8);
        return b;
    }
};

struct einsummable_t {
    std::vector<uint64_t>         join_shape;
    std::vector<std::vector<int>> inns;
    int                           out_rank;
    std::string                   join;  // scalarop text
    std::optional<castable_t>     castable;

    // from_matmul (src/einsummable/einsummable.cc:307-323): ij,jk->ik
    static einsummable_t from_matmul(uint64_t di, uint64_t dj, uint64_t dk, dtype_t d)
    {
        static const char* names[] = {"f16", "f32", "f64", "c64"};
        std::string        n = names[int(d)];
        return einsummable_t{{di, dk, dj},
                             {{0, 2}, {2, 1}},
                             2,
                             "*[hole|" + n + "@0,hole|" + n + "@1]",
                             castable_t::add};
    }
};

struct touchdim_t {
    uint64_t d_inn, d_out, offset_inn, offset_out, size;
};

struct touch_t {
    std::vector<touchdim_t>   selection;
    std::optional<castable_t> castable;
    dtype_t                   dtype;
};

struct fill_t {
    struct constant_t {
        scalar_t              value;
        std::vector<uint64_t> shape;
    };
    struct lowertri_t {
        scalar_t lower, upper;
        uint64_t nrow, ncol;
        int64_t  start;
    };
};

struct workspace_info_t {
    workspace_info_t() {}
    workspace_info_t(uint64_t sz) : workspace_size(sz) {}
    std::optional<uint64_t> workspace_size;
    uint64_t const&         value() const { return workspace_size.value(); }
    bool                    known() const { return bool(workspace_size); }
};

class kernel_manager_t
{
public:
    explicit kernel_manager_t(int device = 0) : h_(es_km_create(device))
    {
        if (!h_) throw std::runtime_error(std::string("kernel_manager_t: ") + es_km_last_error(nullptr));
    }
    ~kernel_manager_t() { es_km_destroy(h_); }
    kernel_manager_t(kernel_manager_t const&) = delete;
    kernel_manager_t& operator=(kernel_manager_t const&) = delete;

    std::optional<workspace_info_t> build(einsummable_t const& e)
    {
        flat_t   f(e);
        uint64_t ws = 0;
        int rc = es_km_build(h_, e.join_shape.data(), int(e.join_shape.size()), f.flat.data(),
                             f.offs.data(), int(e.inns.size()), e.out_rank, e.join.c_str(),
                             castable_char(e.castable), &ws);
        if (rc == ES_KM_UNSUPPORTED) return std::nullopt;
        check(rc);
        return workspace_info_t(ws);
    }

    workspace_info_t workspace_size(einsummable_t const& e) const
    {
        flat_t   f(e);
        uint64_t ws = 0;
        check(es_km_workspace_size(h_, e.join_shape.data(), int(e.join_shape.size()),
                                   f.flat.data(), f.offs.data(), int(e.inns.size()), e.out_rank,
                                   e.join.c_str(), castable_char(e.castable), &ws));
        return workspace_info_t(ws);
    }

    void operator()(touch_t const& touch, void* stream, void* out, void const* inn) const
    {
        static_assert(sizeof(touchdim_t) == 5 * sizeof(uint64_t), "touchdim_t must be packed");
        check(es_km_touch(h_, reinterpret_cast<uint64_t const*>(touch.selection.data()),
                          int(touch.selection.size()), castable_char(touch.castable),
                          int(touch.dtype), stream, out, inn));
    }

    void operator()(einsummable_t const& e, void* stream, void* out,
                    std::vector<void const*>                    inns,
                    std::optional<std::tuple<void*, uint64_t>> workspace = std::nullopt) const
    {
        flat_t f(e);
        check(es_km_execute(h_, e.join_shape.data(), int(e.join_shape.size()), f.flat.data(),
                            f.offs.data(), int(e.inns.size()), e.out_rank, e.join.c_str(),
                            castable_char(e.castable), stream, out, inns.data(), int(inns.size()),
                            workspace ? std::get<0>(workspace.value()) : nullptr,
                            workspace ? std::get<1>(workspace.value()) : 0));
    }

    // The same call for places that must not allocate (under HIP graph capture, in a serving
    // loop): the kernel's scratch comes from the library's static device array instead of a
    // workspace argument (es_km_execute_static_workspace); needs beyond
    // ES_KM_STATIC_WORKSPACE_BYTES are refused.
    void execute_static_workspace(einsummable_t const& e, void* stream, void* out,
                                  std::vector<void const*> inns) const
    {
        flat_t f(e);
        check(es_km_execute_static_workspace(
            h_, e.join_shape.data(), int(e.join_shape.size()), f.flat.data(), f.offs.data(),
            int(e.inns.size()), e.out_rank, e.join.c_str(), castable_char(e.castable), stream, out,
            inns.data(), int(inns.size())));
    }

    void lowerTri_fill(fill_t::lowertri_t const& l, void* stream, void* out) const
    {
        check(es_km_fill_lowertri(h_, int(l.lower.dtype), l.lower.bits(), l.upper.bits(), l.nrow,
                                  l.ncol, l.start, stream, out));
    }

    void constant_fill(fill_t::constant_t const& c, void* stream, void* out) const
    {
        uint64_t n = 1;
        for (uint64_t d : c.shape) n *= d;
        check(es_km_fill_constant(h_, int(c.value.dtype), c.value.bits(), n, stream, out));
    }

private:
    struct flat_t {
        std::vector<int> flat, offs;
        explicit flat_t(einsummable_t const& e)
        {
            offs.push_back(0);
            for (auto const& inn : e.inns) {
                flat.insert(flat.end(), inn.begin(), inn.end());
                offs.push_back(int(flat.size()));
            }
        }
    };

    void check(int rc) const
    {
        if (rc != ES_KM_OK) {
            throw std::runtime_error(std::string("kernel_manager_t: ") + es_km_last_error(h_));
        }
    }

    es_km_t* h_;
    friend class exec_graph_t;
};

// mem_t of the memgraph (src/einsummable/memgraph.h:44-60): a byte range of the arena
struct mem_t {
    uint64_t offset, size;
};

// The exec-node layer: what exec_graph_t::make_gpu_exec_graph builds out of a memgraph's
// apply / constant / copy nodes (src/engine/gpu/exec_graph.cc:60-256) and what
// exec_state_t::event_loop then drives (src/engine/exec_state.cc).  insert_* mirror the op
// types of src/engine/gpu/exec_nodes.h; `inns` are the ids of the nodes to wait for, as in
// exec_graph_t::insert (src/engine/exec_graph.h:53).
class exec_graph_t
{
public:
    explicit exec_graph_t(kernel_manager_t& km) : km_(km), g_(es_km_graph_create(km.h_))
    {
        if (!g_) throw std::runtime_error("exec_graph_t: could not create the graph");
    }
    ~exec_graph_t() { es_km_graph_destroy(g_); }
    exec_graph_t(exec_graph_t const&) = delete;
    exec_graph_t& operator=(exec_graph_t const&) = delete;

    // gpu_einsummable_t: mems[0] is the output
    int insert_einsummable(einsummable_t const& e, std::vector<mem_t> const& mems,
                           std::vector<int> const& inns = {})
    {
        std::vector<int> flat, offs{0};
        for (auto const& inn : e.inns) {
            flat.insert(flat.end(), inn.begin(), inn.end());
            offs.push_back(int(flat.size()));
        }
        std::vector<uint64_t> mo, ms;
        split(mems, mo, ms);
        return id(es_km_graph_add_einsummable(
            g_, e.join_shape.data(), int(e.join_shape.size()), flat.data(), offs.data(),
            int(e.inns.size()), e.out_rank, e.join.c_str(), castable_char(e.castable), mo.data(),
            ms.data(), int(mems.size()), inns.data(), int(inns.size())));
    }
    // gpu_touch_t: group < 0 makes it a copy, the first touch of a group initialises
    int insert_touch(touch_t const& t, int group, mem_t out, mem_t inn,
                     std::vector<int> const& inns = {})
    {
        uint64_t mo[2] = {out.offset, inn.offset}, ms[2] = {out.size, inn.size};
        return id(es_km_graph_add_touch(
            g_, reinterpret_cast<uint64_t const*>(t.selection.data()), int(t.selection.size()),
            castable_char(t.castable), int(t.dtype), group, mo, ms, inns.data(), int(inns.size())));
    }
    // gpu_constant_t / gpu_lowerTri_t
    int insert_constant(fill_t::constant_t const& c, mem_t out, std::vector<int> const& inns = {})
    {
        uint64_t n = 1;
        for (uint64_t d : c.shape) n *= d;
        return id(es_km_graph_add_fill_constant(g_, int(c.value.dtype), c.value.bits(), n,
                                                out.offset, out.size, inns.data(),
                                                int(inns.size())));
    }
    int insert_lowertri(fill_t::lowertri_t const& l, mem_t out, std::vector<int> const& inns = {})
    {
        return id(es_km_graph_add_fill_lowertri(g_, int(l.lower.dtype), l.lower.bits(),
                                                l.upper.bits(), l.nrow, l.ncol, l.start, out.offset,
                                                out.size, inns.data(), int(inns.size())));
    }
    // gpu_copy_t within the device
    int insert_copy(mem_t dst, mem_t src, std::vector<int> const& inns = {})
    {
        if (dst.size != src.size) throw std::runtime_error("exec_graph_t: copy sizes differ");
        return id(es_km_graph_add_copy(g_, dst.offset, src.offset, dst.size, inns.data(),
                                       int(inns.size())));
    }
    // dummy_t: launches nothing, only orders (inputmem / partialize / alloc / del nodes).
    // With a range it stands for the range's del unless is_del is false (the range of an
    // input or an alloc: optimize() never drops what is stored there).
    int insert_dummy(mem_t range = {0, 0}, std::vector<int> const& inns = {}, bool is_del = true)
    {
        auto const add = is_del ? es_km_graph_add_dummy : es_km_graph_add_placeholder;
        return id(add(g_, range.offset, range.size, inns.data(), int(inns.size())));
    }
    // gpu_evict_t / gpu_load_t: arena range <-> host storage slot
    int insert_evict(mem_t src, int storage_id, std::vector<int> const& inns = {})
    {
        return id(es_km_graph_add_evict(g_, src.offset, src.size, storage_id, inns.data(),
                                        int(inns.size())));
    }
    int insert_load(int storage_id, mem_t dst, std::vector<int> const& inns = {})
    {
        return id(es_km_graph_add_load(g_, storage_id, dst.offset, dst.size, inns.data(),
                                       int(inns.size())));
    }
    void storage_write(int storage_id, void const* src, uint64_t size)
    {
        check(es_km_graph_storage_write(g_, storage_id, src, size));
    }
    void storage_read(int storage_id, void* dst, uint64_t size) const
    {
        check(es_km_graph_storage_read(g_, storage_id, dst, size));
    }
    // memgraph_t::from_wire + make_gpu_exec_graph for compute location `loc`: every node of
    // the serialized memgraph becomes the node of the same id (the graph must be empty)
    int load_memgraph(std::string const& wire, int loc = 0,
                      std::map<std::string, double> const& scalar_vars = {})
    {
        std::vector<char const*> names;
        std::vector<double>      values;
        for (auto const& kv : scalar_vars) {
            names.push_back(kv.first.c_str());
            values.push_back(kv.second);
        }
        return id(es_km_graph_load_memgraph(g_, wire.data(), wire.size(), loc, names.data(),
                                            values.data(), int(names.size())));
    }
    uint64_t arena_bytes() const { return es_km_graph_arena_bytes(g_); }
    void add_memory_dependencies() { check(es_km_graph_add_memory_dependencies(g_)); }
    void finalize(int n_streams) { check(es_km_graph_finalize(g_, n_streams)); }
    // optional, before finalize: absorbs whole-range copies into their producers and
    // single-reader elementwise nodes into their readers; returns how many nodes went
    int optimize()
    {
        int n = 0;
        check(es_km_graph_optimize(g_, &n));
        return n;
    }
    // the whole graph, ordered after and before `stream`; no host synchronisation
    void run(void* stream, void* arena) const { check(es_km_graph_run(g_, stream, arena)); }

    // One node at a time, for a host event loop that keeps the dependencies itself
    // (gpu_einsummable_t::launch / gpu_touch_t::launch with a callback,
    // src/engine/gpu/exec_graph.cc:277-335, 354-404): enqueues node `id` on `stream` and,
    // behind it, a host function that calls callback(user) when the node is done.
    void launch(int id, void* stream, void* arena, void* workspace, uint64_t workspace_bytes,
                es_km_callback_t callback, void* user, int first_in_group = -1) const
    {
        check(es_km_graph_launch_node(g_, id, stream, arena, workspace, workspace_bytes,
                                      first_in_group, callback, user));
    }
    uint64_t node_workspace(int id) const
    {
        uint64_t ws = 0;
        check(es_km_graph_node_workspace(g_, id, &ws));
        return ws;
    }
    int node_group(int id) const { return es_km_graph_node_group(g_, id); }
    // dependencies of a node (own and implied), after finalize
    std::vector<int> node_deps(int id) const
    {
        int pos = 0, st = 0, n = 0;
        check(es_km_graph_node_info(g_, id, &pos, &st, nullptr, 0, &n));
        std::vector<int> deps(size_t(n), 0);
        if (n) check(es_km_graph_node_info(g_, id, &pos, &st, deps.data(), n, &n));
        return deps;
    }
    int n_launches() const { return es_km_graph_launches(g_); }

private:
    static void split(std::vector<mem_t> const& m, std::vector<uint64_t>& o,
                      std::vector<uint64_t>& s)
    {
        for (auto const& x : m) {
            o.push_back(x.offset);
            s.push_back(x.size);
        }
    }
    int id(int rc) const
    {
        if (rc < 0) check(rc);
        return rc;
    }
    void check(int rc) const
    {
        if (rc < 0) {
            throw std::runtime_error(std::string("exec_graph_t: ") + es_km_last_error(km_.h_));
        }
    }
    kernel_manager_t& km_;
    es_km_graph_t*    g_;
};

// The workspace pool of src/engine/gpu/workspace.cc:48-91 (first block that is large enough,
// else a new allocation) and the stream pool of src/engine/gpu/stream_pool.cc, for callers of
// exec_graph_t::launch.
class workspace_pool_t
{
public:
    explicit workspace_pool_t(int device) : p_(es_km_workspace_pool_create(device))
    {
        if (!p_) throw std::runtime_error(std::string("workspace_pool_t: ") + es_km_last_error(nullptr));
    }
    ~workspace_pool_t() { es_km_workspace_pool_destroy(p_); }
    workspace_pool_t(workspace_pool_t const&) = delete;
    workspace_pool_t& operator=(workspace_pool_t const&) = delete;
    // a block of at least `bytes` (its real size in *got), or nullptr with bytes == 0
    void* acquire(uint64_t bytes, uint64_t* got = nullptr)
    {
        uint64_t g = 0;
        void*    b = es_km_workspace_pool_acquire(p_, bytes, &g);
        if (!b && bytes) throw std::runtime_error(std::string("workspace_pool_t: ") + es_km_last_error(nullptr));
        if (got) *got = g;
        return b;
    }
    void release(void* block) { es_km_workspace_pool_release(p_, block); }
    int  blocks() const { return es_km_workspace_pool_blocks(p_); }

private:
    es_km_workspace_pool_t* p_;
};

class stream_pool_t
{
public:
    stream_pool_t(int device, int n_streams) : p_(es_km_stream_pool_create(device, n_streams))
    {
        if (!p_) throw std::runtime_error(std::string("stream_pool_t: ") + es_km_last_error(nullptr));
    }
    ~stream_pool_t() { es_km_stream_pool_destroy(p_); }
    stream_pool_t(stream_pool_t const&) = delete;
    stream_pool_t& operator=(stream_pool_t const&) = delete;
    void* try_acquire() { return es_km_stream_pool_try_acquire(p_); }  // nullptr: all in use
    void  release(void* stream) { es_km_stream_pool_release(p_, stream); }

private:
    es_km_stream_pool_t* p_;
};

}  // namespace eskm
