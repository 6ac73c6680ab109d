// extern "C" surface of the kernel manager (see include/es_km.h).  Converts the flat
// descriptor arguments into IR values, forwards to es::kernel_manager_t and maps exceptions to
// return codes.
#include "../../include/es_km.h"

#include "codegen.h"
#include "exec_graph.h"
#include "memgraph_wire.h"
#include "gemm_kernel.h"
#include "kernel_manager.h"
#include "pools.h"
#include "static_workspace.h"

#include <cstring>

struct es_km {
    std::unique_ptr<es::kernel_manager_t> km;
    std::string                           last_error;
};

struct es_km_workspace_pool {
    es::workspace_pool_t pool;
    explicit es_km_workspace_pool(int device) : pool(device) {}
};

struct es_km_stream_pool {
    es::stream_pool_t pool;
    es_km_stream_pool(int device, int n) : pool(device, n) {}
};

struct es_km_graph {
    es_km_t*                            owner;  // may be null (plan-only graph)
    std::unique_ptr<es::apply_graph_t> graph;
};

namespace
{

thread_local std::string g_null_error;

std::string& err_slot(es_km_t* h) { return h ? h->last_error : g_null_error; }

// Key of the descriptor exactly as passed by the caller; cheap to build on the hot path.
std::string raw_key(const uint64_t* join_shape, int join_rank, const int* inns_flat,
                    const int* inns_offsets, int n_inns, int out_rank, const char* join_text,
                    char castable)
{
    std::string k;
    k.reserve(96 + std::strlen(join_text));
    k.append(reinterpret_cast<const char*>(join_shape), sizeof(uint64_t) * size_t(join_rank));
    k.push_back('|');
    k.append(reinterpret_cast<const char*>(inns_offsets), sizeof(int) * size_t(n_inns + 1));
    k.append(reinterpret_cast<const char*>(inns_flat), sizeof(int) * size_t(inns_offsets[n_inns]));
    k.push_back('|');
    k.push_back(char('0' + out_rank));
    k.push_back(castable ? castable : ':');
    k.append(join_text);
    return k;
}

void check_descriptor(const uint64_t* join_shape, int join_rank, const int* inns_flat,
                      const int* inns_offsets, int n_inns, int out_rank, const char* join_text)
{
    if (!join_shape || !inns_flat || !inns_offsets || !join_text) {
        throw es::ir_error("einsummable descriptor: null argument");
    }
    if (join_rank < 1 || join_rank > 32 || n_inns < 1 || n_inns > 32 || out_rank < 1) {
        throw es::ir_error("einsummable descriptor: bad rank or input count");
    }
    if (inns_offsets[0] != 0) throw es::ir_error("einsummable descriptor: inns_offsets[0] != 0");
    for (int k = 0; k != n_inns; ++k) {
        if (inns_offsets[k + 1] < inns_offsets[k] || inns_offsets[k + 1] > 1024) {
            throw es::ir_error("einsummable descriptor: inns_offsets not monotone");
        }
    }
}

es::einsummable_t make_einsummable(const uint64_t* join_shape, int join_rank,
                                   const int* inns_flat, const int* inns_offsets, int n_inns,
                                   int out_rank, const char* join_text, char castable)
{
    std::vector<uint64_t>         shape(join_shape, join_shape + join_rank);
    std::vector<std::vector<int>> inns;
    for (int k = 0; k != n_inns; ++k) {
        inns.emplace_back(inns_flat + inns_offsets[k], inns_flat + inns_offsets[k + 1]);
    }
    return es::einsummable_t::make(std::move(shape), std::move(inns), out_rank,
                                   es::scalarop_t::parse(join_text),
                                   es::castable_from_char(castable));
}

template <typename F>
int guarded(es_km_t* h, F&& f)
{
    try {
        return f();
    } catch (es::km_error const& e) {
        err_slot(h) = e.what();
        return int(e.status);
    } catch (es::ir_error const& e) {
        err_slot(h) = e.what();
        return ES_KM_ERR_INVALID;
    } catch (std::exception const& e) {
        err_slot(h) = e.what();
        return ES_KM_ERR_DEVICE;
    }
}

// One line per node, every decoded field in a fixed order.
std::string describe_memgraph(es::memgraph_t const& mg)
{
    auto u = [](uint64_t v) { return std::to_string(v); };
    auto list = [&](auto const& xs) {
        std::string s = "[";
        for (size_t i = 0; i != xs.size(); ++i) s += (i ? "," : "") + std::to_string(xs[i]);
        return s + "]";
    };
    std::string out = "memgraph compute_locs=" + std::to_string(mg.num_compute_locs) +
                      " storage_locs=" + std::to_string(mg.num_storage_locs) + " map=" +
                      list(mg.storage_locs) + " nodes=" + std::to_string(mg.nodes.size()) + "\n";
    for (size_t id = 0; id != mg.nodes.size(); ++id) {
        es::mg_node_t const& n = mg.nodes[id];
        out += std::to_string(id) + " kind=" + std::to_string(int(n.kind)) +
               " loc=" + std::to_string(n.loc) + " src_loc=" + std::to_string(n.src_loc) +
               " offset=" + u(n.offset) + " size=" + u(n.size) + " src_offset=" + u(n.src_offset) +
               " storage=" + std::to_string(n.storage_loc) + ":" + std::to_string(n.storage_id) +
               " group=" + std::to_string(n.group) + " inns=" + list(n.inns) + " mems=[";
        for (size_t i = 0; i != n.mems.size(); ++i) {
            out += (i ? "," : "") + u(n.mems[i].offset) + ":" + u(n.mems[i].size);
        }
        out += "]";
        if (n.einsummable) {
            es::mg_einsummable_t const& e = *n.einsummable;
            out += " einsummable{" + list(e.join_shape) + ";";
            for (auto const& inn : e.inns) out += list(inn);
            out += ";" + std::to_string(e.out_rank) + ";" + e.join + ";" + e.castable + "}";
        }
        if (n.touch) {
            es::touch_t const& t = *n.touch;
            out += std::string(" touch{") + es::dtype_name(t.dtype) + ";";
            if (t.castable) out += es::castable_to_char(t.castable);
            out += ";";
            for (auto const& d : t.selection) {
                out += list(std::vector<uint64_t>{d.d_inn, d.d_out, d.offset_inn, d.offset_out,
                                                  d.size});
            }
            out += "}";
        }
        if (n.kind == es::mg_kind::constant) {
            es::mg_fill_t const& f = n.fill;
            if (f.is_lowertri) {
                out += " lowertri{" + f.lower + ";" + f.upper + ";" + u(f.nrow) + ";" + u(f.ncol) +
                       ";" + std::to_string(f.start) + "}";
            } else {
                out += " constant{" + f.value + ";" + list(f.shape) + "}";
            }
        }
        out += "\n";
    }
    return out;
}

}  // namespace

extern "C" {

es_km_t* es_km_create(int device)
{
    try {
        auto* h = new es_km;
        h->km = std::make_unique<es::kernel_manager_t>(device);
        return h;
    } catch (std::exception const& e) {
        g_null_error = e.what();
        return nullptr;
    }
}

void es_km_destroy(es_km_t* km) { delete km; }

const char* es_km_last_error(es_km_t* km) { return err_slot(km).c_str(); }

int es_km_build(es_km_t* h, const uint64_t* join_shape, int join_rank, const int* inns_flat,
                const int* inns_offsets, int n_inns, int out_rank, const char* join_text,
                char castable, uint64_t* workspace_bytes)
{
    return guarded(h, [&]() -> int {
        if (!h) throw es::ir_error("null handle");
        check_descriptor(join_shape, join_rank, inns_flat, inns_offsets, n_inns, out_rank,
                         join_text);
        es::einsummable_t e = make_einsummable(join_shape, join_rank, inns_flat, inns_offsets,
                                               n_inns, out_rank, join_text, castable);
        auto ws = h->km->build(e);
        if (!ws) {
            h->last_error = "build: no kernel for einsummable " + e.key();
            return ES_KM_UNSUPPORTED;
        }
        h->km->alias_raw(raw_key(join_shape, join_rank, inns_flat, inns_offsets, n_inns, out_rank,
                                 join_text, castable),
                         e);
        if (workspace_bytes) *workspace_bytes = ws.value();
        return ES_KM_OK;
    });
}

int es_km_workspace_size(es_km_t* h, const uint64_t* join_shape, int join_rank,
                         const int* inns_flat, const int* inns_offsets, int n_inns, int out_rank,
                         const char* join_text, char castable, uint64_t* workspace_bytes)
{
    return guarded(h, [&]() -> int {
        if (!h) throw es::ir_error("null handle");
        check_descriptor(join_shape, join_rank, inns_flat, inns_offsets, n_inns, out_rank,
                         join_text);
        es::plan_t const* p = h->km->find_raw(raw_key(join_shape, join_rank, inns_flat,
                                                      inns_offsets, n_inns, out_rank, join_text,
                                                      castable));
        uint64_t ws;
        if (p) {
            ws = p->workspace_bytes;
        } else {
            ws = h->km->workspace_size(make_einsummable(join_shape, join_rank, inns_flat,
                                                        inns_offsets, n_inns, out_rank, join_text,
                                                        castable));
        }
        if (workspace_bytes) *workspace_bytes = ws;
        return ES_KM_OK;
    });
}

int es_km_execute(es_km_t* h, const uint64_t* join_shape, int join_rank, const int* inns_flat,
                  const int* inns_offsets, int n_inns, int out_rank, const char* join_text,
                  char castable, void* stream, void* out, const void* const* inns,
                  int n_inn_ptrs, void* workspace, uint64_t workspace_bytes)
{
    return guarded(h, [&]() -> int {
        if (!h) throw es::ir_error("null handle");
        check_descriptor(join_shape, join_rank, inns_flat, inns_offsets, n_inns, out_rank,
                         join_text);
        if (!out || !inns) throw es::ir_error("execute: null buffer");
        es::plan_t const* p = h->km->find_raw(raw_key(join_shape, join_rank, inns_flat,
                                                      inns_offsets, n_inns, out_rank, join_text,
                                                      castable));
        if (p) {
            h->km->run_plan(*p, static_cast<hipStream_t>(stream), out, inns, n_inn_ptrs, workspace,
                            workspace_bytes);
            return ES_KM_OK;
        }
        // Not seen under this spelling: an equal einsummable may still have been built
        // (two descriptors that merge to the same form share a kernel).
        es::einsummable_t e = make_einsummable(join_shape, join_rank, inns_flat, inns_offsets,
                                               n_inns, out_rank, join_text, castable);
        std::vector<void const*> v(inns, inns + n_inn_ptrs);
        std::optional<std::tuple<void*, uint64_t>> ws;
        if (workspace) ws = std::make_tuple(workspace, workspace_bytes);
        (*h->km)(e, static_cast<hipStream_t>(stream), out, v, ws);
        return ES_KM_OK;
    });
}

int es_km_execute_static_workspace(es_km_t* h, const uint64_t* join_shape, int join_rank,
                                   const int* inns_flat, const int* inns_offsets, int n_inns,
                                   int out_rank, const char* join_text, char castable,
                                   void* stream, void* out, const void* const* inns,
                                   int n_inn_ptrs)
{
    return guarded(h, [&]() -> int {
        if (!h) throw es::ir_error("null handle");
        check_descriptor(join_shape, join_rank, inns_flat, inns_offsets, n_inns, out_rank,
                         join_text);
        if (!out || !inns) throw es::ir_error("execute: null buffer");
        es::plan_t const* p = h->km->find_raw(raw_key(join_shape, join_rank, inns_flat,
                                                      inns_offsets, n_inns, out_rank, join_text,
                                                      castable));
        if (!p) {
            p = h->km->plan_of(make_einsummable(join_shape, join_rank, inns_flat, inns_offsets,
                                                n_inns, out_rank, join_text, castable));
        }
        if (!p) throw es::km_error(es::km_status::not_built, "execute: einsummable was not built");
        if (p->workspace_bytes > es::STATIC_WORKSPACE_BYTES) {
            throw es::km_error(es::km_status::workspace,
                               "execute_static_workspace: this einsummable needs " +
                                   std::to_string(p->workspace_bytes) +
                                   " bytes of workspace, the library's own holds " +
                                   std::to_string(es::STATIC_WORKSPACE_BYTES) +
                                   "; use es_km_execute with a workspace of the caller");
        }
        void* ws = es::static_workspace(h->km->device());
        if (!ws) throw es::km_error(es::km_status::device, "static workspace not initialised");
        h->km->run_plan(*p, static_cast<hipStream_t>(stream), out, inns, n_inn_ptrs, ws,
                        es::STATIC_WORKSPACE_BYTES);
        return ES_KM_OK;
    });
}

int es_km_describe(es_km_t* h, const uint64_t* join_shape, int join_rank, const int* inns_flat,
                   const int* inns_offsets, int n_inns, int out_rank, const char* join_text,
                   char castable, char* out, size_t cap)
{
    return guarded(h, [&]() -> int {
        if (!h) throw es::ir_error("null handle");
        check_descriptor(join_shape, join_rank, inns_flat, inns_offsets, n_inns, out_rank,
                         join_text);
        std::string d = h->km->describe(make_einsummable(join_shape, join_rank, inns_flat,
                                                         inns_offsets, n_inns, out_rank, join_text,
                                                         castable));
        if (!out || cap == 0) throw es::ir_error("describe: no output buffer");
        std::strncpy(out, d.c_str(), cap - 1);
        out[cap - 1] = 0;
        return ES_KM_OK;
    });
}

int es_km_touch(es_km_t* h, const uint64_t* touchdims, int rank, char castable, int dtype,
                void* stream, void* out, const void* inn)
{
    return guarded(h, [&]() -> int {
        if (!h) throw es::ir_error("null handle");
        if (!touchdims || rank < 1 || rank > 64) throw es::ir_error("touch: bad selection");
        if (dtype < 0 || dtype > 3) throw es::ir_error("touch: bad dtype");
        if (!out || !inn) throw es::ir_error("touch: null buffer");
        es::touch_t t;
        t.dtype = es::dtype_t(dtype);
        t.castable = es::castable_from_char(castable);
        t.selection.resize(size_t(rank));
        for (int i = 0; i != rank; ++i) {
            const uint64_t* d = touchdims + 5 * i;
            t.selection[i] = es::touchdim_t{d[0], d[1], d[2], d[3], d[4]};
        }
        (*h->km)(t, static_cast<hipStream_t>(stream), out, inn);
        return ES_KM_OK;
    });
}

int es_km_fill_constant(es_km_t* h, int dtype, uint64_t value_bits, uint64_t nelem, void* stream,
                        void* out)
{
    return guarded(h, [&]() -> int {
        if (!h) throw es::ir_error("null handle");
        if (dtype < 0 || dtype > 3) throw es::ir_error("fill: bad dtype");
        if (!out) throw es::ir_error("fill: null buffer");
        h->km->constant_fill(es::dtype_t(dtype), value_bits, nelem,
                             static_cast<hipStream_t>(stream), out);
        return ES_KM_OK;
    });
}

int es_km_fill_lowertri(es_km_t* h, int dtype, uint64_t lower_bits, uint64_t upper_bits,
                        uint64_t nrow, uint64_t ncol, int64_t start, void* stream, void* out)
{
    return guarded(h, [&]() -> int {
        if (!h) throw es::ir_error("null handle");
        if (dtype < 0 || dtype > 3) throw es::ir_error("fill: bad dtype");
        if (!out) throw es::ir_error("fill: null buffer");
        h->km->lowerTri_fill(es::dtype_t(dtype), lower_bits, upper_bits, nrow, ncol, start,
                             static_cast<hipStream_t>(stream), out);
        return ES_KM_OK;
    });
}

int es_km_codegen_source(const uint64_t* join_shape, int join_rank, const int* inns_flat,
                         const int* inns_offsets, int n_inns, int out_rank, const char* join_text,
                         char castable, int compile, char* out, size_t cap)
{
    return guarded(nullptr, [&]() -> int {
        check_descriptor(join_shape, join_rank, inns_flat, inns_offsets, n_inns, out_rank,
                         join_text);
        es::einsummable_t e = make_einsummable(join_shape, join_rank, inns_flat, inns_offsets,
                                               n_inns, out_rank, join_text, castable)
                                  .merge_adjacent_dims();
        es::cg_kernel_t k = es::generate_kernel(e);
        if (compile) es::compile_hip_source(k.source, "es_generated.hip", "gfx950");
        if (out && cap) {
            std::strncpy(out, k.source.c_str(), cap - 1);
            out[cap - 1] = 0;
        }
        return ES_KM_OK;
    });
}

int es_km_scalarop_roundtrip(const char* text, char* out, size_t cap, int* out_dtype,
                             int* n_inputs)
{
    return guarded(nullptr, [&]() -> int {
        if (!text) throw es::ir_error("null text");
        es::scalarop_t op = es::scalarop_t::parse(text);
        std::string    s = op.str();
        if (out && cap) {
            if (s.size() + 1 > cap) throw es::ir_error("roundtrip: buffer too small");
            std::memcpy(out, s.c_str(), s.size() + 1);
        }
        if (out_dtype) *out_dtype = int(op.out_dtype());
        if (n_inputs) *n_inputs = op.num_inputs();
        return ES_KM_OK;
    });
}

int es_km_scalarop_simplify(const char* text, const char* const* var_names,
                            const double* var_values, int n_vars, char* out, size_t cap)
{
    return guarded(nullptr, [&]() -> int {
        if (!text || !out || cap == 0) throw es::ir_error("simplify: null argument");
        if (n_vars < 0 || (n_vars > 0 && (!var_names || !var_values))) {
            throw es::ir_error("simplify: bad variable list");
        }
        std::vector<std::pair<std::string, double>> vars;
        for (int i = 0; i != n_vars; ++i) vars.emplace_back(var_names[i], var_values[i]);
        std::string const s = es::scalarop_t::parse(text).replace_variables(vars).simplify().str();
        if (s.size() + 1 > cap) throw es::ir_error("simplify: buffer too small");
        std::memcpy(out, s.c_str(), s.size() + 1);
        return ES_KM_OK;
    });
}

int es_km_merge_adjacent_dims(const uint64_t* join_shape, int join_rank, const int* inns_flat,
                              const int* inns_offsets, int n_inns, int out_rank,
                              const char* join_text, char castable, uint64_t* new_join_shape,
                              int* new_inns_flat, int* new_inns_offsets, int* new_out_rank,
                              char* str_out, size_t str_cap)
{
    return guarded(nullptr, [&]() -> int {
        check_descriptor(join_shape, join_rank, inns_flat, inns_offsets, n_inns, out_rank,
                         join_text);
        es::einsummable_t e = make_einsummable(join_shape, join_rank, inns_flat, inns_offsets,
                                               n_inns, out_rank, join_text, castable)
                                  .merge_adjacent_dims();
        int pos = 0;
        for (size_t i = 0; i != e.join_shape.size(); ++i) new_join_shape[i] = e.join_shape[i];
        for (size_t k = 0; k != e.inns.size(); ++k) {
            new_inns_offsets[k] = pos;
            for (int m : e.inns[k]) new_inns_flat[pos++] = m;
        }
        new_inns_offsets[e.inns.size()] = pos;
        *new_out_rank = e.out_rank;
        if (str_out && str_cap) {
            std::string s = e.str();
            std::strncpy(str_out, s.c_str(), str_cap - 1);
            str_out[str_cap - 1] = 0;
        }
        return int(e.join_shape.size());
    });
}

int es_km_touch_batch(es_km_t* h, int n_touches, const uint64_t* touchdims, const int* ranks,
                      const char* castables, int dtype, void* stream, void* out,
                      const void* const* inns)
{
    return guarded(h, [&]() -> int {
        if (!h) throw es::ir_error("null handle");
        if (n_touches < 0 || (n_touches > 0 && (!touchdims || !ranks || !castables || !inns))) {
            throw es::ir_error("touch_batch: bad arguments");
        }
        if (dtype < 0 || dtype > 3) throw es::ir_error("touch_batch: bad dtype");
        if (!out) throw es::ir_error("touch_batch: null buffer");
        std::vector<es::touch_t> ts;
        ts.resize(size_t(n_touches));
        std::vector<void const*> ptrs(inns, inns + n_touches);
        const uint64_t*          d = touchdims;
        for (int i = 0; i != n_touches; ++i) {
            if (ranks[i] < 1 || ranks[i] > 64) throw es::ir_error("touch_batch: bad rank");
            ts[i].dtype = es::dtype_t(dtype);
            ts[i].castable = es::castable_from_char(castables[i]);
            for (int k = 0; k != ranks[i]; ++k, d += 5) {
                ts[i].selection.push_back(es::touchdim_t{d[0], d[1], d[2], d[3], d[4]});
            }
            if (!ptrs[i]) throw es::ir_error("touch_batch: null input");
        }
        h->km->touch_batch(ts, static_cast<hipStream_t>(stream), out, ptrs);
        return ES_KM_OK;
    });
}

double es_km_probe_mfma_f16(es_km_t* h, const void* operands, void* scratch, int blocks, int iters,
                            void* stream)
{
    if (!h || !operands || !scratch || blocks < 1 || iters < 1) return -1.0;
    return es::gemm::probe_mfma_f16(operands, scratch, blocks, iters,
                                    static_cast<hipStream_t>(stream));
}

// ---- exec-node layer (see exec_graph.h)

es_km_graph_t* es_km_graph_create(es_km_t* h)
{
    try {
        auto* g = new es_km_graph;
        g->owner = h;
        g->graph = std::make_unique<es::apply_graph_t>(h ? h->km.get() : nullptr);
        return g;
    } catch (std::exception const& e) {
        err_slot(h) = e.what();
        return nullptr;
    }
}

void es_km_graph_destroy(es_km_graph_t* g) { delete g; }

extern "C++" {
namespace
{
std::vector<es::mem_t> make_mems(const uint64_t* offsets, const uint64_t* sizes, int n)
{
    if (!offsets || !sizes || n < 1) throw es::ir_error("graph node: bad memory ranges");
    std::vector<es::mem_t> m;
    for (int i = 0; i != n; ++i) m.push_back(es::mem_t{offsets[i], sizes[i]});
    return m;
}
std::vector<int> make_deps(const int* deps, int n)
{
    if (n < 0 || (n > 0 && !deps)) throw es::ir_error("graph node: bad dependency list");
    return std::vector<int>(deps, deps + n);
}
}  // namespace
}  // extern "C++"

int es_km_graph_add_einsummable(es_km_graph_t* g, const uint64_t* join_shape, int join_rank,
                                const int* inns_flat, const int* inns_offsets, int n_inns,
                                int out_rank, const char* join_text, char castable,
                                const uint64_t* mem_offsets, const uint64_t* mem_sizes, int n_mems,
                                const int* deps, int n_deps)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        check_descriptor(join_shape, join_rank, inns_flat, inns_offsets, n_inns, out_rank,
                         join_text);
        es::einsummable_t e = make_einsummable(join_shape, join_rank, inns_flat, inns_offsets,
                                               n_inns, out_rank, join_text, castable);
        return g->graph->add_einsummable(e, make_mems(mem_offsets, mem_sizes, n_mems),
                                         make_deps(deps, n_deps));
    });
}

int es_km_graph_add_touch(es_km_graph_t* g, const uint64_t* touchdims, int rank, char castable,
                          int dtype, int group, const uint64_t* mem_offsets,
                          const uint64_t* mem_sizes, const int* deps, int n_deps)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        if (!touchdims || rank < 1 || rank > 64) throw es::ir_error("touch: bad selection");
        if (dtype < 0 || dtype > 3) throw es::ir_error("touch: bad dtype");
        es::touch_t t;
        t.dtype = es::dtype_t(dtype);
        t.castable = es::castable_from_char(castable);
        t.selection.resize(size_t(rank));
        for (int i = 0; i != rank; ++i) {
            const uint64_t* d = touchdims + 5 * i;
            t.selection[size_t(i)] = es::touchdim_t{d[0], d[1], d[2], d[3], d[4]};
        }
        return g->graph->add_touch(t, group, make_mems(mem_offsets, mem_sizes, 2),
                                   make_deps(deps, n_deps));
    });
}

int es_km_graph_add_fill_constant(es_km_graph_t* g, int dtype, uint64_t value_bits,
                                  uint64_t nelem, uint64_t offset, uint64_t size, const int* deps,
                                  int n_deps)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        if (dtype < 0 || dtype > 3) throw es::ir_error("fill: bad dtype");
        return g->graph->add_constant_fill(es::dtype_t(dtype), value_bits, nelem,
                                           es::mem_t{offset, size}, make_deps(deps, n_deps));
    });
}

int es_km_graph_add_fill_lowertri(es_km_graph_t* g, int dtype, uint64_t lower_bits,
                                  uint64_t upper_bits, uint64_t nrow, uint64_t ncol, int64_t start,
                                  uint64_t offset, uint64_t size, const int* deps, int n_deps)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        if (dtype < 0 || dtype > 3) throw es::ir_error("fill: bad dtype");
        return g->graph->add_lowertri_fill(es::dtype_t(dtype), lower_bits, upper_bits, nrow, ncol,
                                           start, es::mem_t{offset, size},
                                           make_deps(deps, n_deps));
    });
}

int es_km_graph_add_copy(es_km_graph_t* g, uint64_t dst_offset, uint64_t src_offset, uint64_t size,
                         const int* deps, int n_deps)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        return g->graph->add_copy(es::mem_t{dst_offset, size}, es::mem_t{src_offset, size},
                                  make_deps(deps, n_deps));
    });
}

int es_km_graph_add_memory_dependencies(es_km_graph_t* g)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        g->graph->add_memory_dependencies();
        return ES_KM_OK;
    });
}

int es_km_graph_optimize(es_km_graph_t* g, int* n_absorbed)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        int const n = g->graph->optimize();
        if (n_absorbed) *n_absorbed = n;
        return ES_KM_OK;
    });
}

int es_km_graph_finalize(es_km_graph_t* g, int n_streams)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        g->graph->finalize(n_streams);
        return ES_KM_OK;
    });
}

int es_km_graph_run(es_km_graph_t* g, void* stream, void* arena)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        if (!arena) throw es::ir_error("graph run: null arena");
        g->graph->run(static_cast<hipStream_t>(stream), arena);
        return ES_KM_OK;
    });
}

int es_km_graph_node_info(es_km_graph_t* g, int id, int* position, int* stream, int* deps, int cap,
                          int* n_deps)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        if (id < 0 || id >= g->graph->n_nodes()) throw es::ir_error("graph: no such node");
        if (position) *position = g->graph->position_of(id);
        if (stream) *stream = g->graph->stream_of(id);
        std::vector<int> const& d = g->graph->deps_of(id);
        if (n_deps) *n_deps = int(d.size());
        for (int i = 0; deps && i < cap && i < int(d.size()); ++i) deps[i] = d[size_t(i)];
        return ES_KM_OK;
    });
}

int es_km_graph_cross_stream_waits(es_km_graph_t* g)
{
    return g ? g->graph->n_cross_stream_waits() : ES_KM_ERR_INVALID;
}

int es_km_graph_launch_node(es_km_graph_t* g, int id, void* stream, void* arena, void* workspace,
                            uint64_t workspace_bytes, int first_in_group,
                            es_km_callback_t callback, void* user)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        if (!arena) throw es::ir_error("graph launch: null arena");
        g->graph->launch_node(id, static_cast<hipStream_t>(stream), arena, workspace,
                              workspace_bytes, first_in_group, callback, user);
        return ES_KM_OK;
    });
}

int es_km_graph_node_workspace(es_km_graph_t* g, int id, uint64_t* workspace_bytes)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        if (id < 0 || id >= g->graph->n_nodes()) throw es::ir_error("graph: no such node");
        if (workspace_bytes) *workspace_bytes = g->graph->node_workspace(id);
        return ES_KM_OK;
    });
}

int es_km_graph_node_group(es_km_graph_t* g, int id)
{
    if (!g || id < 0 || id >= g->graph->n_nodes()) return -1;
    return g->graph->kind_of(id) == 1 ? g->graph->group_of(id) : -1;
}

es_km_workspace_pool_t* es_km_workspace_pool_create(int device)
{
    try {
        return new es_km_workspace_pool(device);
    } catch (std::exception const& e) {
        g_null_error = e.what();
        return nullptr;
    }
}

void es_km_workspace_pool_destroy(es_km_workspace_pool_t* p) { delete p; }

void* es_km_workspace_pool_acquire(es_km_workspace_pool_t* p, uint64_t bytes, uint64_t* got_bytes)
{
    try {
        if (!p) throw es::ir_error("null pool");
        return p->pool.acquire(bytes, got_bytes);
    } catch (std::exception const& e) {
        g_null_error = e.what();
        return nullptr;
    }
}

int es_km_workspace_pool_release(es_km_workspace_pool_t* p, void* block)
{
    return guarded(nullptr, [&]() -> int {
        if (!p) throw es::ir_error("null pool");
        p->pool.release(block);
        return ES_KM_OK;
    });
}

int es_km_workspace_pool_blocks(es_km_workspace_pool_t* p)
{
    return p ? p->pool.n_blocks() : ES_KM_ERR_INVALID;
}

es_km_stream_pool_t* es_km_stream_pool_create(int device, int n_streams)
{
    try {
        return new es_km_stream_pool(device, n_streams);
    } catch (std::exception const& e) {
        g_null_error = e.what();
        return nullptr;
    }
}

void es_km_stream_pool_destroy(es_km_stream_pool_t* p) { delete p; }

void* es_km_stream_pool_try_acquire(es_km_stream_pool_t* p)
{
    return p ? static_cast<void*>(p->pool.try_acquire()) : nullptr;
}

int es_km_stream_pool_release(es_km_stream_pool_t* p, void* stream)
{
    return guarded(nullptr, [&]() -> int {
        if (!p) throw es::ir_error("null pool");
        p->pool.release(static_cast<hipStream_t>(stream));
        return ES_KM_OK;
    });
}

int64_t es_km_graph_node_describe(es_km_graph_t* g, int id, char* out, uint64_t cap)
{
    if (!g || id < 0 || id >= g->graph->n_nodes()) return ES_KM_ERR_INVALID;
    std::string const s = g->graph->describe(id);
    if (out && cap) {
        uint64_t const n = std::min<uint64_t>(cap - 1, s.size());
        std::memcpy(out, s.data(), n);
        out[n] = 0;
    }
    return int64_t(s.size());
}

int64_t es_km_graph_node_source(es_km_graph_t* g, int id, int compile, char* out, uint64_t cap)
{
    if (!g || id < 0 || id >= g->graph->n_nodes()) return ES_KM_ERR_INVALID;
    int64_t   length = 0;
    int const rc = guarded(g->owner, [&]() -> int {
        std::string const s = g->graph->generated_source(id);
        if (compile && !s.empty()) es::compile_hip_source(s, "es_generated.hip", "gfx950");
        if (out && cap) {
            uint64_t const n = std::min<uint64_t>(cap - 1, s.size());
            std::memcpy(out, s.data(), n);
            out[n] = 0;
        }
        length = int64_t(s.size());
        return ES_KM_OK;
    });
    return rc < 0 ? rc : length;
}

int es_km_graph_launches(es_km_graph_t* g)
{
    return g ? g->graph->n_launches() : ES_KM_ERR_INVALID;
}

int es_km_graph_add_dummy(es_km_graph_t* g, uint64_t offset, uint64_t size, const int* deps,
                          int n_deps)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        return g->graph->add_dummy(es::mem_t{offset, size}, make_deps(deps, n_deps));
    });
}

int es_km_graph_add_placeholder(es_km_graph_t* g, uint64_t offset, uint64_t size, const int* deps,
                                int n_deps)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        return g->graph->add_dummy(es::mem_t{offset, size}, make_deps(deps, n_deps), false);
    });
}

int es_km_graph_add_evict(es_km_graph_t* g, uint64_t offset, uint64_t size, int storage_id,
                          const int* deps, int n_deps)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        return g->graph->add_evict(es::mem_t{offset, size}, storage_id, make_deps(deps, n_deps));
    });
}

int es_km_graph_add_load(es_km_graph_t* g, int storage_id, uint64_t offset, uint64_t size,
                         const int* deps, int n_deps)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        return g->graph->add_load(storage_id, es::mem_t{offset, size}, make_deps(deps, n_deps));
    });
}

int es_km_graph_declare_storage(es_km_graph_t* g, int storage_id, uint64_t size)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        g->graph->declare_storage(storage_id, size);
        return ES_KM_OK;
    });
}

int es_km_graph_storage_write(es_km_graph_t* g, int storage_id, const void* src, uint64_t size)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        if (!src && size) throw es::ir_error("storage write: null source");
        g->graph->storage_write(storage_id, src, size);
        return ES_KM_OK;
    });
}

int es_km_graph_storage_read(es_km_graph_t* g, int storage_id, void* dst, uint64_t size)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        if (!dst && size) throw es::ir_error("storage read: null destination");
        g->graph->storage_read(storage_id, dst, size);
        return ES_KM_OK;
    });
}

int es_km_graph_load_memgraph(es_km_graph_t* g, const void* bytes, uint64_t size, int loc,
                              const char* const* var_names, const double* var_values, int n_vars)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        if (n_vars < 0 || (n_vars > 0 && (!var_names || !var_values))) {
            throw es::ir_error("memgraph: bad scalar variables");
        }
        std::vector<std::pair<std::string, double>> vars;
        for (int i = 0; i != n_vars; ++i) vars.push_back({var_names[i], var_values[i]});
        es::memgraph_t mg = es::decode_memgraph(bytes, size);
        mg.populate(*g->graph, loc, vars);
        return g->graph->n_nodes();
    });
}

int es_km_graph_num_nodes(es_km_graph_t* g) { return g ? g->graph->n_nodes() : ES_KM_ERR_INVALID; }

uint64_t es_km_graph_arena_bytes(es_km_graph_t* g) { return g ? g->graph->arena_bytes() : 0; }

int es_km_graph_node_mems(es_km_graph_t* g, int id, int* kind, uint64_t* offsets, uint64_t* sizes,
                          int cap, int* n_mems)
{
    return guarded(g ? g->owner : nullptr, [&]() -> int {
        if (!g) throw es::ir_error("null graph");
        if (id < 0 || id >= g->graph->n_nodes()) throw es::ir_error("graph: no such node");
        if (kind) *kind = g->graph->kind_of(id);
        std::vector<es::mem_t> const& m = g->graph->mems_of(id);
        if (n_mems) *n_mems = int(m.size());
        for (int i = 0; i < cap && i < int(m.size()); ++i) {
            if (offsets) offsets[i] = m[size_t(i)].offset;
            if (sizes) sizes[i] = m[size_t(i)].size;
        }
        return ES_KM_OK;
    });
}

int64_t es_km_memgraph_describe(const void* bytes, uint64_t size, char* out, uint64_t cap)
{
    try {
        es::memgraph_t mg = es::decode_memgraph(bytes, size);
        std::string    s = describe_memgraph(mg);
        if (out && cap) {
            uint64_t const n = std::min<uint64_t>(cap - 1, s.size());
            std::memcpy(out, s.data(), n);
            out[n] = 0;
        }
        return int64_t(s.size());
    } catch (std::exception const& e) {
        g_null_error = e.what();
        return ES_KM_ERR_INVALID;
    }
}

}
