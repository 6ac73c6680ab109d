#include "exec_graph.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>

namespace es
{
namespace
{

void check(hipError_t err, const char* what)
{
    if (err != hipSuccess) {
        throw km_error(km_status::device, std::string(what) + ": " + hipGetErrorString(err));
    }
}

bool overlaps(mem_t const& a, mem_t const& b)
{
    return a.size != 0 && b.size != 0 && a.offset < b.offset + b.size &&
           b.offset < a.offset + a.size;
}

}  // namespace

apply_graph_t::apply_graph_t(kernel_manager_t* km) : km_(km) {}

apply_graph_t::~apply_graph_t()
{
    for (size_t s = 1; s < streams_.size(); ++s) (void)hipStreamDestroy(streams_[s]);
    for (void* w : workspace_) {
        if (w) (void)hipFree(w);
    }
    for (auto& s : slots_) {
        if (s.second.host) (void)hipHostFree(s.second.host);
    }
    for (hipEvent_t e : events_) (void)hipEventDestroy(e);
    for (hipEvent_t e : joins_) (void)hipEventDestroy(e);
    if (fork_) (void)hipEventDestroy(fork_);
}

int apply_graph_t::insert(node_t&& n, std::vector<int> const& deps)
{
    if (finalized_) throw km_error(km_status::invalid, "apply graph: already finalized");
    int const id = int(nodes_.size());
    for (int d : deps) {
        // insertion order is the launch order, so a node can only wait for earlier ones
        if (d < 0 || d >= id) {
            throw km_error(km_status::invalid,
                           "apply graph: node " + std::to_string(id) + " depends on node " +
                               std::to_string(d) + ", which is not an earlier node");
        }
    }
    n.deps = deps;
    std::sort(n.deps.begin(), n.deps.end());
    n.deps.erase(std::unique(n.deps.begin(), n.deps.end()), n.deps.end());
    nodes_.push_back(std::move(n));
    return id;
}

int apply_graph_t::add_einsummable(einsummable_t const& e, std::vector<mem_t> const& mems,
                                   std::vector<int> const& deps)
{
    if (mems.size() != e.inns.size() + 1) {
        throw km_error(km_status::inputs, "apply graph: einsummable with " +
                                              std::to_string(e.inns.size()) + " inputs given " +
                                              std::to_string(mems.size()) + " memory ranges");
    }
    node_t n;
    n.kind = kind_t::einsummable;
    n.e = e;
    n.mems = mems;
    return insert(std::move(n), deps);
}

int apply_graph_t::add_touch(touch_t const& t, int group, std::vector<mem_t> const& mems,
                             std::vector<int> const& deps_)
{
    if (mems.size() != 2) {
        throw km_error(km_status::inputs, "apply graph: a touch takes an output and an input");
    }
    t.validate();
    node_t n;
    n.kind = kind_t::touch;
    n.touch = t;
    n.group = group;
    n.mems = mems;
    std::vector<int> deps = deps_;
    // A touch outside any group is the only writer of its bytes: a copy.  Inside a group
    // the touches are serialised in insertion order and the first one initialises.
    int previous = -1;
    if (group >= 0) {
        for (int i = int(nodes_.size()) - 1; i >= 0 && previous < 0; --i) {
            if (nodes_[i].kind == kind_t::touch && nodes_[i].group == group) previous = i;
        }
    }
    n.group_castable = t.castable;
    if (previous < 0) {
        n.touch.castable = std::nullopt;
    } else {
        deps.push_back(previous);
    }
    return insert(std::move(n), deps);
}

int apply_graph_t::add_constant_fill(dtype_t dtype, uint64_t value_bits, uint64_t nelem,
                                     mem_t out, std::vector<int> const& deps)
{
    node_t n;
    n.kind = kind_t::constant;
    n.dtype = dtype;
    n.bits0 = value_bits;
    n.n0 = nelem;
    n.mems = {out};
    return insert(std::move(n), deps);
}

int apply_graph_t::add_lowertri_fill(dtype_t dtype, uint64_t lower_bits, uint64_t upper_bits,
                                     uint64_t nrow, uint64_t ncol, int64_t start, mem_t out,
                                     std::vector<int> const& deps)
{
    node_t n;
    n.kind = kind_t::lowertri;
    n.dtype = dtype;
    n.bits0 = lower_bits;
    n.bits1 = upper_bits;
    n.n0 = nrow;
    n.n1 = ncol;
    n.start = start;
    n.mems = {out};
    return insert(std::move(n), deps);
}

int apply_graph_t::add_copy(mem_t dst, mem_t src, std::vector<int> const& deps)
{
    if (dst.size != src.size) {
        throw km_error(km_status::invalid, "apply graph: copy between ranges of different size");
    }
    node_t n;
    n.kind = kind_t::copy;
    n.mems = {dst, src};
    return insert(std::move(n), deps);
}

int apply_graph_t::add_dummy(mem_t range, std::vector<int> const& deps)
{
    node_t n;
    n.kind = kind_t::dummy;
    n.mems = {range};
    return insert(std::move(n), deps);
}

apply_graph_t::slot_t* apply_graph_t::slot(int storage_id)
{
    for (auto& s : slots_) {
        if (s.first == storage_id) return &s.second;
    }
    return nullptr;
}

apply_graph_t::slot_t const* apply_graph_t::slot(int storage_id) const
{
    return const_cast<apply_graph_t*>(this)->slot(storage_id);
}

void apply_graph_t::declare_storage(int storage_id, uint64_t size)
{
    if (finalized_) throw km_error(km_status::invalid, "apply graph: already finalized");
    if (storage_id < 0) throw km_error(km_status::invalid, "apply graph: negative storage id");
    slot_t* s = slot(storage_id);
    if (!s) {
        slots_.push_back({storage_id, slot_t{}});
        s = &slots_.back().second;
    }
    s->size = std::max(s->size, size);
}

int apply_graph_t::add_evict(mem_t src, int storage_id, std::vector<int> const& deps)
{
    declare_storage(storage_id, src.size);
    node_t n;
    n.kind = kind_t::evict;
    n.storage_id = storage_id;
    n.mems = {mem_t{0, 0}, src};  // reads the arena, writes none of it
    return insert(std::move(n), deps);
}

int apply_graph_t::add_load(int storage_id, mem_t dst, std::vector<int> const& deps)
{
    declare_storage(storage_id, dst.size);
    node_t n;
    n.kind = kind_t::load;
    n.storage_id = storage_id;
    n.mems = {dst};
    return insert(std::move(n), deps);
}

void apply_graph_t::storage_write(int storage_id, void const* src, uint64_t size)
{
    slot_t* s = slot(storage_id);
    if (!finalized_ || !s || !s->host) {
        throw km_error(km_status::invalid, "apply graph: no storage slot " +
                                               std::to_string(storage_id) +
                                               " (declared slots exist after finalize)");
    }
    if (size > s->size) throw km_error(km_status::invalid, "apply graph: storage slot too small");
    std::memcpy(s->host, src, size);
}

void apply_graph_t::storage_read(int storage_id, void* dst, uint64_t size) const
{
    slot_t const* s = slot(storage_id);
    if (!finalized_ || !s || !s->host) {
        throw km_error(km_status::invalid, "apply graph: no storage slot " +
                                               std::to_string(storage_id) +
                                               " (declared slots exist after finalize)");
    }
    if (size > s->size) throw km_error(km_status::invalid, "apply graph: storage slot too small");
    std::memcpy(dst, s->host, size);
}

std::string apply_graph_t::describe(int id) const
{
    static const char* names[] = {"einsummable", "touch", "constant", "lowertri",
                                  "copy",        "dummy", "evict",    "load"};
    node_t const& n = nodes_[size_t(id)];
    std::string   s = names[int(n.kind)];
    for (mem_t const& m : n.mems) s += " " + std::to_string(m.offset) + ":" + std::to_string(m.size);
    if (n.kind == kind_t::einsummable) s += " | " + n.e.key();
    return s;
}

uint64_t apply_graph_t::arena_bytes() const
{
    uint64_t need = 0;
    for (node_t const& n : nodes_) {
        for (mem_t const& m : n.mems) {
            if (m.size) need = std::max(need, m.offset + m.size);
        }
    }
    return need;
}

void apply_graph_t::add_memory_dependencies()
{
    if (finalized_) throw km_error(km_status::invalid, "apply graph: already finalized");
    for (size_t v = 0; v != nodes_.size(); ++v) {
        node_t& nv = nodes_[v];
        if (nv.kind == kind_t::dummy) continue;
        for (size_t u = 0; u != v; ++u) {
            node_t const& nu = nodes_[u];
            if (nu.kind == kind_t::dummy) continue;
            bool dep = false;
            // v reads or rewrites what u wrote; v overwrites what u read
            for (mem_t const& m : nv.mems) dep = dep || overlaps(nu.mems[0], m);
            for (size_t k = 1; k < nu.mems.size(); ++k) dep = dep || overlaps(nv.mems[0], nu.mems[k]);
            // the storage slot is memory too: evict writes it, load reads it
            if (nu.storage_id >= 0 && nu.storage_id == nv.storage_id) dep = true;
            if (dep) nv.deps.push_back(int(u));
        }
        std::sort(nv.deps.begin(), nv.deps.end());
        nv.deps.erase(std::unique(nv.deps.begin(), nv.deps.end()), nv.deps.end());
    }
}

namespace
{

bool covers(mem_t const& a, mem_t const& b)
{
    return a.offset <= b.offset && b.offset + b.size <= a.offset + a.size;
}

bool same_range(mem_t const& a, mem_t const& b) { return a.offset == b.offset && a.size == b.size; }

bool is_iota(std::vector<int> const& inn, int rank)
{
    if (int(inn.size()) != rank) return false;
    for (int i = 0; i != rank; ++i) {
        if (inn[size_t(i)] != i) return false;
    }
    return true;
}

bool is_increasing(std::vector<int> const& inn)
{
    for (size_t i = 1; i < inn.size(); ++i) {
        if (inn[i] <= inn[i - 1]) return false;
    }
    return true;
}

// u: elementwise (no aggregation), every input straight or broadcast.
bool absorbable_producer(einsummable_t const& u)
{
    if (u.has_aggregation() || u.join.has_variables()) return false;
    for (auto const& inn : u.inns) {
        if (!is_increasing(inn)) return false;
    }
    return true;
}

// The einsummable that computes v with u in place of its input k, or nothing when the two
// do not line up.  v reads input k position by position over its join modes.
std::optional<einsummable_t> merged(einsummable_t const& u, einsummable_t const& v, int k)
{
    int const Ru = int(u.join_shape.size());
    int const Rv = int(v.join_shape.size());
    if (u.out_dtype() != v.inn_dtype(k) || u.out_nelem() != v.inn_nelem(k)) return std::nullopt;
    if (u.inns.size() + v.inns.size() - 1 > 6) return std::nullopt;
    std::vector<std::vector<int>> u_inns = u.inns, v_inns = v.inns;
    std::vector<uint64_t>         shape = v.join_shape;
    int                           out_rank = v.out_rank;
    auto all_iota = [](einsummable_t const& e) {
        if (e.has_aggregation()) return false;
        for (auto const& inn : e.inns) {
            if (!is_iota(inn, int(e.join_shape.size()))) return false;
        }
        return true;
    };
    auto iota = [](int rank) {
        std::vector<int> r(size_t(rank), 0);
        for (int i = 0; i != rank; ++i) r[size_t(i)] = i;
        return r;
    };
    if (u.join_shape == v.join_shape) {
        // as they are
    } else if (all_iota(v)) {
        // v is a map over positions: it takes the shape u gives them
        shape = u.join_shape;
        out_rank = Ru;
        for (auto& inn : v_inns) inn = iota(Ru);
    } else if (all_iota(u)) {
        for (auto& inn : u_inns) inn = iota(Rv);
    } else {
        return std::nullopt;
    }
    std::vector<std::vector<int>> inns = u_inns;
    for (int i = 0; i != int(v_inns.size()); ++i) {
        if (i != k) inns.push_back(v_inns[size_t(i)]);
    }
    try {
        return einsummable_t::make(shape, inns, out_rank, scalarop_t::compose(v.join, k, u.join),
                                   v.castable);
    } catch (ir_error const&) {
        return std::nullopt;
    }
}

}  // namespace

bool apply_graph_t::absorb_producer(int v)
{
    node_t& nv = nodes_[size_t(v)];
    int const n = int(nodes_.size());
    std::vector<int> candidates;  // indices into nv.mems
    bool const copy = nv.kind == kind_t::touch;
    if (copy) {
        touch_t const t = nv.touch.simplify();
        if (t.castable || t.selection.size() != 1) return false;
        touchdim_t const& d = t.selection[0];
        if (d.d_inn != d.size || d.d_out != d.size || d.offset_inn || d.offset_out) return false;
        if (d.size * dtype_size(t.dtype) != nv.mems[0].size || nv.mems[1].size != nv.mems[0].size) {
            return false;
        }
        for (int w = 0; nv.group >= 0 && w != n; ++w) {
            if (w != v && nodes_[size_t(w)].kind == kind_t::touch && nodes_[size_t(w)].group == nv.group) {
                return false;
            }
        }
        candidates.push_back(1);
    } else if (nv.kind == kind_t::einsummable) {
        einsummable_t const& e = nv.e;
        if (e.join.has_variables() || (e.has_aggregation() && e.inns.size() != 1)) return false;
        for (int k = 0; k != int(e.inns.size()); ++k) {
            if (is_iota(e.inns[size_t(k)], int(e.join_shape.size()))) candidates.push_back(k + 1);
        }
    }
    for (int slot : candidates) {
        mem_t const S = nv.mems[size_t(slot)];
        if (S.size == 0) continue;
        bool clean = true;
        for (size_t i = 0; i != nv.mems.size(); ++i) {
            if (int(i) != slot && overlaps(nv.mems[i], S)) clean = false;
        }
        if (!clean) continue;
        // the node that wrote S: the last one before v to write any of it
        int u = -1;
        for (int w = v - 1; w >= 0 && u < 0; --w) {
            node_t const& nw = nodes_[size_t(w)];
            if (nw.kind == kind_t::dummy || nw.kind == kind_t::evict) continue;
            if (overlaps(nw.mems[0], S)) u = w;
        }
        if (u < 0) continue;
        node_t& nu = nodes_[size_t(u)];
        if (nu.kind != kind_t::einsummable || !same_range(nu.mems[0], S)) continue;
        if (!copy && !absorbable_producer(nu.e)) continue;
        for (size_t i = 1; i != nu.mems.size(); ++i) {
            // u reads at v's place now: not what it would write there, not its own old output
            if (overlaps(nu.mems[i], nv.mems[0]) || overlaps(nu.mems[i], S)) clean = false;
        }
        // between the two: nobody else reads S, nobody writes what u reads
        for (int w = u + 1; w < v && clean; ++w) {
            node_t const& nw = nodes_[size_t(w)];
            if (nw.kind == kind_t::dummy) continue;
            for (size_t i = 1; i < nw.mems.size(); ++i) clean = clean && !overlaps(nw.mems[i], S);
            if (nw.kind == kind_t::evict) continue;
            for (size_t i = 1; i != nu.mems.size(); ++i) {
                clean = clean && !overlaps(nw.mems[0], nu.mems[i]);
            }
        }
        if (!clean) continue;
        // after v: S is deleted before anybody reads or rewrites it
        bool deleted = false;
        for (int w = v + 1; w < n && clean && !deleted; ++w) {
            node_t const& nw = nodes_[size_t(w)];
            if (nw.kind == kind_t::dummy) {
                deleted = covers(nw.mems[0], S) &&
                          std::binary_search(nw.deps.begin(), nw.deps.end(), v);
                continue;
            }
            for (size_t i = nw.kind == kind_t::evict ? 1 : 0; i < nw.mems.size(); ++i) {
                clean = clean && !overlaps(nw.mems[i], S);
            }
        }
        if (!clean || !deleted) continue;

        einsummable_t fused = nu.e;
        if (!copy) {
            std::optional<einsummable_t> m = merged(nu.e, nv.e, slot - 1);
            if (!m) continue;
            fused = std::move(m.value());
        }
        if (km_ && !copy) {
            try {
                if (!km_->build(fused)) continue;
            } catch (km_error const&) {
                continue;
            } catch (ir_error const&) {
                continue;
            }
        }
        std::vector<mem_t> mems{nv.mems[0]};
        for (size_t i = 1; i != nu.mems.size(); ++i) mems.push_back(nu.mems[i]);
        for (size_t i = 1; i != nv.mems.size(); ++i) {
            if (!copy && int(i) != slot) mems.push_back(nv.mems[i]);
        }
        std::vector<int> deps = nv.deps;
        deps.erase(std::remove(deps.begin(), deps.end(), u), deps.end());
        deps.insert(deps.end(), nu.deps.begin(), nu.deps.end());
        std::sort(deps.begin(), deps.end());
        deps.erase(std::unique(deps.begin(), deps.end()), deps.end());
        nv.kind = kind_t::einsummable;
        nv.e = std::move(fused);
        nv.mems = std::move(mems);
        nv.deps = std::move(deps);
        nv.group = -1;
        nu.kind = kind_t::dummy;
        nu.mems = {S};
        // whoever waited for u to be done with its inputs waits for the node that reads them now
        for (int w = v + 1; w < n; ++w) {
            std::vector<int>& d = nodes_[size_t(w)].deps;
            if (std::binary_search(d.begin(), d.end(), u) && !std::binary_search(d.begin(), d.end(), v)) {
                d.insert(std::upper_bound(d.begin(), d.end(), v), v);
            }
        }
        return true;
    }
    return false;
}

int apply_graph_t::optimize()
{
    if (finalized_) throw km_error(km_status::invalid, "apply graph: already finalized");
    int absorbed = 0;
    for (int v = 0; v != int(nodes_.size()); ++v) {
        while (absorb_producer(v)) ++absorbed;
    }
    return absorbed;
}

void apply_graph_t::finalize(int n_streams)
{
    if (finalized_) throw km_error(km_status::invalid, "apply graph: already finalized");
    if (n_streams < 1 || n_streams > 16) {
        throw km_error(km_status::invalid, "apply graph: between 1 and 16 streams");
    }
    int const n = int(nodes_.size());
    if (km_) {
        for (node_t const& nd : nodes_) {
            if (nd.kind != kind_t::einsummable) continue;
            if (!km_->build(nd.e)) {
                throw km_error(km_status::invalid, "apply graph: no kernel for an einsummable "
                                                   "(build returned unsupported)");
            }
        }
    }

    // Placement, in launch order.  A node continues the stream of a dependency that is
    // still the last node of its stream (the most recent such dependency): that needs no
    // wait at all.  Otherwise it takes the stream whose last node is oldest, and independent
    // branches spread over the pool.
    std::vector<int> last(size_t(n_streams), -1);
    std::vector<std::vector<int>> synced(size_t(n_streams), std::vector<int>(size_t(n_streams), -1));
    order_.resize(size_t(n));
    n_waits_ = 0;
    for (int v = 0; v != n; ++v) {
        node_t& nv = nodes_[v];
        nv.position = v;
        order_[size_t(v)] = v;
        int best = -1;
        for (int d : nv.deps) {
            int s = nodes_[d].stream;
            if (last[size_t(s)] == d && (best < 0 || d > last[size_t(best)])) best = s;
        }
        if (best < 0) {
            best = 0;
            for (int s = 1; s != n_streams; ++s) {
                if (last[size_t(s)] < last[size_t(best)]) best = s;
            }
        }
        nv.stream = best;
        last[size_t(best)] = v;
        // waits: a stream runs in order, so waiting for a node covers everything its stream
        // launched before it
        nv.waits.clear();
        std::vector<int> deps = nv.deps;
        std::sort(deps.begin(), deps.end(), [](int x, int y) { return x > y; });
        for (int d : deps) {
            int sd = nodes_[d].stream;
            if (sd == best) continue;
            if (synced[size_t(best)][size_t(sd)] >= d) continue;
            synced[size_t(best)][size_t(sd)] = d;
            nv.waits.push_back(d);
            nodes_[d].record = true;
            ++n_waits_;
        }
    }

    // Runs of grouped touches.  The reference's engine launches the touches of a group one
    // by one (gpu/exec_graph.cc:354-404); a launch costs more than a small window's copy, and
    // each rereads and rewrites the output.  Nodes v, v+1, .. that are all touches of one
    // group into the same output range (same dtype, same output extents) are folded into one
    // touch_batch launch at v's place: nothing lies between them in launch order, every
    // dependency of a later member is an earlier node, and the chain within the group has
    // put them on one stream.
    for (int v = 0; v < n;) {
        node_t& head = nodes_[v];
        int     end = v + 1;
        if (head.kind == kind_t::touch && head.group >= 0) {
            auto same = [&](node_t const& x) {
                if (x.kind != kind_t::touch || x.group != head.group || x.stream != head.stream ||
                    x.mems[0].offset != head.mems[0].offset || x.mems[0].size != head.mems[0].size ||
                    x.touch.dtype != head.touch.dtype ||
                    x.touch.selection.size() != head.touch.selection.size()) {
                    return false;
                }
                for (size_t d = 0; d != x.touch.selection.size(); ++d) {
                    if (x.touch.selection[d].d_out != head.touch.selection[d].d_out) return false;
                }
                return true;
            };
            while (end < n && same(nodes_[end])) ++end;
        }
        if (end - v >= 2) {
            for (int m = v; m != end; ++m) {
                nodes_[m].batch_head = v;
                head.batch.push_back(m);
            }
        }
        v = end;
    }

    if (km_) {
        check(hipSetDevice(km_->device()), "hipSetDevice");
        streams_.assign(size_t(n_streams), nullptr);  // slot 0 is the caller's stream
        for (int s = 1; s != n_streams; ++s) {
            check(hipStreamCreateWithFlags(&streams_[size_t(s)], hipStreamNonBlocking),
                  "hipStreamCreateWithFlags");
        }
        event_of_.assign(size_t(n), -1);
        for (int v = 0; v != n; ++v) {
            if (!nodes_[v].record) continue;
            hipEvent_t e;
            check(hipEventCreateWithFlags(&e, hipEventDisableTiming), "hipEventCreateWithFlags");
            event_of_[size_t(v)] = int(events_.size());
            events_.push_back(e);
        }
        workspace_.assign(size_t(n_streams), nullptr);
        workspace_bytes_.assign(size_t(n_streams), 0);
        for (node_t const& nd : nodes_) {
            if (nd.kind != kind_t::einsummable) continue;
            uint64_t& need = workspace_bytes_[size_t(nd.stream)];
            need = std::max(need, km_->workspace_size(nd.e));
        }
        for (int s = 0; s != n_streams; ++s) {
            if (workspace_bytes_[size_t(s)] == 0) continue;
            check(hipMalloc(&workspace_[size_t(s)], workspace_bytes_[size_t(s)]), "hipMalloc");
        }
        for (auto& s : slots_) {
            if (s.second.size == 0) continue;
            check(hipHostMalloc(&s.second.host, s.second.size, hipHostMallocDefault),
                  "hipHostMalloc");
        }
        check(hipEventCreateWithFlags(&fork_, hipEventDisableTiming), "hipEventCreateWithFlags");
        for (int s = 1; s != n_streams; ++s) {
            hipEvent_t e;
            check(hipEventCreateWithFlags(&e, hipEventDisableTiming), "hipEventCreateWithFlags");
            joins_.push_back(e);
        }
    }
    finalized_ = true;
}

uint64_t apply_graph_t::node_workspace(int id) const
{
    node_t const& n = nodes_[size_t(id)];
    if (n.kind != kind_t::einsummable || !km_) return 0;
    return km_->workspace_size(n.e);
}

void apply_graph_t::launch_node(int id, hipStream_t stream, void* arena_, void* workspace,
                                uint64_t workspace_bytes, int first_in_group,
                                void (*callback)(void*), void* user) const
{
    if (!finalized_) throw km_error(km_status::not_built, "apply graph: launch before finalize");
    if (!km_) throw km_error(km_status::device, "apply graph: planned without a kernel manager");
    if (id < 0 || id >= int(nodes_.size())) throw km_error(km_status::invalid, "no such node");
    char* const   arena = static_cast<char*>(arena_);
    node_t const& n = nodes_[size_t(id)];
    switch (n.kind) {
        case kind_t::einsummable: {
            plan_t const* p = km_->plan_of(n.e);
            if (!p) throw km_error(km_status::not_built, "apply graph: einsummable not built");
            std::vector<void const*> ptrs;
            for (size_t i = 1; i != n.mems.size(); ++i) ptrs.push_back(arena + n.mems[i].offset);
            km_->run_plan(*p, stream, arena + n.mems[0].offset, ptrs.data(), int(ptrs.size()),
                          workspace, workspace_bytes);
            break;
        }
        case kind_t::touch: {
            touch_t t = n.touch;
            if (n.group >= 0 && first_in_group >= 0) {
                // the graph cleared the castable of the first member inserted; the caller's
                // group manager says which one really runs first
                if (first_in_group) {
                    t.castable = std::nullopt;
                } else if (!t.castable) {
                    t.castable = n.group_castable;
                }
            }
            (*km_)(t, stream, arena + n.mems[0].offset, arena + n.mems[1].offset);
            break;
        }
        default:
            launch(n, stream, arena);
            break;
    }
    if (callback) check(hipLaunchHostFunc(stream, callback, user), "hipLaunchHostFunc");
}

int apply_graph_t::n_launches() const
{
    int count = 0;
    for (node_t const& n : nodes_) {
        if (n.kind == kind_t::dummy) continue;
        if (n.batch_head >= 0 && n.batch_head != n.position) continue;
        ++count;
    }
    return count;
}

void apply_graph_t::launch(node_t const& n, hipStream_t stream, char* arena) const
{
    if (n.kind == kind_t::dummy) return;
    void* const out = arena + n.mems[0].offset;
    switch (n.kind) {
        case kind_t::einsummable: {
            plan_t const* p = km_->plan_of(n.e);
            if (!p) throw km_error(km_status::not_built, "apply graph: einsummable not built");
            void const* inns[8];
            std::vector<void const*> many;
            void const** ptrs = inns;
            size_t const k = n.mems.size() - 1;
            if (k > 8) {
                many.resize(k);
                ptrs = many.data();
            }
            for (size_t i = 0; i != k; ++i) ptrs[i] = arena + n.mems[i + 1].offset;
            km_->run_plan(*p, stream, out, ptrs, int(k), workspace_[size_t(n.stream)],
                          workspace_bytes_[size_t(n.stream)]);
            break;
        }
        case kind_t::touch:
            (*km_)(n.touch, stream, out, arena + n.mems[1].offset);
            break;
        case kind_t::constant:
            km_->constant_fill(n.dtype, n.bits0, n.n0, stream, out);
            break;
        case kind_t::lowertri:
            km_->lowerTri_fill(n.dtype, n.bits0, n.bits1, n.n0, n.n1, n.start, stream, out);
            break;
        case kind_t::copy:
            check(hipMemcpyAsync(out, arena + n.mems[1].offset, n.mems[0].size,
                                 hipMemcpyDeviceToDevice, stream),
                  "hipMemcpyAsync");
            break;
        case kind_t::evict:
            if (n.mems[1].size == 0) break;
            check(hipMemcpyAsync(slot(n.storage_id)->host, arena + n.mems[1].offset,
                                 n.mems[1].size, hipMemcpyDeviceToHost, stream),
                  "hipMemcpyAsync");
            break;
        case kind_t::load:
            if (n.mems[0].size == 0) break;
            check(hipMemcpyAsync(out, slot(n.storage_id)->host, n.mems[0].size,
                                 hipMemcpyHostToDevice, stream),
                  "hipMemcpyAsync");
            break;
        case kind_t::dummy:
            break;
    }
}

void apply_graph_t::run(hipStream_t main, void* arena_) const
{
    if (!finalized_) throw km_error(km_status::not_built, "apply graph: run before finalize");
    if (!km_) throw km_error(km_status::device, "apply graph: planned without a kernel manager");
    char* const arena = static_cast<char*>(arena_);
    size_t const ns = streams_.size();
    auto stream_at = [&](int s) { return s == 0 ? main : streams_[size_t(s)]; };
    if (ns > 1) {
        // Forking the pool streams off a stream that is being captured into a HIP graph
        // crashed inside the HIP runtime (a host-side segmentation fault during the capture):
        // refused here, for every caller.  A graph finalized on one stream can be captured.
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        check(hipStreamIsCapturing(main, &capturing), "hipStreamIsCapturing");
        if (capturing != hipStreamCaptureStatusNone) {
            throw km_error(km_status::invalid,
                           "apply graph: a run on more than one stream cannot be captured into "
                           "a HIP graph; finalize the graph on one stream for that");
        }
        check(hipEventRecord(fork_, main), "hipEventRecord");
        for (size_t s = 1; s != ns; ++s) {
            check(hipStreamWaitEvent(streams_[s], fork_, 0), "hipStreamWaitEvent");
        }
    }
    for (int v : order_) {
        node_t const&     n = nodes_[size_t(v)];
        hipStream_t const st = stream_at(n.stream);
        if (n.batch_head >= 0) {
            if (n.batch_head != v) continue;  // launched with its head
            std::vector<touch_t>     touches;
            std::vector<void const*> inns;
            for (int m : n.batch) {
                node_t const& nm = nodes_[size_t(m)];
                for (int d : nm.waits) {
                    check(hipStreamWaitEvent(st, events_[size_t(event_of_[size_t(d)])], 0),
                          "hipStreamWaitEvent");
                }
                touches.push_back(nm.touch);
                inns.push_back(arena + nm.mems[1].offset);
            }
            km_->touch_batch(touches, st, arena + n.mems[0].offset, inns);
            for (int m : n.batch) {
                if (nodes_[size_t(m)].record) {
                    check(hipEventRecord(events_[size_t(event_of_[size_t(m)])], st),
                          "hipEventRecord");
                }
            }
            continue;
        }
        for (int d : n.waits) {
            check(hipStreamWaitEvent(st, events_[size_t(event_of_[size_t(d)])], 0),
                  "hipStreamWaitEvent");
        }
        launch(n, st, arena);
        if (n.record) {
            check(hipEventRecord(events_[size_t(event_of_[size_t(v)])], st), "hipEventRecord");
        }
    }
    for (size_t s = 1; s != ns; ++s) {
        check(hipEventRecord(joins_[s - 1], streams_[s]), "hipEventRecord");
        check(hipStreamWaitEvent(main, joins_[s - 1], 0), "hipStreamWaitEvent");
    }
}

}  // namespace es
