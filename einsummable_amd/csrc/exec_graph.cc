#include "exec_graph.h"

#include "codegen.h"

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

int apply_graph_t::add_dummy(mem_t range, std::vector<int> const& deps, bool is_del)
{
    node_t n;
    n.kind = kind_t::dummy;
    n.mems = {range};
    n.is_del = is_del && range.size != 0;
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
    static const char* names[] = {"einsummable", "touch", "constant", "lowertri", "copy",
                                  "dummy",       "evict", "load",     "chain"};
    node_t const& n = nodes_[size_t(id)];
    std::string   s = names[int(n.kind)];
    for (mem_t const& m : n.mems) s += " " + std::to_string(m.offset) + ":" + std::to_string(m.size);
    if (n.kind == kind_t::einsummable) s += " | " + n.e.key();
    if (n.kind == kind_t::chain) {
        s += " | " + std::to_string(n.chain_stages) + " stages, the last " + n.e.key();
    }
    return s;
}

std::string apply_graph_t::generated_source(int id) const
{
    node_t const& n = nodes_[size_t(id)];
    if (n.kind == kind_t::chain) return n.chain_plan ? n.chain_plan->source() : std::string();
    if (n.kind != kind_t::einsummable) return std::string();
    einsummable_t const e = n.e.merge_adjacent_dims();
    if (e.is_contraction() || e.join.has_variables()) return std::string();
    try {
        return generate_kernel(e).source;
    } catch (ir_error const&) {
        return std::string();
    }
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

// Two row-major shapes of the same element count cut into the coarsest common pieces:
// `parts_a[i]` / `parts_b[j]` list the pieces (indices into `pieces`) of mode i / j, outermost
// first.  False when a mode of one shape straddles a boundary of the other unevenly
// ([6, 4] against [4, 6]).
bool refine(std::vector<uint64_t> const& a, std::vector<uint64_t> const& b,
            std::vector<uint64_t>& pieces, std::vector<std::vector<int>>& parts_a,
            std::vector<std::vector<int>>& parts_b)
{
    std::vector<uint64_t>         rev;  // innermost first
    std::vector<std::vector<int>> pa(a.size()), pb(b.size());
    int      i = int(a.size()) - 1, j = int(b.size()) - 1;
    uint64_t ra = i >= 0 ? a[size_t(i)] : 1, rb = j >= 0 ? b[size_t(j)] : 1;
    while (i >= 0 && j >= 0) {
        uint64_t const g = std::min(ra, rb);
        if (ra % g != 0 || rb % g != 0) return false;
        int const id = int(rev.size());
        rev.push_back(g);
        pa[size_t(i)].push_back(id);
        pb[size_t(j)].push_back(id);
        ra /= g;
        rb /= g;
        if (ra == 1 && --i >= 0) ra = a[size_t(i)];
        if (rb == 1 && --j >= 0) rb = b[size_t(j)];
    }
    // what is left on either side can only be modes of extent one
    for (; i >= 0; --i) {
        if (ra != 1) return false;
        if (i > 0) ra = a[size_t(i - 1)];
    }
    for (; j >= 0; --j) {
        if (rb != 1) return false;
        if (j > 0) rb = b[size_t(j - 1)];
    }
    int const n = int(rev.size());
    pieces.assign(rev.rbegin(), rev.rend());
    auto flip = [&](std::vector<std::vector<int>>& p) {
        for (auto& v : p) {
            for (int& x : v) x = n - 1 - x;
            std::reverse(v.begin(), v.end());
        }
    };
    flip(pa);
    flip(pb);
    parts_a = pa;
    parts_b = pb;
    return true;
}

std::vector<int> expand(std::vector<int> const& inn, std::vector<std::vector<int>> const& parts)
{
    std::vector<int> r;
    for (int m : inn) r.insert(r.end(), parts[size_t(m)].begin(), parts[size_t(m)].end());
    return r;
}

// The einsummable that computes v with u in place of its input k, or nothing when the two
// do not line up.  v reads input k position by position over its join modes; u has no
// aggregation.  The two may cut the same elements into modes differently ([32, 4194304]
// against [65536, 2048]): both are rewritten over the common pieces first.
// exactly to_<to>[hole|<from>@0] over one straight input
bool is_plain_conversion(einsummable_t const& e, dtype_t from, dtype_t to)
{
    node_t const& r = e.join.root;
    return !e.has_aggregation() && e.inns.size() == 1 && is_iota(e.inns[0], int(e.join_shape.size())) &&
           !e.any_half_pairs() && r.kind == op_kind::convert && r.dtype == to && r.children.size() == 1 &&
           r.children[0].kind == op_kind::hole && r.children[0].arg == 0 && r.children[0].dtype == from;
}

// Conversions around a complex view.  A complex node that reads, as c64, the f32 tensor a
// conversion from f16 has just written takes the f16 tensor itself, pairs of f16 widened on
// the load (u the conversion, v the complex node); a conversion to f16 that reads, as f32,
// what a complex node wrote becomes that node with its result rounded to pairs of f16 on
// the store (u the complex node, v the conversion).  Rotary embeddings are spelled that
// way: to_f32, the product with the frequencies on the buffer seen as complex, to_f16.
std::optional<einsummable_t> merged_across_a_complex_view(einsummable_t const& u,
                                                         einsummable_t const& v, int k)
{
    int const rank_v = int(v.join_shape.size());
    if (u.out_dtype() == dtype_t::f32 && v.inn_dtype(k) == dtype_t::c64) {
        if (!is_plain_conversion(u, dtype_t::f16, dtype_t::f32) || v.has_aggregation() ||
            u.out_nelem() != 2 * v.inn_nelem(k) || !is_iota(v.inns[size_t(k)], rank_v) ||
            v.stored_as_half_pairs(1 + k)) {
            return std::nullopt;
        }
        scalarop_t identity;
        identity.root.kind = op_kind::hole;
        identity.root.dtype = dtype_t::c64;
        identity.root.arg = 0;
        identity.hole_dtypes = {dtype_t::c64};
        std::vector<std::vector<int>> inns{v.inns[size_t(k)]};
        std::vector<char>             half(v.inns.size() + 1, 0);
        half[0] = v.stored_as_half_pairs(0);
        half[1] = 1;
        for (int i = 0, at = 2; i != int(v.inns.size()); ++i) {
            if (i == k) continue;
            inns.push_back(v.inns[size_t(i)]);
            half[size_t(at++)] = v.stored_as_half_pairs(1 + i);
        }
        try {
            einsummable_t r = einsummable_t::make(v.join_shape, inns, v.out_rank,
                                                  scalarop_t::compose(v.join, k, identity), v.castable);
            r.half_complex = half;
            return r;
        } catch (ir_error const&) {
            return std::nullopt;
        }
    }
    if (u.out_dtype() == dtype_t::c64 && v.inn_dtype(k) == dtype_t::f32) {
        if (!is_plain_conversion(v, dtype_t::f32, dtype_t::f16) || u.has_aggregation() ||
            v.out_nelem() != 2 * u.out_nelem() || u.stored_as_half_pairs(0)) {
            return std::nullopt;
        }
        einsummable_t r = u;
        r.half_complex.resize(u.inns.size() + 1, 0);
        r.half_complex[0] = 1;
        return r;
    }
    return std::nullopt;
}

std::optional<einsummable_t> merged(einsummable_t const& u, einsummable_t const& v, int k)
{
    if ((u.out_dtype() == dtype_t::f32 && v.inn_dtype(k) == dtype_t::c64) ||
        (u.out_dtype() == dtype_t::c64 && v.inn_dtype(k) == dtype_t::f32)) {
        return merged_across_a_complex_view(u, v, k);
    }
    if (u.any_half_pairs() || v.any_half_pairs()) return std::nullopt;
    if (u.out_dtype() != v.inn_dtype(k) || u.out_nelem() != v.inn_nelem(k)) return std::nullopt;
    if (u.inns.size() + v.inns.size() - 1 > 6) return std::nullopt;
    std::vector<uint64_t>         shape;
    std::vector<std::vector<int>> pu, pv;
    if (!refine(u.join_shape, v.join_shape, shape, pu, pv)) return std::nullopt;
    if (shape.size() > 8) return std::nullopt;
    int out_rank = 0;
    for (int m = 0; m != v.out_rank; ++m) out_rank += int(pv[size_t(m)].size());
    if (out_rank == 0) return std::nullopt;
    std::vector<std::vector<int>> inns;
    for (auto const& inn : u.inns) inns.push_back(expand(inn, pu));
    for (int i = 0; i != int(v.inns.size()); ++i) {
        if (i != k) inns.push_back(expand(v.inns[size_t(i)], pv));
    }
    // einsummable_t::make numbers aggregated modes by first appearance: they must already
    // appear in ascending order, or extents and modes would part ways
    int next = out_rank;
    for (auto const& inn : inns) {
        if (inn.empty()) return std::nullopt;
        for (int m : inn) {
            if (m > next) return std::nullopt;
            if (m == next) ++next;
        }
    }
    try {
        return einsummable_t::make(shape, inns, out_rank, scalarop_t::compose(v.join, k, u.join),
                                   v.castable);
    } catch (ir_error const&) {
        return std::nullopt;
    }
}

// Smallest element among the output and the inputs: the generated reductions take 16 bytes of
// it per lane, so it decides how a row's elements are dealt to the lanes, i.e. the order of
// the sum.
uint64_t smallest_element(einsummable_t const& e)
{
    uint64_t m = dtype_size(e.out_dtype());
    for (int k = 0; k != int(e.inns.size()); ++k) m = std::min(m, dtype_size(e.inn_dtype(k)));
    return m;
}

uint64_t input_bytes(einsummable_t const& e)
{
    uint64_t b = 0;
    for (int k = 0; k != int(e.inns.size()); ++k) b += e.inn_nelem(k) * dtype_size(e.inn_dtype(k));
    return b;
}

}  // namespace

// Tries to make node u's output unnecessary: every node that reads it computes it for itself
// (or, for a whole-range copy, u writes the copy's output).  True when u became a dummy.
bool apply_graph_t::absorb_into_readers(int u)
{
    int const n = int(nodes_.size());
    node_t&   nu = nodes_[size_t(u)];
    if (nu.kind != kind_t::einsummable) return false;
    mem_t const S = nu.mems[0];
    if (S.size == 0) return false;
    for (size_t i = 1; i != nu.mems.size(); ++i) {
        if (overlaps(nu.mems[i], S)) return false;
    }
    // who reads S before it is deleted; nobody may rewrite it or, while readers are still to
    // come, what u reads
    std::vector<int> readers, slots;
    bool             deleted = false, clobbered = false;
    for (int w = u + 1; w < n && !deleted; ++w) {
        node_t const& nw = nodes_[size_t(w)];
        if (nw.kind == kind_t::dummy) {
            deleted = nw.is_del && !readers.empty() && covers(nw.mems[0], S) &&
                      std::binary_search(nw.deps.begin(), nw.deps.end(), readers.back());
            continue;
        }
        bool const writes = nw.kind != kind_t::evict;
        int        slot = -1, touching = 0;
        for (size_t i = 1; i < nw.mems.size(); ++i) {
            if (!overlaps(nw.mems[i], S)) continue;
            ++touching;
            if (same_range(nw.mems[i], S)) slot = int(i);
        }
        if (touching) {
            if (touching != 1 || slot < 0 || clobbered) return false;
            if (writes && overlaps(nw.mems[0], S)) return false;
            for (size_t i = 1; writes && i != nu.mems.size(); ++i) {
                if (overlaps(nw.mems[0], nu.mems[i])) return false;  // it would overwrite what it now reads
            }
            readers.push_back(w);
            slots.push_back(slot);
            continue;
        }
        if (!writes) continue;
        if (overlaps(nw.mems[0], S)) return false;
        for (size_t i = 1; i != nu.mems.size(); ++i) clobbered = clobbered || overlaps(nw.mems[0], nu.mems[i]);
    }
    if (!deleted || readers.empty()) return false;

    // what each reader becomes
    std::vector<einsummable_t> fused;
    node_t const&              first = nodes_[size_t(readers[0])];
    bool const copy = readers.size() == 1 && first.kind == kind_t::touch;
    if (copy) {
        touch_t const t = first.touch.simplify();
        if (t.castable || t.selection.size() != 1) return false;
        touchdim_t const& d = t.selection[0];
        if (d.d_inn != d.size || d.d_out != d.size || d.offset_inn || d.offset_out) return false;
        if (d.size * dtype_size(t.dtype) != first.mems[0].size || first.mems[1].size != first.mems[0].size) {
            return false;
        }
        for (int w = 0; first.group >= 0 && w != n; ++w) {
            if (w != readers[0] && nodes_[size_t(w)].kind == kind_t::touch &&
                nodes_[size_t(w)].group == first.group) {
                return false;
            }
        }
        fused.push_back(nu.e);
    } else {
        if (!absorbable_producer(nu.e)) return false;
        // every reader repeats u's reads; worth it while that is less than writing S once and
        // reading it once per reader
        uint64_t const in_u = input_bytes(nu.e), nr = readers.size();
        if (nr > 1 && (nr - 1) * in_u >= (nr + 1) * S.size) return false;
        for (size_t r = 0; r != readers.size(); ++r) {
            node_t const& nv = nodes_[size_t(readers[r])];
            if (nv.kind != kind_t::einsummable) return false;
            einsummable_t const& e = nv.e;
            int const            k = slots[r] - 1;
            if (e.join.has_variables() || (e.has_aggregation() && e.inns.size() != 1)) return false;
            if (!is_iota(e.inns[size_t(k)], int(e.join_shape.size()))) return false;
            std::optional<einsummable_t> m = merged(nu.e, e, k);
            if (!m) return false;
            // A sum (or product) keeps its bits only if its elements are added in the same
            // order: dealt to the lanes in the same way (row reductions deal 2- and 4-byte
            // elements alike), over the same innermost extent.  min and max do not care.
            if (e.has_aggregation() && (e.castable.value() == castable_t::add ||
                                        e.castable.value() == castable_t::mul)) {
                bool const row = is_row_reduction(e);
                bool const same_deal =
                    row ? row_reduction_lane_elems(int(smallest_element(m.value()))) ==
                              row_reduction_lane_elems(int(smallest_element(e)))
                        : smallest_element(m.value()) == smallest_element(e);
                if (row != is_row_reduction(m.value()) || !same_deal ||
                    m.value().join_shape.back() != e.join_shape.back()) {
                    return false;
                }
            }
            if (km_) {
                try {
                    // (compiled at finalize, with the graph's other kernels)
                    if (!km_->buildable(m.value())) return false;
                } catch (km_error const&) {
                    return false;
                } catch (ir_error const&) {
                    return false;
                }
            }
            fused.push_back(std::move(m.value()));
        }
    }

    // Who waits for u: u itself and every dummy that, through dummies, depends on it (the
    // del of one of u's inputs stands right behind u, before the readers).  A node that
    // depends on any of them was promised that u is done with its inputs; those are now read
    // by the readers.
    std::vector<char> waits_for_u(size_t(n), 0);
    waits_for_u[size_t(u)] = 1;
    for (int w = u + 1; w < n; ++w) {
        node_t const& nw = nodes_[size_t(w)];
        if (nw.kind != kind_t::dummy) continue;
        for (int d : nw.deps) {
            if (waits_for_u[size_t(d)]) {
                waits_for_u[size_t(w)] = 1;
                break;
            }
        }
    }
    for (size_t r = 0; r != readers.size(); ++r) {
        int const v = readers[r];
        node_t&   nv = nodes_[size_t(v)];
        std::vector<mem_t> mems{nv.mems[0]};
        for (size_t i = 1; i != nu.mems.size(); ++i) mems.push_back(nu.mems[i]);
        for (size_t i = 1; i != nv.mems.size(); ++i) {
            if (!copy && int(i) != slots[r]) mems.push_back(nv.mems[i]);
        }
        std::vector<int> deps = nv.deps;
        deps.erase(std::remove(deps.begin(), deps.end(), u), deps.end());
        deps.insert(deps.end(), nu.deps.begin(), nu.deps.end());
        std::sort(deps.begin(), deps.end());
        deps.erase(std::unique(deps.begin(), deps.end()), deps.end());
        nv.kind = kind_t::einsummable;
        nv.e = std::move(fused[r]);
        nv.mems = std::move(mems);
        nv.deps = std::move(deps);
        nv.group = -1;
        // whoever waited for u to be done with its inputs waits for the nodes that read them now
        // (the other readers only shared u with this one)
        for (int w = v + 1; w < n; ++w) {
            if (std::find(readers.begin(), readers.end(), w) != readers.end()) continue;
            std::vector<int>& d = nodes_[size_t(w)].deps;
            bool const promised = std::any_of(d.begin(), d.end(),
                                              [&](int x) { return waits_for_u[size_t(x)] != 0; });
            if (promised && !std::binary_search(d.begin(), d.end(), v)) {
                d.insert(std::upper_bound(d.begin(), d.end(), v), v);
            }
        }
    }
    nu.kind = kind_t::dummy;
    nu.mems = {S};
    nu.is_del = false;
    return true;
}

// Tries to make node v, an elementwise einsummable, the last stage of a chain over rows: the
// producers of its per-row inputs (and of theirs) that are row reductions over v's shape or
// pointwise nodes over its rows, whose outputs nobody else reads and which are deleted
// afterwards.  Returns the number of nodes absorbed (0: v stays as it is).
int apply_graph_t::fuse_row_chain(int v)
{
    int const n = int(nodes_.size());
    node_t&   nv = nodes_[size_t(v)];
    if (nv.kind != kind_t::einsummable || nv.e.has_aggregation() || nv.e.join.has_variables() ||
        nv.e.any_half_pairs()) {
        return 0;
    }
    int const R = int(nv.e.join_shape.size());
    if (R < 2) return 0;
    int const O = R - 1;
    std::vector<uint64_t> const shape = nv.e.join_shape;
    std::vector<uint64_t> const rows(shape.begin(), shape.begin() + O);

    // members in the order found; producer_of[(member, slot)] = member index
    std::vector<int> members{v};
    struct link_t {
        int member, slot, producer;
    };
    std::vector<link_t> links;
    auto writer_of = [&](mem_t const& m, int before) {
        for (int u = before - 1; u >= 0; --u) {
            node_t const& nu = nodes_[size_t(u)];
            if (nu.kind == kind_t::dummy || nu.kind == kind_t::evict) continue;
            if (overlaps(nu.mems[0], m)) return same_range(nu.mems[0], m) ? u : -1;
        }
        return -1;
    };
    auto stage_kind = [&](einsummable_t const& e) {  // 1 reduction over the row, 2 pointwise on rows
        if (e.join.has_variables() || e.any_half_pairs()) return 0;
        if (e.has_aggregation()) return e.join_shape == shape && e.out_rank == O ? 1 : 0;
        return e.join_shape == rows ? 2 : 0;
    };
    for (size_t at = 0; at != members.size(); ++at) {
        node_t const& nm = nodes_[size_t(members[at])];
        for (size_t k = 0; k != nm.e.inns.size(); ++k) {
            if (!is_iota(nm.e.inns[k], O)) continue;
            int const u = writer_of(nm.mems[k + 1], members[at]);
            if (u < 0 || nodes_[size_t(u)].kind != kind_t::einsummable) continue;
            if (!stage_kind(nodes_[size_t(u)].e)) continue;
            if (std::find(members.begin(), members.end(), u) == members.end()) members.push_back(u);
            links.push_back({members[at], int(k), u});
        }
    }
    if (members.size() < 2) return 0;

    // A producer stays a member only if its output is read by members alone, through the
    // links found, and deleted after the last of them.  One that does not qualify is an
    // ordinary input; members that hang on it alone go with it.
    auto qualifies = [&](int u, std::vector<int> const& in) {
        mem_t const S = nodes_[size_t(u)].mems[0];
        if (S.size == 0) return false;
        for (size_t i = 1; i != nodes_[size_t(u)].mems.size(); ++i) {
            if (overlaps(nodes_[size_t(u)].mems[i], S)) return false;
        }
        int  last_reader = -1;
        bool deleted = false;
        for (int w = u + 1; w < n && !deleted; ++w) {
            node_t const& nw = nodes_[size_t(w)];
            if (nw.kind == kind_t::dummy) {
                deleted = nw.is_del && last_reader >= 0 && covers(nw.mems[0], S) &&
                          std::binary_search(nw.deps.begin(), nw.deps.end(), last_reader);
                continue;
            }
            bool reads = false;
            for (size_t i = 1; i < nw.mems.size(); ++i) {
                if (!overlaps(nw.mems[i], S)) continue;
                bool linked = false;
                for (link_t const& l : links) {
                    linked = linked || (l.member == w && l.slot + 1 == int(i) && l.producer == u);
                }
                if (!linked || std::find(in.begin(), in.end(), w) == in.end()) return false;
                reads = true;
            }
            if (reads) last_reader = w;
            if (nw.kind != kind_t::evict && overlaps(nw.mems[0], S)) return false;
        }
        return deleted;
    };
    for (bool changed = true; changed;) {
        changed = false;
        for (size_t i = 1; i < members.size(); ++i) {
            if (qualifies(members[i], members)) continue;
            members.erase(members.begin() + long(i));
            changed = true;
            break;
        }
        // members no link from a member reaches any more
        for (size_t i = 1; i < members.size() && !changed; ++i) {
            bool reached = false;
            for (link_t const& l : links) {
                reached = reached || (l.producer == members[i] &&
                                      std::find(members.begin(), members.end(), l.member) != members.end());
            }
            if (!reached) {
                members.erase(members.begin() + long(i));
                changed = true;
            }
        }
    }
    if (members.size() < 2) return 0;
    std::sort(members.begin(), members.end());  // insertion order is a valid order of execution
    bool any_reduction = false;
    for (int m : members) any_reduction = any_reduction || nodes_[size_t(m)].e.has_aggregation();
    if (!any_reduction) return 0;
    auto stage_of = [&](int node) {
        return int(std::find(members.begin(), members.end(), node) - members.begin());
    };

    // the chain's inputs and stages
    cg_chain_t         c;
    std::vector<mem_t> ext_mems;
    c.shape = shape;
    mem_t const P = nv.mems[0];
    if (P.offset % 16) return 0;
    for (int m : members) {
        node_t const&       nm = nodes_[size_t(m)];
        cg_chain_t::stage_t st;
        st.join = nm.e.join;
        st.castable = nm.e.castable;
        for (size_t k = 0; k != nm.e.inns.size(); ++k) {
            int producer = -1;
            for (link_t const& l : links) {
                if (l.member == m && l.slot == int(k) &&
                    std::find(members.begin(), members.end(), l.producer) != members.end()) {
                    producer = l.producer;
                }
            }
            if (producer >= 0) {
                st.args.push_back(-1 - stage_of(producer));
                continue;
            }
            mem_t const&     mem = nm.mems[k + 1];
            dtype_t const    dt = nm.e.inn_dtype(int(k));
            std::vector<int> modes = nm.e.inns[k];
            if (!is_increasing(modes) || mem.offset % 16) return 0;
            if (!modes.empty() && modes.back() > R - 1) return 0;
            int found = -1;
            for (size_t x = 0; x != ext_mems.size(); ++x) {
                if (same_range(ext_mems[x], mem) && c.exts[x].dtype == dt && c.exts[x].modes == modes) {
                    found = int(x);
                }
            }
            if (found < 0) {
                // the output may lie exactly on an input it is computed from, nowhere else
                if (overlaps(P, mem) &&
                    !(same_range(P, mem) && is_iota(modes, R) &&
                      dtype_size(dt) == dtype_size(nv.e.out_dtype()))) {
                    return 0;
                }
                found = int(ext_mems.size());
                ext_mems.push_back(mem);
                c.exts.push_back({dt, modes});
            }
            st.args.push_back(found);
        }
        c.stages.push_back(std::move(st));
    }
    if (c.exts.size() > 8) return 0;
    // the intermediate results lie apart from everything the chain touches
    for (int m : members) {
        if (m == v) continue;
        mem_t const& S = nodes_[size_t(m)].mems[0];
        if (overlaps(S, P)) return 0;
        for (mem_t const& x : ext_mems) {
            if (overlaps(S, x)) return 0;
        }
    }
    // nobody between the first member and v may rewrite what the chain reads (it is read at
    // v's place now)
    for (int w = members.front() + 1; w < v; ++w) {
        node_t const& nw = nodes_[size_t(w)];
        if (nw.kind == kind_t::dummy || nw.kind == kind_t::evict) continue;
        if (std::find(members.begin(), members.end(), w) != members.end()) continue;
        for (mem_t const& m : ext_mems) {
            if (overlaps(nw.mems[0], m)) return 0;
        }
    }
    std::shared_ptr<plan_t> plan;
    try {
        if (km_) check(hipSetDevice(km_->device()), "hipSetDevice");
        // (compiled at finalize, all chains of the graph as one program)
        plan = plan_row_chain(c, km_ ? km_->device() : -1, true);
    } catch (ir_error const&) {
        return 0;
    } catch (km_error const&) {
        return 0;
    }

    // v stands for the whole chain; the others become dummies
    std::vector<char> waits_for(size_t(n), 0);
    std::vector<int>  deps;
    for (int m : members) {
        if (m != v) waits_for[size_t(m)] = 1;
        deps.insert(deps.end(), nodes_[size_t(m)].deps.begin(), nodes_[size_t(m)].deps.end());
    }
    for (int w = members.front() + 1; w < n; ++w) {
        node_t const& nw = nodes_[size_t(w)];
        if (nw.kind != kind_t::dummy) continue;
        for (int d : nw.deps) {
            if (waits_for[size_t(d)]) {
                waits_for[size_t(w)] = 1;
                break;
            }
        }
    }
    deps.erase(std::remove_if(deps.begin(), deps.end(),
                              [&](int d) {
                                  return std::find(members.begin(), members.end(), d) != members.end();
                              }),
               deps.end());
    std::sort(deps.begin(), deps.end());
    deps.erase(std::unique(deps.begin(), deps.end()), deps.end());
    // whoever waited for an absorbed node to be done with its inputs waits for v, which reads
    // them now
    for (int w = v + 1; w < n; ++w) {
        std::vector<int>& d = nodes_[size_t(w)].deps;
        bool const promised =
            std::any_of(d.begin(), d.end(), [&](int x) { return waits_for[size_t(x)] != 0; });
        if (promised && !std::binary_search(d.begin(), d.end(), v)) {
            d.insert(std::upper_bound(d.begin(), d.end(), v), v);
        }
    }
    for (int m : members) {
        if (m == v) continue;
        node_t& nm = nodes_[size_t(m)];
        mem_t const S = nm.mems[0];
        nm.kind = kind_t::dummy;
        nm.mems = {S};
        nm.is_del = false;
    }
    nv.kind = kind_t::chain;
    nv.mems = {P};
    nv.mems.insert(nv.mems.end(), ext_mems.begin(), ext_mems.end());
    nv.deps = std::move(deps);
    nv.chain_plan = std::move(plan);
    nv.chain_stages = int(members.size());
    return int(members.size()) - 1;
}

int apply_graph_t::optimize()
{
    if (finalized_) throw km_error(km_status::invalid, "apply graph: already finalized");
    int absorbed = 0;
    for (int u = 0; u != int(nodes_.size()); ++u) {
        if (absorb_into_readers(u)) ++absorbed;
    }
    const char* env = std::getenv("ES_KM_ROW_CHAINS");
    if (!(env && env[0] == '0')) {
        for (int v = 0; v != int(nodes_.size()); ++v) absorbed += fuse_row_chain(v);
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
        // the graph's distinct einsummables are built together, on several threads
        std::vector<einsummable_t> es;
        for (node_t const& nd : nodes_) {
            if (nd.kind == kind_t::einsummable) es.push_back(nd.e);
        }
        for (std::optional<uint64_t> const& ws : km_->build_many(es)) {
            if (!ws) {
                throw km_error(km_status::invalid, "apply graph: no kernel for an einsummable "
                                                   "(build returned unsupported)");
            }
        }
        // ... and so are the chains over rows that optimize() made
        std::vector<plan_t*> waiting;
        for (node_t const& nd : nodes_) {
            if (nd.kind == kind_t::chain && nd.chain_plan) nd.chain_plan->deferred(waiting);
        }
        if (!waiting.empty()) {
            check(hipSetDevice(km_->device()), "hipSetDevice");
            finish_codegen_plans(waiting, km_->device());
        }
    }

    // Placement, in launch order.  A node continues the stream of a dependency that is
    // still the last node of its stream (the most recent such dependency): that needs no
    // wait at all.  Otherwise it takes the stream whose last node is oldest, and independent
    // branches spread over the pool.
    // A node that moves 4 MiB or more fills the device by itself: beside another one it gains
    // nothing, while every change of stream costs an event and a wait (some microseconds
    // each; the LLaMA-7B layer's 28 launches took 1.58 ms spread over four streams and 1.44
    // on one).  Such nodes all go to the first stream, in launch order; the pool is for the
    // small ones.
    auto wide = [](node_t const& x) {
        if (x.kind == kind_t::dummy) return false;
        uint64_t bytes = 0;
        for (mem_t const& m : x.mems) bytes += m.size;
        return bytes >= (4ull << 20);
    };
    std::vector<int> last(size_t(n_streams), -1);
    std::vector<std::vector<int>> synced(size_t(n_streams), std::vector<int>(size_t(n_streams), -1));
    order_.resize(size_t(n));
    n_waits_ = 0;
    // A dummy launches nothing: it takes no place on a stream and nobody waits for it; who
    // depends on it depends on what it depends on.
    std::vector<std::vector<int>> real_deps{size_t(n)};
    for (int v = 0; v != n; ++v) {
        node_t& nv = nodes_[v];
        nv.position = v;
        order_[size_t(v)] = v;
        std::vector<int>& deps = real_deps[size_t(v)];
        for (int d : nv.deps) {
            if (nodes_[d].kind == kind_t::dummy) {
                deps.insert(deps.end(), real_deps[size_t(d)].begin(), real_deps[size_t(d)].end());
            } else {
                deps.push_back(d);
            }
        }
        std::sort(deps.begin(), deps.end(), [](int x, int y) { return x > y; });
        deps.erase(std::unique(deps.begin(), deps.end()), deps.end());
        nv.waits.clear();
        if (nv.kind == kind_t::dummy) {
            nv.stream = 0;
            continue;
        }
        bool const first_stream = wide(nv);
        int        best = first_stream ? 0 : -1;
        for (int d : deps) {
            if (first_stream) break;
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
        // launched before it (deps: latest first)
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

    // A pool stream is forked off the caller's stream only if it holds a node, and joined at
    // the end only if its last node is not already waited for by a node of the first stream:
    // each fork and join is an event and a wait that the first stream pays for.
    stream_used_.assign(size_t(n_streams), 0);
    stream_joins_.assign(size_t(n_streams), 0);
    for (int s = 1; s != n_streams; ++s) {
        stream_used_[size_t(s)] = last[size_t(s)] >= 0;
        stream_joins_[size_t(s)] = last[size_t(s)] >= 0 && synced[0][size_t(s)] < last[size_t(s)];
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

    // Runs of sibling products.  Einsummables of one key that follow each other in launch
    // order (dummies aside) on one stream, none depending on another -- the q, k and v
    // projections of one input, w1 and w3 -- go out as one launch when their kernel takes
    // several runs at once (plan_t::max_group): at the first one's place, like the touches.
    for (int v = 0; km_ && v < n; ++v) {
        node_t& head = nodes_[v];
        if (head.kind != kind_t::einsummable || head.batch_head >= 0) continue;
        plan_t const* const plan = km_->plan_of(head.e);
        int const           cap = plan ? plan->max_group() : 1;
        if (cap < 2) continue;
        std::string const key = head.e.merge_adjacent_dims().key();
        std::vector<int>  members{v};
        for (int w = v + 1; w < n && int(members.size()) < cap; ++w) {
            node_t const& x = nodes_[w];
            if (x.kind == kind_t::dummy) continue;
            if (x.kind != kind_t::einsummable || x.batch_head >= 0 || x.stream != head.stream ||
                x.e.merge_adjacent_dims().key() != key) {
                break;
            }
            // independent of the members before it: what it waits for lies before the head
            bool early = true;
            for (int d : real_deps[size_t(w)]) early = early && d < v;
            if (!early) break;
            members.push_back(w);
        }
        if (members.size() < 2) continue;
        for (int m : members) {
            nodes_[m].batch_head = v;
            head.batch.push_back(m);
        }
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
        case kind_t::chain: {
            if (!n.chain_plan) throw km_error(km_status::not_built, "apply graph: chain not built");
            void const*  ptrs[8];
            size_t const k = n.mems.size() - 1;
            for (size_t i = 0; i != k; ++i) ptrs[i] = arena + n.mems[i + 1].offset;
            km_->run_plan(*n.chain_plan, stream, out, ptrs, int(k), nullptr, 0);
            break;
        }
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
        bool forked = false;
        for (size_t s = 1; s != ns; ++s) {
            if (!stream_used_[s]) continue;
            if (!forked) check(hipEventRecord(fork_, main), "hipEventRecord");
            forked = true;
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
            std::vector<void*>       outs;
            for (int m : n.batch) {
                node_t const& nm = nodes_[size_t(m)];
                for (int d : nm.waits) {
                    check(hipStreamWaitEvent(st, events_[size_t(event_of_[size_t(d)])], 0),
                          "hipStreamWaitEvent");
                }
                if (n.kind == kind_t::einsummable) {
                    outs.push_back(arena + nm.mems[0].offset);
                    for (size_t i = 1; i != nm.mems.size(); ++i) inns.push_back(arena + nm.mems[i].offset);
                } else {
                    touches.push_back(nm.touch);
                    inns.push_back(arena + nm.mems[1].offset);
                }
            }
            if (n.kind == kind_t::einsummable) {
                plan_t const* const plan = km_->plan_of(n.e);
                if (!plan) throw km_error(km_status::not_built, "apply graph: einsummable not built");
                plan->run_group(st, int(outs.size()), outs.data(), inns.data());
            } else {
                km_->touch_batch(touches, st, arena + n.mems[0].offset, inns);
            }
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
        if (!stream_joins_[s]) continue;
        check(hipEventRecord(joins_[s - 1], streams_[s]), "hipEventRecord");
        check(hipStreamWaitEvent(main, joins_[s - 1], 0), "hipStreamWaitEvent");
    }
}

}  // namespace es
