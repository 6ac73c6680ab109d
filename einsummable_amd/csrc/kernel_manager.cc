#include "kernel_manager.h"

#include "launch.h"
#include "static_workspace.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdlib>
#include <cstring>

namespace es
{

namespace
{

void hip_check(hipError_t err, const char* what)
{
    if (err != hipSuccess) {
        throw km_error(km_status::device, std::string(what) + ": " + hipGetErrorString(err));
    }
}

// An elementwise node one of whose inputs is laid out with another inner mode than the output
// (say ab,ba->ab): read in place, that input is gathered element by element, every lane a
// cache line of its own (1.0-1.4 TB/s on 8192 x 8192 f16).  Such an input is first brought
// into the output's mode order by the LDS transpose, into the workspace, and the elementwise
// kernel then reads only rows: two more passes over that input, all of them at row speed.
struct staged_plan_t : plan_t {
    struct stage_t {
        int                     input;
        std::shared_ptr<plan_t> plan;
        uint64_t                offset;
    };
    std::vector<stage_t>    stages;
    std::shared_ptr<plan_t> main;
    uint64_t                main_offset = 0;

    void run(hipStream_t stream, void* out, void const* const* inns, void* workspace,
             uint64_t) const override
    {
        std::vector<void const*> ptrs(inns, inns + n_inns);
        char* const              ws = static_cast<char*>(workspace);
        for (stage_t const& s : stages) {
            void const* one[1] = {inns[s.input]};
            s.plan->run(stream, ws + s.offset, one, nullptr, 0);
            ptrs[size_t(s.input)] = ws + s.offset;
        }
        main->run(stream, out, ptrs.data(), main->workspace_bytes ? ws + main_offset : nullptr,
                  main->workspace_bytes);
    }
    void deferred(std::vector<plan_t*>& out) override { main->deferred(out); }
};

std::shared_ptr<plan_t> plan_staged_elementwise(einsummable_t const& e, int device, bool defer = false)
{
    if (e.has_aggregation()) return nullptr;
    int const R = int(e.join_shape.size());
    if (R < 2) return nullptr;
    // measured on ab,ba->ab: 2 M elements is where the extra launch is paid for (f16: 12.0
    // against 13.8 us at 4 MiB, 11.2 against 9.0 at 2 MiB; f32: 16.7 against 17.6 us at 8 MiB)
    uint64_t min_elems = 1ull << 21;
    if (const char* env = std::getenv("ES_KM_EW_STAGE_MIN")) {  // tuning and tests; 0: never
        min_elems = std::strtoull(env, nullptr, 10);
        if (min_elems == 0) return nullptr;
    }
    auto           plan = std::make_shared<staged_plan_t>();
    einsummable_t  main = e;
    uint64_t       offset = 0;
    std::string    what;
    for (int k = 0; k != int(e.inns.size()); ++k) {
        std::vector<int> const& inn = e.inns[size_t(k)];
        auto const              at = std::find(inn.begin(), inn.end(), R - 1);
        if (at == inn.end() || at + 1 == inn.end()) continue;  // broadcast along, or rows of, R-1
        dtype_t const  dt = e.inn_dtype(k);
        uint64_t const bytes = e.inn_nelem(k) * dtype_size(dt);
        if (e.inn_nelem(k) < min_elems) continue;
        std::vector<int> sorted = inn;
        std::sort(sorted.begin(), sorted.end());
        std::vector<uint64_t> shape;
        for (int m : sorted) shape.push_back(e.join_shape[size_t(m)]);
        std::vector<int> from;  // the input's modes, numbered by their place in the sorted order
        for (int m : inn) {
            from.push_back(int(std::find(sorted.begin(), sorted.end(), m) - sorted.begin()));
        }
        einsummable_t perm = einsummable_t::make(
            shape, {from}, int(sorted.size()),
            scalarop_t::parse(std::string("hole|") + dtype_name(dt) + "@0"), std::nullopt);
        perm = perm.merge_adjacent_dims();
        std::shared_ptr<plan_t> pp = plan_transpose(perm, device);
        if (!pp || pp->workspace_bytes != 0) return nullptr;
        pp->n_inns = 1;
        plan->stages.push_back({k, pp, offset});
        offset += (bytes + 255) / 256 * 256;
        main.inns[size_t(k)] = sorted;
        what += (what.empty() ? "" : "; ") + std::string("input ") + std::to_string(k) + ": " +
                pp->description;
    }
    if (plan->stages.empty()) return nullptr;
    main = main.merge_adjacent_dims();
    plan->main = plan_codegen(main, device, defer);
    if (!plan->main) return nullptr;
    plan->main->n_inns = int(main.inns.size());
    plan->main_offset = offset;
    plan->workspace_bytes = offset + plan->main->workspace_bytes;
    plan->description = "staged [" + what + "] then " + plan->main->description;
    return plan;
}

}  // namespace

kernel_manager_t::kernel_manager_t(int device) : device_(device)
{
    int count = 0;
    hip_check(hipGetDeviceCount(&count), "hipGetDeviceCount");
    if (device < 0 || device >= count) {
        throw km_error(km_status::device, "kernel_manager_t: no such device " +
                                              std::to_string(device) + " (" +
                                              std::to_string(count) + " visible)");
    }
    hip_check(hipSetDevice(device), "hipSetDevice");
    static_workspace_init(device);
}

kernel_manager_t::~kernel_manager_t() = default;

plan_t const* kernel_manager_t::find(einsummable_t const& merged) const
{
    auto it = plans_.find(merged.key());
    return it == plans_.end() ? nullptr : it->second.get();
}

std::optional<uint64_t> kernel_manager_t::build(einsummable_t const& e_)
{
    if (e_.join.has_variables()) {
        // the caller substitutes scalar variables before building
        // (src/engine/gpu/exec_graph.cc:106-108, kernel_executor.cc:64-66)
        return std::nullopt;
    }
    einsummable_t e = e_.merge_adjacent_dims();
    std::string   key = e.key();
    auto          it = plans_.find(key);
    if (it != plans_.end()) return it->second->workspace_bytes;

    std::shared_ptr<plan_t> p;
    auto                    planned = planned_.find(key);
    if (planned != planned_.end()) {
        p = std::move(planned->second);
        planned_.erase(planned);
        std::vector<plan_t*> waiting;
        p->deferred(waiting);
        finish_codegen_plans(waiting, device_);
    } else {
        p = make_plan(e);
    }
    if (!p) return std::nullopt;
    plans_.emplace(key, p);
    return p->workspace_bytes;
}

bool kernel_manager_t::buildable(einsummable_t const& e_)
{
    if (e_.join.has_variables()) return false;
    einsummable_t     e = e_.merge_adjacent_dims();
    std::string const key = e.key();
    if (plans_.count(key) || planned_.count(key)) return true;
    std::shared_ptr<plan_t> p = make_plan(e, true);
    if (!p) return false;
    planned_.emplace(key, std::move(p));
    return true;
}

std::shared_ptr<plan_t> kernel_manager_t::make_plan(einsummable_t const& e, bool defer) const
{
    // (complex tensors kept as f16 pairs: the generated elementwise kernels only)
    std::shared_ptr<plan_t> p = e.any_half_pairs() ? plan_codegen(e, device_, defer)
                                                   : plan_contraction(e, device_);
    if (!p && e.any_half_pairs()) return nullptr;
    if (!p) p = plan_complex_contraction(e, device_);
    if (!p) p = plan_transpose(e, device_);
    if (!p) p = plan_staged_elementwise(e, device_, defer);
    if (!p) p = plan_codegen(e, device_, defer);
    if (p) p->n_inns = int(e.inns.size());
    return p;
}

std::vector<std::optional<uint64_t>> kernel_manager_t::build_many(
    std::vector<einsummable_t> const& es)
{
    std::vector<std::string>                                 keys(es.size());
    std::vector<std::pair<std::string, std::shared_ptr<plan_t>>> fresh;
    std::unordered_map<std::string, size_t>                  seen;
    for (size_t i = 0; i != es.size(); ++i) {
        if (es[i].join.has_variables()) continue;  // build() answers nullopt
        einsummable_t merged = es[i].merge_adjacent_dims();
        keys[i] = merged.key();
        if (plans_.count(keys[i]) || seen.count(keys[i])) continue;
        seen.emplace(keys[i], fresh.size());
        auto planned = planned_.find(keys[i]);
        if (planned != planned_.end()) {
            fresh.emplace_back(keys[i], std::move(planned->second));
            planned_.erase(planned);
        } else {
            fresh.emplace_back(keys[i], make_plan(merged, true));
        }
    }
    std::vector<plan_t*> waiting;
    for (auto const& kp : fresh) {
        if (kp.second) kp.second->deferred(waiting);
    }
    finish_codegen_plans(waiting, device_);
    for (auto& kp : fresh) {
        if (kp.second) plans_.emplace(kp.first, std::move(kp.second));
    }
    std::vector<std::optional<uint64_t>> ret(es.size());
    for (size_t i = 0; i != es.size(); ++i) {
        if (keys[i].empty()) continue;
        auto it = plans_.find(keys[i]);
        if (it != plans_.end()) ret[i] = it->second->workspace_bytes;
    }
    return ret;
}

uint64_t kernel_manager_t::workspace_size(einsummable_t const& e) const
{
    plan_t const* p = find(e.merge_adjacent_dims());
    if (!p) throw km_error(km_status::not_built, "workspace_size: einsummable was not built");
    return p->workspace_bytes;
}

std::string kernel_manager_t::describe(einsummable_t const& e) const
{
    plan_t const* p = find(e.merge_adjacent_dims());
    if (!p) throw km_error(km_status::not_built, "describe: einsummable was not built");
    return p->description;
}

plan_t const* kernel_manager_t::find_raw(std::string const& raw_key) const
{
    auto it = raw_plans_.find(raw_key);
    return it == raw_plans_.end() ? nullptr : it->second.get();
}

void kernel_manager_t::alias_raw(std::string const& raw_key, einsummable_t const& e)
{
    auto it = plans_.find(e.merge_adjacent_dims().key());
    if (it != plans_.end()) raw_plans_[raw_key] = it->second;
}

void kernel_manager_t::run_plan(plan_t const& p, hipStream_t stream, void* out,
                                void const* const* inns, int n_inns, void* workspace,
                                uint64_t workspace_bytes) const
{
    if (n_inns != p.n_inns) {
        throw km_error(km_status::inputs, "execute: " + std::to_string(n_inns) +
                                              " inputs given, einsummable has " +
                                              std::to_string(p.n_inns));
    }
    if (p.workspace_bytes > 0 && (!workspace || workspace_bytes < p.workspace_bytes)) {
        throw km_error(km_status::workspace,
                       "execute: workspace of " + std::to_string(p.workspace_bytes) +
                           " bytes required, " + std::to_string(workspace ? workspace_bytes : 0) +
                           " given");
    }
    p.run(stream, out, inns, workspace, workspace_bytes);
}

void kernel_manager_t::operator()(einsummable_t const& e, hipStream_t stream, void* out,
                                  std::vector<void const*> const&             inns,
                                  std::optional<std::tuple<void*, uint64_t>> workspace) const
{
    plan_t const* p = find(e.merge_adjacent_dims());
    if (!p) throw km_error(km_status::not_built, "execute: einsummable was not built");
    void*    ws = workspace ? std::get<0>(workspace.value()) : nullptr;
    uint64_t wsz = workspace ? std::get<1>(workspace.value()) : 0;
    run_plan(*p, stream, out, inns.data(), int(inns.size()), ws, wsz);
}

void kernel_manager_t::operator()(touch_t const& touch_, hipStream_t stream, void* out,
                                  void const* inn) const
{
    touch_.validate();
    touch_t t = touch_.simplify();
    int     r = int(t.selection.size());
    if (r > 4) {
        throw km_error(km_status::invalid, "touch: more than four dimensions after simplify");
    }
    int const esz = int(dtype_size(t.dtype));
    int const vmax = 16 / esz;

    touchdim_t const& last = t.selection[r - 1];
    bool              wide = (last.size % vmax == 0) && (last.offset_inn % vmax == 0) &&
                (last.offset_out % vmax == 0) &&
                (reinterpret_cast<uintptr_t>(out) % 16 == 0) &&
                (reinterpret_cast<uintptr_t>(inn) % 16 == 0);
    if (r > 1) wide = wide && (last.d_inn % vmax == 0) && (last.d_out % vmax == 0);
    if (!wide && vmax > 1) {
        // A window that is not vector aligned, in an output whose rows are: the kernel of
        // the grouped path walks the output in 16-byte vectors and handles the window's
        // ragged edges and the unaligned input element by element.
        bool out_rows_wide = reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
                             (r == 1 || last.d_out % uint64_t(vmax) == 0);
        uint64_t volume = 1;
        for (auto const& d : t.selection) {
            out_rows_wide = out_rows_wide && d.d_out < (1ull << 32);
            volume *= d.size;
        }
        // (small windows are bound by the launch, and this path costs more on the host)
        if (out_rows_wide && volume >= (1ull << 21)) {
            touch_batch({t}, stream, out, {inn});
            return;
        }
    }

    touch_launch_t a;
    a.vec = wide ? vmax : 1;
    a.vec_per_row = last.size / uint64_t(a.vec);
    a.base_inn = 0;
    a.base_out = 0;
    // element strides of every dimension
    uint64_t si = 1, so = 1;
    uint64_t str_i[4], str_o[4];
    for (int d = r - 1; d >= 0; --d) {
        str_i[d] = si;
        str_o[d] = so;
        a.base_inn += t.selection[d].offset_inn * si;
        a.base_out += t.selection[d].offset_out * so;
        si *= t.selection[d].d_inn;
        so *= t.selection[d].d_out;
    }
    // outer dimensions right-aligned into the three slots
    a.n_vec = a.vec_per_row;
    bool small = a.vec_per_row < (1ull << 32);
    for (int s = 0; s != 3; ++s) {
        int d = (r - 1) - 3 + s;  // dimension feeding slot s
        if (d >= 0) {
            a.size[s] = t.selection[d].size;
            a.str_inn[s] = str_i[d];
            a.str_out[s] = str_o[d];
        } else {
            a.size[s] = 1;
            a.str_inn[s] = 0;
            a.str_out[s] = 0;
        }
        a.n_vec *= a.size[s];
        small = small && a.size[s] < (1ull << 32);
    }
    a.small = small && a.n_vec < (1ull << 32);
    a.outer = a.size[0] != 1 || a.size[1] != 1 ? 3 : (a.size[2] != 1 ? 1 : 0);

    int op = 0;
    if (t.castable) op = 1 + int(t.castable.value());
    launch_touch(a, esz, int(t.dtype), op, stream, out, inn);
    hip_check(hipGetLastError(), "touch launch");
}

void kernel_manager_t::touch_batch(std::vector<touch_t> const& touches_, hipStream_t stream,
                                   void* out, std::vector<void const*> const& inns) const
{
    if (touches_.empty()) return;
    if (touches_.size() != inns.size()) {
        throw km_error(km_status::inputs, "touch_batch: one input per touch expected");
    }
    size_t const n = touches_.size();
    size_t const rank0 = touches_[0].selection.size();
    dtype_t const dt = touches_[0].dtype;
    for (auto const& t : touches_) {
        t.validate();
        if (t.dtype != dt || t.selection.size() != rank0) {
            throw km_error(km_status::invalid, "touch_batch: touches differ in dtype or rank");
        }
        for (size_t d = 0; d != rank0; ++d) {
            if (t.selection[d].d_out != touches_[0].selection[d].d_out) {
                throw km_error(km_status::invalid,
                               "touch_batch: touches address differently shaped outputs");
            }
        }
    }
    // joint simplify: a dimension is folded into its predecessor only when every touch copies
    // it in full (touch.cc:3-28 applied to the whole group)
    std::vector<touch_t> ts(n);
    for (size_t i = 0; i != n; ++i) {
        ts[i].castable = touches_[i].castable;
        ts[i].dtype = dt;
    }
    for (size_t d = 0; d != rank0; ++d) {
        bool whole = d > 0;
        for (auto const& t : touches_) {
            touchdim_t const& x = t.selection[d];
            whole = whole && x.d_inn == x.d_out && x.offset_inn == 0 && x.offset_out == 0 &&
                    x.d_inn == x.size;
        }
        for (size_t i = 0; i != n; ++i) {
            touchdim_t const& x = touches_[i].selection[d];
            if (whole) {
                touchdim_t& b = ts[i].selection.back();
                b.d_inn *= x.d_inn;
                b.d_out *= x.d_inn;
                b.offset_inn *= x.d_inn;
                b.offset_out *= x.d_inn;
                b.size *= x.d_inn;
            } else {
                ts[i].selection.push_back(x);
            }
        }
    }
    int const r = int(ts[0].selection.size());
    if (r > 4) throw km_error(km_status::invalid, "touch_batch: more than four dimensions");
    int const esz = int(dtype_size(dt));
    int const vmax = 16 / esz;

    // the output is walked in 16-byte vectors whenever its rows allow it
    bool out_wide = reinterpret_cast<uintptr_t>(out) % 16 == 0;
    for (size_t i = 0; i != n; ++i) {
        touchdim_t const& last = ts[i].selection[r - 1];
        out_wide = out_wide && last.d_out % vmax == 0;
        for (auto const& d : ts[i].selection) {
            if (d.d_out >= (1ull << 32)) {
                throw km_error(km_status::invalid, "touch_batch: extent beyond 2^32");
            }
        }
    }
    bool const wide = out_wide;
    uint64_t out_str[4];
    {
        uint64_t s = 1;
        for (int d = r - 1; d >= 0; --d) {
            out_str[d] = s;
            s *= ts[0].selection[d].d_out;
        }
    }
    // every touch as a four-dimensional window of the output
    std::vector<touch_item_t> items(n);
    for (size_t i = 0; i != n; ++i) {
        touch_t const& t = ts[i];
        touch_item_t&  it = items[i];
        it.inn = inns[i];
        it.op = t.castable ? 1 + int(t.castable.value()) : 0;
        it.base_inn = 0;
        uint64_t si = 1;
        uint64_t str_i[4] = {0, 0, 0, 0};
        for (int d = r - 1; d >= 0; --d) {
            str_i[d] = si;
            it.base_inn += t.selection[d].offset_inn * si;
            si *= t.selection[d].d_inn;
        }
        for (int s = 0; s != 4; ++s) {
            int d = r - 4 + s;  // dimension feeding slot s
            if (d >= 0) {
                it.lo[s] = uint32_t(t.selection[d].offset_out);
                it.size[s] = uint32_t(t.selection[d].size);
                if (s < 3) it.str_inn[s] = str_i[d];
            } else {
                it.lo[s] = 0;
                it.size[s] = 1;
                if (s < 3) it.str_inn[s] = 0;
            }
        }
        // input vectors line up with output vectors when the window's origin has the same
        // phase in both tensors and every input row starts on a vector boundary; with
        // another phase (shift, in elements) the owner kernel still reads whole input vectors
        bool rows = wide && reinterpret_cast<uintptr_t>(inns[i]) % 16 == 0;
        for (int s = 0; s != 3; ++s) {
            rows = rows && (it.size[s] == 1 || it.str_inn[s] % uint64_t(vmax) == 0);
        }
        uint64_t const shift = (it.base_inn + uint64_t(vmax) - it.lo[3] % uint32_t(vmax)) %
                               uint64_t(vmax);
        it.vec_inn = rows && shift == 0 ? 1 : 0;
        it.vec_rows = rows ? 1 : 0;
        it.shift = int(shift);
    }
    uint64_t out_str4[3];
    for (int s = 0; s != 3; ++s) {
        int d = r - 4 + s;
        out_str4[s] = d >= 0 ? out_str[d] : 0;
    }
    auto overlap = [](touch_item_t const& x, touch_item_t const& y) {
        for (int s = 0; s != 4; ++s) {
            if (x.lo[s] + uint64_t(x.size[s]) <= y.lo[s] || y.lo[s] + uint64_t(y.size[s]) <= x.lo[s]) {
                return false;
            }
        }
        return true;
    };

    // Two ways to keep the sequential result.  Usually the owner of each output vector folds
    // the touches that cover it, in list order: one launch over the windows' bounding box, the
    // output read and written once however many windows overlap.  When the windows are
    // islands in a much larger box (the walk over the empty part would cost more than the
    // touches), they are sorted into levels instead (a touch goes one level above the last
    // earlier touch it overlaps); a level's windows are disjoint and run as one launch, each
    // streaming through its own window.
    int const    R = std::max(1, r);  // stored dimensions per item
    size_t const cap = size_t(touch_list_capacity(R));
    bool         strides_fit = true;
    for (size_t i = 0; i != n; ++i) {
        for (int s = 0; s != 3; ++s) strides_fit = strides_fit && items[i].str_inn[s] < (1ull << 32);
    }
    constexpr size_t SPAN = 2048;  // the level search is quadratic: bounded spans of the list
    for (size_t span0 = 0; span0 < n; span0 += SPAN) {
        size_t const span_n = std::min(SPAN, n - span0);
        uint64_t     blo[4], bhi[4];
        for (int s = 0; s != 4; ++s) {
            blo[s] = ~0ull;
            bhi[s] = 0;
        }
        double span_volume = 0;
        for (size_t i = span0; i != span0 + span_n; ++i) {
            double vol = 1;
            for (int s = 0; s != 4; ++s) {
                blo[s] = std::min<uint64_t>(blo[s], items[i].lo[s]);
                bhi[s] = std::max<uint64_t>(bhi[s], items[i].lo[s] + uint64_t(items[i].size[s]));
                vol *= double(items[i].size[s]);
            }
            span_volume += vol;
        }
        double box_volume = 1;
        for (int s = 0; s != 4; ++s) box_volume *= double(bhi[s] - blo[s]);
        bool by_owner = strides_fit && box_volume <= 8.0 * span_volume;
        if (const char* env = std::getenv("ES_KM_TOUCH_BATCH")) {  // tuning and tests
            if (env[0] == 'o') by_owner = strides_fit;  // owner computes
            if (env[0] == 'l') by_owner = false;        // levels
        }

        if (!by_owner) {
            std::vector<int> level(span_n, 0);
            int              top = 0;
            for (size_t i = 0; i != span_n; ++i) {
                for (size_t j = 0; j != i; ++j) {
                    if (level[j] >= level[i] && overlap(items[span0 + i], items[span0 + j])) {
                        level[i] = level[j] + 1;
                    }
                }
                top = std::max(top, level[i]);
            }
            for (int l = 0; l <= top; ++l) {
                touch_level_t b;
                b.vec = wide ? vmax : 1;
                for (int s = 0; s != 3; ++s) b.out_str[s] = out_str4[s];
                b.n = 0;
                b.max_vec = 0;
                bool castable = false;
                auto flush = [&]() {
                    if (b.n == 0) return;
                    launch_touch_level(b, esz, int(dt), castable, stream, out);
                    hip_check(hipGetLastError(), "touch_batch launch");
                    b.n = 0;
                    b.max_vec = 0;
                    castable = false;
                };
                for (size_t i = 0; i != span_n; ++i) {
                    if (level[i] != l) continue;
                    touch_item_t const& it = items[span0 + i];
                    uint64_t const v = uint64_t(b.vec);
                    uint64_t const vpr = (it.lo[3] + uint64_t(it.size[3]) - 1) / v - it.lo[3] / v + 1;
                    uint64_t const nv = uint64_t(it.size[0]) * it.size[1] * it.size[2] * vpr;
                    if (nv >= (1ull << 39)) {
                        throw km_error(km_status::invalid, "touch_batch: window too large");
                    }
                    b.items[b.n++] = it;
                    b.max_vec = std::max(b.max_vec, nv);
                    castable = castable || it.op != 0;
                    if (b.n == TOUCH_BATCH_MAX) flush();
                }
                flush();
            }
            continue;
        }

        // as many items per launch as the kernel arguments hold; consecutive launches keep
        // the list order
        for (size_t first = span0; first < span0 + span_n; first += cap) {
            size_t const cnt = std::min(cap, span0 + span_n - first);
            touch_list_t b;
            b.n = uint32_t(cnt);
            b.rank = uint32_t(R);
            b.vec = uint32_t(wide ? vmax : 1);
            bool     castable = false;
            uint64_t lo[4], hi[4];
            for (int s = 0; s != 4; ++s) {
                lo[s] = ~0ull;
                hi[s] = 0;
            }
            uint32_t const W = uint32_t(touch_list_item_words(R));
            int const      ND = R > 2 ? 4 : 2;
            double         covered = 0;  // elements, counted once per window
            uint32_t const first_op = uint32_t(items[first].op);
            bool           all_vectors = true;  // ... and all with the first item's op
            for (size_t i = 0; i != cnt; ++i) {
                touch_item_t const& it = items[first + i];
                all_vectors = all_vectors && it.vec_rows && uint32_t(it.op) == first_op;
                covered += double(it.size[0]) * it.size[1] * it.size[2] * it.size[3];
                uint32_t* const     w = b.w + i * W;
                std::memset(w, 0, W * sizeof(uint32_t));
                uint64_t const p = reinterpret_cast<uint64_t>(it.inn);
                w[0] = uint32_t(p);
                w[1] = uint32_t(p >> 32);
                w[2] = uint32_t(it.base_inn);
                w[3] = uint32_t(it.base_inn >> 32);
                for (int d = 0; d != ND; ++d) {
                    int const s = 4 - ND + d;
                    w[4 + d] = it.lo[s];
                    w[4 + ND + d] = it.size[s];
                    if (d + 1 != ND) w[4 + 2 * ND + d] = uint32_t(it.str_inn[s]);
                }
                w[4 + 3 * ND - 1] =
                    uint32_t(it.op) | (uint32_t(it.vec_rows) << 8) | (uint32_t(it.shift) << 16);
                castable = castable || it.op != 0;
                for (int s = 0; s != 4; ++s) {
                    lo[s] = std::min<uint64_t>(lo[s], it.lo[s]);
                    hi[s] = std::max<uint64_t>(hi[s], it.lo[s] + uint64_t(it.size[s]));
                }
            }
            lo[3] = lo[3] / uint64_t(b.vec) * uint64_t(b.vec);
            hi[3] = (hi[3] + uint64_t(b.vec) - 1) / uint64_t(b.vec) * uint64_t(b.vec);
            uint64_t rows = 1;
            for (int s = 0; s != 4; ++s) {
                b.box_lo[s] = uint32_t(lo[s]);
                b.box_size[s] = uint32_t(hi[s] - lo[s]);
                if (s < 3) {
                    b.out_str[s] = out_str4[s];
                    rows *= hi[s] - lo[s];
                }
            }
            b.eager = covered >= 0.5 * double(rows) * double(hi[3] - lo[3]);
            b.uniform_op = all_vectors ? 1 + first_op : 0;
            uint64_t const vpr = (hi[3] - lo[3]) / uint64_t(b.vec);
            b.chunks_per_row = uint32_t((vpr + TOUCH_LIST_BLOCK_HOST - 1) / TOUCH_LIST_BLOCK_HOST);
            if (rows * b.chunks_per_row >= (1ull << 31)) {
                throw km_error(km_status::invalid, "touch_batch: bounding box too large");
            }
            launch_touch_list(b, esz, int(dt), castable, stream, out);
            hip_check(hipGetLastError(), "touch_batch launch");
        }
    }
}

void kernel_manager_t::constant_fill(dtype_t dtype, uint64_t value_bits, uint64_t nelem,
                                     hipStream_t stream, void* out) const
{
    launch_fill_constant(int(dtype_size(dtype)), value_bits, nelem, stream, out);
    hip_check(hipGetLastError(), "constant_fill launch");
}

void kernel_manager_t::lowerTri_fill(dtype_t dtype, uint64_t lower_bits, uint64_t upper_bits,
                                     uint64_t nrow, uint64_t ncol, int64_t start,
                                     hipStream_t stream, void* out) const
{
    launch_fill_lowertri(int(dtype_size(dtype)), lower_bits, upper_bits, nrow, ncol, start, stream,
                         out);
    hip_check(hipGetLastError(), "lowerTri_fill launch");
}

}  // namespace es
