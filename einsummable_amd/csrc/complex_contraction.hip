// c64 contractions on the matrix cores, as an fp32 contraction of twice the depth.
//
// With every complex number kept as the (re, im) pair of floats it is stored as,
//   C[m, n] = sum_k A[m, k] * B[n, k]
// is the real product
//   C'[m, (n, d)] = sum_(k, c) A'[m, (k, c)] * B'[(n, d), (k, c)]
// where A' is A read as floats (c = 0: re, c = 1: im), C' is C read as floats (d likewise) and
//   B'[(n, 0), (k, .)] = ( re B, -im B )        B'[(n, 1), (k, .)] = ( im B,  re B ).
// That is 8 M N K real flops, exactly the work of the complex product, through
// v_mfma_f32_32x32x2_f32.  The reference hands c64 matmuls to cublasCgemm and other complex
// contractions to cuTENSOR (src/engine/gpu/gpu_kernel_manager.cc:1543-1558, 1319-1452).
//
// The operand that owns the output's innermost mode plays B: it is expanded into the
// workspace by one pass (16 bytes written per complex element), laid out so that whatever is
// contiguous in it stays contiguous (along k: rows (n, d) of (k, c); along n: rows (k, c) of
// (n, d)).  The other operand is read in place when a summed mode is its innermost one --
// then (k, c) is contiguous in memory as it stands -- and otherwise split into a plane of real
// and a plane of imaginary parts, rows (k, c) of m.  The fp32 contraction planner then sees an
// ordinary einsummable with two more modes and picks tile, load path and split as for any
// other.
#include "kernel_manager.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <string>

namespace es
{
namespace
{

constexpr int MAXD = 8;

enum class prep_t : uint32_t {
    rows_of_k = 0,  // B' rows (n, d) of (k, c)
    rows_of_n = 1,  // B' rows (k, c) of (n, d)
    planes = 2      // A' rows (k, c) of m
};

struct prep_args_t {
    void const* in;
    float*      out;
    uint64_t    n;       // complex elements
    uint64_t    inner;   // extent of the innermost group of the canonical order
    uint32_t    nd;
    uint32_t    kind;
    uint32_t    size[MAXD];    // canonical order, innermost first
    int64_t     stride[MAXD];  // in complex elements of the source
};

template <bool WIDE>
__global__ __launch_bounds__(256) void complex_prepare_kernel(prep_args_t a)
{
    uint64_t const t = uint64_t(blockIdx.x) * 256 + threadIdx.x;
    if (t >= a.n) return;
    uint64_t rem = t;
    int64_t  src = 0;
#pragma unroll
    for (int d = 0; d != MAXD; ++d) {
        if (d < int(a.nd)) {
            uint64_t const q = rem / a.size[d];
            src += int64_t(rem - q * a.size[d]) * a.stride[d];
            rem = q;
        }
    }
    float re, im;
    if constexpr (WIDE) {
        float2 const v = static_cast<float2 const*>(a.in)[src];
        re = v.x;
        im = v.y;
    } else {
        float const* p = static_cast<float const*>(a.in) + 2 * src;
        re = p[0];
        im = p[1];
    }
    uint64_t const row = t / a.inner, col = t - row * a.inner;
    if (a.kind == uint32_t(prep_t::planes)) {
        float* o = a.out + row * 2 * a.inner + col;
        o[0] = re;
        o[a.inner] = im;
        return;
    }
    // the workspace is 16-byte aligned and every pair starts on an even float
    float2* o = reinterpret_cast<float2*>(a.out + row * 4 * a.inner + 2 * col);
    if (a.kind == uint32_t(prep_t::rows_of_k)) {
        o[0] = float2{re, -im};
        o[a.inner] = float2{im, re};
    } else {
        o[0] = float2{re, im};
        o[a.inner] = float2{-im, re};
    }
}

struct complex_contraction_plan_t : plan_t {
    struct stage_t {
        int         input;
        prep_args_t args;
        uint64_t    offset;
    };
    std::vector<stage_t>    stages;
    std::shared_ptr<plan_t> inner;
    uint64_t                inner_offset = 0;

    void run(hipStream_t stream, void* out, void const* const* inns, void* workspace,
             uint64_t) const override
    {
        void const* ptrs[2] = {inns[0], inns[1]};
        char* const ws = static_cast<char*>(workspace);
        if (reinterpret_cast<uintptr_t>(ws) % 16 != 0) {
            throw km_error(km_status::workspace, "complex contraction: workspace not 16-byte aligned");
        }
        for (stage_t const& s : stages) {
            prep_args_t a = s.args;
            a.in = inns[s.input];
            a.out = reinterpret_cast<float*>(ws + s.offset);
            dim3 const grid(unsigned((a.n + 255) / 256)), block(256);
            if (reinterpret_cast<uintptr_t>(a.in) % 8 == 0) {
                hipLaunchKernelGGL(complex_prepare_kernel<true>, grid, block, 0, stream, a);
            } else {
                hipLaunchKernelGGL(complex_prepare_kernel<false>, grid, block, 0, stream, a);
            }
            ptrs[s.input] = a.out;
        }
        hipError_t err = hipGetLastError();
        if (err != hipSuccess) {
            throw km_error(km_status::device,
                           std::string("complex contraction launch: ") + hipGetErrorString(err));
        }
        inner->run(stream, out, ptrs, inner->workspace_bytes ? ws + inner_offset : nullptr,
                   inner->workspace_bytes);
    }
};

}  // namespace

std::shared_ptr<plan_t> plan_complex_contraction(einsummable_t const& e, int device)
{
    if (!e.is_contraction() || e.out_dtype() != dtype_t::c64) return nullptr;
    if (e.inn_dtype(0) != dtype_t::c64 || e.inn_dtype(1) != dtype_t::c64) return nullptr;
    int const R = int(e.join_shape.size()), O = e.out_rank;
    auto has = [&](int k, int m) {
        return std::find(e.inns[size_t(k)].begin(), e.inns[size_t(k)].end(), m) != e.inns[size_t(k)].end();
    };
    // b: both and out, j: both and summed, 0 / 1: that operand and out
    enum { batch, summed, own0, own1 };
    std::vector<int> kind(size_t(R), batch);
    for (int m = 0; m != R; ++m) {
        bool const l = has(0, m), r = has(1, m), o = m < O;
        if (l && r && o) {
            kind[size_t(m)] = batch;
        } else if (l && r && !o) {
            kind[size_t(m)] = summed;
        } else if (l && !r && o) {
            kind[size_t(m)] = own0;
        } else if (!l && r && o) {
            kind[size_t(m)] = own1;
        } else {
            return nullptr;
        }
    }
    int const last = kind[size_t(O - 1)];
    if (last != own0 && last != own1) return nullptr;  // a batch mode innermost in the output
    int const y = last == own0 ? 0 : 1, x = 1 - y;
    int const own_y = last, own_x = last == own0 ? own1 : own0;
    int const x_inner = kind[size_t(e.inns[size_t(x)].back())];
    int const y_inner = kind[size_t(e.inns[size_t(y)].back())];
    if (x_inner == batch || y_inner == batch) return nullptr;
    if (int(e.inns[0].size()) > MAXD || int(e.inns[1].size()) > MAXD) return nullptr;
    if (e.inn_nelem(0) >= (1ull << 38) || e.inn_nelem(1) >= (1ull << 38)) return nullptr;

    // modes of the fp32 einsummable: d follows the output modes, c follows everything
    auto ren = [&](int m) { return m < O ? m : m + 1; };
    int const d = O, c = R + 1;
    std::vector<uint64_t> shape;
    for (int m = 0; m != O; ++m) shape.push_back(e.join_shape[size_t(m)]);
    shape.push_back(2);
    for (int m = O; m != R; ++m) shape.push_back(e.join_shape[size_t(m)]);
    shape.push_back(2);

    auto modes_of = [&](int want, std::vector<int> const& order) {
        std::vector<int> r;
        for (int m : order) {
            if (kind[size_t(m)] == want) r.push_back(m);
        }
        return r;
    };
    std::vector<int> out_order(size_t(O), 0);
    for (int m = 0; m != O; ++m) out_order[size_t(m)] = m;
    std::vector<int> const bs = modes_of(batch, out_order);
    std::vector<int> const ks = modes_of(summed, e.inns[size_t(x)]);  // as the in-place operand has them
    std::vector<int> const ns = modes_of(own_y, out_order);
    std::vector<int> const ms = modes_of(own_x, out_order);

    auto p = std::make_shared<complex_contraction_plan_t>();
    uint64_t offset = 0;
    auto stride_in = [&](int k, int m) {
        int64_t s = 1;
        auto const& inn = e.inns[size_t(k)];
        for (int i = int(inn.size()) - 1; i >= 0; --i) {
            if (inn[size_t(i)] == m) return s;
            s *= int64_t(e.join_shape[size_t(inn[size_t(i)])]);
        }
        return int64_t(0);
    };
    // `groups`: outermost first; the last one is the innermost group of the canonical order
    auto stage = [&](int input, prep_t what, std::vector<std::vector<int>> const& groups,
                     uint64_t floats_per_element) {
        complex_contraction_plan_t::stage_t s;
        s.input = input;
        s.offset = offset;
        prep_args_t& a = s.args;
        a.in = nullptr;
        a.out = nullptr;
        a.n = e.inn_nelem(input);
        a.kind = uint32_t(what);
        a.nd = 0;
        a.inner = 1;
        for (int m : groups.back()) a.inner *= e.join_shape[size_t(m)];
        for (int i = 0; i != MAXD; ++i) {
            a.size[i] = 1;
            a.stride[i] = 0;
        }
        for (auto g = groups.rbegin(); g != groups.rend(); ++g) {
            for (auto m = g->rbegin(); m != g->rend(); ++m) {
                a.size[a.nd] = uint32_t(e.join_shape[size_t(*m)]);
                a.stride[a.nd] = stride_in(input, *m);
                ++a.nd;
            }
        }
        p->stages.push_back(s);
        offset += (a.n * floats_per_element * 4 + 255) / 256 * 256;
    };
    for (uint64_t s : e.join_shape) {
        if (s >= (1ull << 31)) return nullptr;
    }

    std::vector<std::vector<int>> inns32(2);
    auto append = [&](std::vector<int>& to, std::vector<int> const& from) {
        for (int m : from) to.push_back(ren(m));
    };
    std::string how;
    // the operand that stays on the left of the product
    if (x_inner == summed) {
        append(inns32[size_t(x)], e.inns[size_t(x)]);
        inns32[size_t(x)].push_back(c);
        how = "in place";
    } else {
        if (ms.empty()) return nullptr;
        append(inns32[size_t(x)], bs);
        append(inns32[size_t(x)], ks);
        inns32[size_t(x)].push_back(c);
        append(inns32[size_t(x)], ms);
        stage(x, prep_t::planes, {bs, ks, ms}, 2);
        how = "planes";
    }
    // the operand that is expanded
    if (ns.empty()) return nullptr;
    if (y_inner == summed) {
        append(inns32[size_t(y)], bs);
        append(inns32[size_t(y)], ns);
        inns32[size_t(y)].push_back(d);
        append(inns32[size_t(y)], ks);
        inns32[size_t(y)].push_back(c);
        stage(y, prep_t::rows_of_k, {bs, ns, ks}, 4);
        how += ", expanded along k";
    } else {
        append(inns32[size_t(y)], bs);
        append(inns32[size_t(y)], ks);
        inns32[size_t(y)].push_back(c);
        append(inns32[size_t(y)], ns);
        inns32[size_t(y)].push_back(d);
        stage(y, prep_t::rows_of_n, {bs, ks, ns}, 4);
        how += ", expanded along n";
    }

    // summed modes are numbered in the order the operands first name them
    {
        std::vector<int> order;
        for (auto const& inn : inns32) {
            for (int m : inn) {
                if (m > O && std::find(order.begin(), order.end(), m) == order.end()) order.push_back(m);
            }
        }
        std::vector<uint64_t> renumbered(shape.begin(), shape.begin() + O + 1);
        for (int m : order) renumbered.push_back(shape[size_t(m)]);
        for (auto& inn : inns32) {
            for (int& m : inn) {
                if (m > O) m = O + 1 + int(std::find(order.begin(), order.end(), m) - order.begin());
            }
        }
        shape = renumbered;
    }
    einsummable_t e32;
    try {
        e32 = einsummable_t::make(shape, inns32, O + 1,
                                  scalarop_t::parse("*[hole|f32@0,hole|f32@1]"), castable_t::add)
                  .merge_adjacent_dims();
    } catch (ir_error const&) {
        return nullptr;
    }
    p->inner = plan_contraction(e32, device);
    if (!p->inner) return nullptr;
    p->inner->n_inns = 2;
    p->inner_offset = offset;
    p->workspace_bytes = offset + p->inner->workspace_bytes;
    p->description = "contraction_c64_as_f32 [operand " + std::to_string(x) + " " + how +
                     " (operand " + std::to_string(y) + ")] then " + p->inner->description;
    return p;
}

}  // namespace es
