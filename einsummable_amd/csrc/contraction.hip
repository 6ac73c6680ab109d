// Contraction planner and MFMA GEMM kernels for gfx950.
//
// Any two-input einsummable with join x0*x1 and castable add whose modes split into
//   b (lhs, rhs and out), i (lhs and out), j (lhs and rhs, summed), k (rhs and out)
// (the classification of src/engine/cpu/contraction.cc:186-221) is run as ONE batched GEMM
//   C[b, m, n] = sum_k A[b, m, k] * B[b, n, k]
// where m, n, k and b are *groups* of modes: the kernel decomposes a group index into its
// mode digits and applies per-tensor strides, so transposed, batched and non-contiguous-mode
// contractions (e.g. acbe,adbe->abcd, adbe,cde->abc) read their operands in place.  The
// reference reaches the same results with cuBLAS for four matmul spellings and cuTENSOR for
// the rest (src/engine/gpu/gpu_kernel_manager.cc:1265-1452), or on the CPU by permuting
// operands into a workspace before a batched GEMM (contraction.cc:103-177); here no operand
// is ever copied and no workspace is needed.
//
// Kernel: 256 threads = 4 wavefronts in a 2x2 grid, macro tile BM x BN, K staged through LDS
// in slices of 128 bytes per row (64 f16 / 32 f32 / 16 f64), double buffered, with the next
// slice's global loads in flight while the matrix cores consume the current one.  LDS rows are
// padded to 144 bytes, which makes the 16-byte-per-lane fragment reads conflict free.  The
// MFMA is issued with the B fragment as the row operand so that every lane ends up holding
// four consecutive n of one m: the epilogue stores them with one 8 / 16-byte write.
// fp16 inputs accumulate in fp32 (v_mfma_f32_32x32x16_f16; the persistent kernels use
// v_mfma_f32_16x16x32_f16), fp32 uses v_mfma_f32_32x32x2_f32, f64 uses v_mfma_f64_16x16x4_f64.
#include "gemm_dma_kernel.h"
#include "gemm_pc_kernel.h"
#include "gemm_kernel.h"
#include "kernel_manager.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace es
{
namespace
{

using namespace gemm;

// ----------------------------------------------------------------------------- planner

struct mode_info_t {
    int      mode;
    uint64_t size;
    int64_t  s_lhs, s_rhs, s_out;  // element strides, 0 when absent
};

void fill_group(group_t& g, std::vector<mode_info_t> const& ms,
                int64_t mode_info_t::*x, int64_t mode_info_t::*y, int64_t mode_info_t::*z)
{
    g.n = uint32_t(std::max<size_t>(ms.size(), 1));
    for (int d = 0; d != MAXG; ++d) {
        g.size[d] = 1;
        g.sx[d] = g.sy[d] = g.sz[d] = 0;
    }
    for (size_t d = 0; d != ms.size(); ++d) {
        g.size[d] = uint32_t(ms[d].size);
        g.sx[d] = x ? ms[d].*x : 0;
        g.sy[d] = y ? ms[d].*y : 0;
        g.sz[d] = z ? ms[d].*z : 0;
    }
}

// Macro tile for a problem.  Larger tiles cost less LDS and L1 traffic per flop, which is what
// limits the fp16 kernels (measured full-chip rates on MI355X with the direct-to-LDS kernel:
// 256x256 ~1.2 PFLOP/s, 128x256 ~0.98, 128x128 ~0.8), but there are fewer of them to spread
// over the 256 compute units.  fp32 is bound by the matrix cores at every tile size, so only
// the spread matters.  Estimate: tiles per compute unit, rounded up, times the time of a tile.
// ES_KM_GEMM_TILE=128x128|128x256|256x128|256x256 overrides the choice (tuning aid).
struct tile_option_t {
    int    bm, bn;
    double eff16, eff32;  // relative rate of a compute unit running this tile
};

void choose_tile(dtype_t dt, uint64_t M, uint64_t N, uint64_t K, uint64_t batch, bool dma_ok,
                 bool big_ok, int& bm, int& bn)
{
    bm = 128;
    bn = 128;
    if (dt == dtype_t::f64) return;
    if (const char* env = std::getenv("ES_KM_GEMM_TILE")) {
        int x = 0, y = 0;
        if (std::sscanf(env, "%dx%d", &x, &y) == 2 && (x == 128 || x == 256) &&
            (y == 128 || y == 256)) {
            // rectangular tiles exist in the direct-to-LDS kernel only
            if (x == y || dma_ok) {
                bm = x;
                bn = y;
            }
            return;
        }
    }
    // short reductions are bound by the output write: small tiles, several per compute unit
    if (K < 512) return;
    if (!dma_ok) {
        // register-staged 256x256 kernel: only pays with several full rounds of tiles
        uint64_t big_tiles = ((M + 255) / 256) * ((N + 255) / 256) * batch;
        if (K >= 1024 && M >= 512 && N >= 512 && big_tiles >= 768) bm = bn = 256;
        return;
    }
    // Streaming shapes (one operand read once, little reuse: attention's P.V, a vector or a
    // few rows against a weight matrix) are bound by HBM: the small tile's extra workgroups
    // per compute unit keep more loads in flight
    double const elem = double(dtype_size(dt));
    double const intensity = 2.0 * double(M) * double(N) * double(K) /
                             ((double(M) * K + double(N) * K + double(M) * N) * elem);
    if (dt == dtype_t::f16 && intensity < 150.0) {
        // ... unless the streamed operand has rows for 256 of them and that still leaves a
        // tile for every compute unit: twice the bytes of it under way per workgroup, with
        // three stages (P.V of 32 and of 128 heads of 2048 x 2048: 7 % faster)
        if (N <= 128 && M >= 256 && ((M + 255) / 256) * batch >= 256) bm = 256;
        return;
    }
    static tile_option_t const options[] = {{256, 256, 1.00, 1.00},
                                            {128, 256, 0.88, 1.00},
                                            {256, 128, 0.88, 1.00},
                                            {128, 128, 0.68, 1.00}};
    double best = 0;
    uint64_t const nk = K * dtype_size(dt) / 64;
    for (tile_option_t const& o : options) {
        if (o.bm == 256 && o.bn == 256 && !big_ok) continue;
        uint64_t tiles = ((M + o.bm - 1) / o.bm) * ((N + o.bn - 1) / o.bn) * batch;
        // at most 128 tiles and a long reduction: plan_contraction will cut k into splits
        // (same rule as there), which costs a pass over the fp32 partial tiles.  In units of
        // tile area per matrix-core time: bytes moved at ~4 TB/s against 2 K flop per unit
        // of area at the compute unit's share of ~1.2 PFLOP/s (f16) or ~0.14 PFLOP/s (f32)
        uint64_t const S = (tiles <= 128 && nk >= 16) ? std::min<uint64_t>({256 / tiles, nk / 8, 64}) : 1;
        double fold = 0;
        if (S > 1) {
            double const ratio = dt == dtype_t::f16 ? 1.5 : 0.14;
            fold = (4.0 * double(S) + elem) * double(M) * double(N) * double(batch) * ratio /
                   (2.0 * double(K));
        }
        uint64_t rounds = (tiles * S + 255) / 256;
        double   t = double(rounds) * double(o.bm) * double(o.bn) / double(S) /
                       (dt == dtype_t::f16 ? o.eff16 : o.eff32) +
                   fold;
        if (best == 0 || t < best * 0.97) {  // near ties go to the larger tile (listed first)
            best = t;
            bm = o.bm;
            bn = o.bn;
        }
    }
}

// Adjacent modes of a group that are also adjacent (same order, dense) in every tensor that
// holds them were already fused by merge_adjacent_dims; what is left is genuinely strided.
struct contraction_plan_t : plan_t {
    gemm_args_t args;
    dtype_t     dtype;
    bool        swapped;
    bool        planned_dma = false;
    int         bm, bn;

    void run(hipStream_t stream, void* out, void const* const* inns, void* workspace,
             uint64_t) const override
    {
        gemm_args_t a = args;
        a.ws = static_cast<float*>(workspace);
        a.A = swapped ? inns[1] : inns[0];
        a.B = swapped ? inns[0] : inns[1];
        a.C = out;
        // vector paths need 16-byte aligned operands
        auto mis = [](void const* p) { return reinterpret_cast<uintptr_t>(p) % 16 != 0; };
        bool const misaligned = mis(a.A) || mis(a.B) || mis(a.C);
        if (mis(a.A) && a.a_mode != 2) a.a_mode = 2;
        if (mis(a.B) && a.b_mode != 2) a.b_mode = 2;
        if (mis(a.C) && a.c_mode != 2) a.c_mode = 2;
        // the wide epilogue lives in the direct-to-LDS kernel and in the register-staged
        // one (A along k, B along k or n)
        bool const dma = (dtype == dtype_t::f16 && gemm_dma_eligible<_Float16>(a)) ||
                         (dtype == dtype_t::f32 && gemm_dma_eligible<float>(a)) ||
                         (dtype == dtype_t::f64 && gemm_dma_wide_eligible<double>(a, 4));
        if (a.c_mode == 3 && !dma && !(a.a_mode == 0 && a.b_mode != 2)) a.c_mode = 0;
        // what build() described is what runs, unless a buffer's alignment forbids it
        if (!dma) a.splits = 1;  // only the direct-to-LDS kernel splits k
        if (planned_dma && !dma && !misaligned) {
            throw km_error(km_status::device,
                           "contraction: the planned direct-to-LDS kernel cannot be launched");
        }
        launch(a, stream);
        hipError_t err = hipGetLastError();
        if (err != hipSuccess) {
            throw km_error(km_status::device,
                           std::string("contraction launch: ") + hipGetErrorString(err));
        }
    }

    // Products of this shape on other buffers ride along as batch entries of one launch of
    // the persistent 128 x 256 kernel when one of them has at most a tile per compute unit (a
    // LLaMA projection of 2048 tokens): set-up, first loads and the last epilogue are then
    // paid once instead of once per product.  What that buys is small -- the q, k and v
    // projections 176 us as one launch against 188 as three: under the board's power limit
    // the time saved is partly given back as clock -- and with several rounds of tiles per
    // product it buys nothing (w1 and w3: 362 against 358 us), so those stay as they are.
    int max_group() const override
    {
        const char* env = std::getenv("ES_KM_GEMM_GROUPS");  // tuning and tests
        bool const  off = env && env[0] == '0';
        bool const fits = dtype == dtype_t::f16 && args.persistent == 2 && args.batch == 1 &&
                          args.splits <= 1 && workspace_bytes == 0 &&
                          uint64_t(args.tiles_m) * args.tiles_n <= args.workgroups;
        return fits && !off ? 8 : 1;
    }

    void run_group(hipStream_t stream, int runs, void* const* outs,
                   void const* const* inns) const override
    {
        if (runs < 1 || runs > max_group()) {
            throw km_error(km_status::invalid, "contraction: too many runs for one launch");
        }
        gemm_args_t a = args;
        a.ws = nullptr;
        a.A = swapped ? inns[1] : inns[0];
        a.B = swapped ? inns[0] : inns[1];
        a.C = outs[0];
        auto mis = [](void const* p) { return reinterpret_cast<uintptr_t>(p) % 16 != 0; };
        bool aligned = true;
        for (int g = 0; g != runs; ++g) {
            void const* const x = swapped ? inns[2 * g + 1] : inns[2 * g];
            void const* const y = swapped ? inns[2 * g] : inns[2 * g + 1];
            aligned = aligned && !mis(x) && !mis(y) && !mis(outs[g]);
            a.group_off[0][g] = (static_cast<char const*>(x) - static_cast<char const*>(a.A)) / 2;
            a.group_off[1][g] = (static_cast<char const*>(y) - static_cast<char const*>(a.B)) / 2;
            a.group_off[2][g] = (static_cast<char const*>(outs[g]) - static_cast<char const*>(a.C)) / 2;
        }
        if (runs == 1 || !aligned || !gemm::pc::gemm_pc_eligible(a)) {
            // what one launch cannot take runs one by one
            for (int g = 0; g != runs; ++g) run(stream, outs[g], inns + 2 * g, nullptr, 0);
            return;
        }
        a.grouped = 1;
        a.batch = uint32_t(runs);
        a.gb.n = 1;
        a.gb.size[0] = uint32_t(runs);
        a.gb.sx[0] = a.gb.sy[0] = a.gb.sz[0] = 0;
        a.xcd_total = uint32_t(uint64_t(a.tiles_m) * a.tiles_n * uint64_t(runs));
        launch(a, stream);
        hipError_t err = hipGetLastError();
        if (err != hipSuccess) {
            throw km_error(km_status::device,
                           std::string("contraction launch: ") + hipGetErrorString(err));
        }
    }

    void launch(gemm_args_t const& a, hipStream_t stream) const
    {
        switch (dtype) {
            case dtype_t::f16:
                return launch_gemm_f16(bm, bn, a, stream);
            case dtype_t::f32:
                return launch_gemm_f32(bm, bn, a, stream);
            case dtype_t::f64:
                return launch_gemm_f64(bm, bn, a, stream);
            default:
                return;
        }
    }
};

}  // namespace

std::shared_ptr<plan_t> plan_contraction(einsummable_t const& e, int)
{
    double alpha = 1.0;
    if (!e.is_scaled_contraction(alpha)) return nullptr;
    dtype_t const dt = e.out_dtype();
    if (dt == dtype_t::c64) return nullptr;  // complex contractions use the generated kernels
    if (e.inn_dtype(0) != dt || e.inn_dtype(1) != dt) return nullptr;

    int const R = int(e.join_shape.size());
    auto stride_in = [&](std::vector<int> const& modes, int m) -> int64_t {
        int64_t s = 1;
        for (int i = int(modes.size()) - 1; i >= 0; --i) {
            if (modes[i] == m) return s;
            s *= int64_t(e.join_shape[modes[i]]);
        }
        return 0;
    };
    std::vector<int> out_modes(e.out_rank);
    for (int i = 0; i != e.out_rank; ++i) out_modes[i] = i;

    std::vector<mode_info_t> bs, is, js, ks;
    for (int m = 0; m != R; ++m) {
        mode_info_t mi{m, e.join_shape[m], stride_in(e.inns[0], m), stride_in(e.inns[1], m),
                       m < e.out_rank ? stride_in(out_modes, m) : 0};
        bool in_l = mi.s_lhs != 0, in_r = mi.s_rhs != 0, in_o = m < e.out_rank;
        if (in_l && in_r && in_o) {
            bs.push_back(mi);
        } else if (in_l && in_r && !in_o) {
            js.push_back(mi);
        } else if (in_l && !in_r && in_o) {
            is.push_back(mi);
        } else if (!in_l && in_r && in_o) {
            ks.push_back(mi);
        } else {
            return nullptr;  // summed over one operand only: not a GEMM
        }
    }
    if (js.empty()) return nullptr;
    if (bs.size() > MAXG || is.size() > MAXG || js.size() > MAXG || ks.size() > MAXG) {
        return nullptr;
    }

    // The operand whose modes own the output's innermost position plays "B" (its group is n,
    // contiguous in C).  If the innermost output mode is a batch mode C is written elementwise.
    bool swapped = false;
    {
        int last = e.out_rank - 1;
        for (auto const& mi : is) swapped = swapped || mi.mode == last;
    }
    auto p = std::make_shared<contraction_plan_t>();
    p->dtype = dt;
    p->swapped = swapped;
    p->bm = 128;
    p->bn = 128;

    std::vector<mode_info_t> gm = swapped ? ks : is;
    std::vector<mode_info_t> gn = swapped ? is : ks;
    int64_t mode_info_t::*sA = swapped ? &mode_info_t::s_rhs : &mode_info_t::s_lhs;
    int64_t mode_info_t::*sB = swapped ? &mode_info_t::s_lhs : &mode_info_t::s_rhs;
    int64_t mode_info_t::*sC = &mode_info_t::s_out;

    // innermost first: m and k ordered by their layout in A, n by its layout in C
    auto by = [](int64_t mode_info_t::*s) {
        return [s](mode_info_t const& x, mode_info_t const& y) { return x.*s < y.*s; };
    };
    std::sort(gm.begin(), gm.end(), by(sA));
    std::sort(gn.begin(), gn.end(), by(sC));
    std::sort(js.begin(), js.end(), by(sA));
    std::sort(bs.begin(), bs.end(), by(sC));

    gemm_args_t& a = p->args;
    std::memset(&a, 0, sizeof(a));
    fill_group(a.gm, gm, sA, sC, nullptr);
    fill_group(a.gn, gn, sB, sC, nullptr);
    fill_group(a.gk, js, sA, sB, nullptr);
    fill_group(a.gb, bs, sA, sB, sC);
    auto prod = [](std::vector<mode_info_t> const& v) {
        uint64_t n = 1;
        for (auto const& m : v) n *= m.size;
        return n;
    };
    uint64_t M = prod(gm), N = prod(gn), K = prod(js), Bt = prod(bs);
    if (gm.empty() || gn.empty()) {
        // matrix-vector shapes keep a unit m / n
    }
    uint64_t const lim = 1ull << 31;
    if (M >= lim || N >= lim || K >= lim || Bt >= 65536) return nullptr;
    if (e.inn_nelem(0) >= (1ull << 40) || e.inn_nelem(1) >= (1ull << 40)) return nullptr;
    a.M = uint32_t(M);
    a.N = uint32_t(N);
    a.K = uint32_t(K);
    a.batch = uint32_t(Bt);

    int const VL = 16 / int(dtype_size(dt));
    auto vec_ok = [&](std::vector<mode_info_t> const& g, int64_t mode_info_t::*s, int q) {
        return !g.empty() && g[0].*s == 1 && g[0].size % uint64_t(q) == 0;
    };
    a.a_mode = vec_ok(js, sA, VL) ? 0 : (vec_ok(gm, sA, VL) ? 1 : 2);
    a.b_mode = vec_ok(js, sB, VL) ? 0 : (vec_ok(gn, sB, VL) ? 1 : 2);
    a.c_mode = vec_ok(gn, sC, VL) ? 3 : (vec_ok(gn, sC, 4) ? 0 : 2);
    a.c_stream = e.out_nelem() * dtype_size(dt) >= (64ull << 20);
    a.offsets_fit_32 = e.inn_nelem(0) * dtype_size(dt) < (1ull << 32) &&
                       e.inn_nelem(1) * dtype_size(dt) < (1ull << 32);

    bool const dma_ok = (dt == dtype_t::f16 && gemm_dma_eligible<_Float16>(a)) ||
                        (dt == dtype_t::f32 && gemm_dma_eligible<float>(a)) ||
                        (dt == dtype_t::f64 && gemm_dma_wide_eligible<double>(a, 4));
    // large tiles exist in the direct-to-LDS kernel (both operands on a vector path) and, for
    // A along k, in the register-staged one
    if (dma_ok || (a.a_mode == 0 && a.b_mode != 2)) {
        // The f16 256 x 256 tile is taken where the eight-wavefront kernel can run it (K in
        // whole 128-byte slices): the four-wavefront instance of that tile needs more registers
        // than a wave has and spills.
        const char* waves = std::getenv("ES_KM_GEMM_WAVES");
        bool const  big_ok = dt != dtype_t::f16 || !dma_ok ||
                            (K % 64 == 0 && !(waves && waves[0] == '4'));
        choose_tile(dt, M, N, K, Bt, dma_ok, big_ok, p->bm, p->bn);
    }
    a.tiles_m = uint32_t((M + p->bm - 1) / p->bm);
    a.tiles_n = uint32_t((N + p->bn - 1) / p->bn);
    if (uint64_t(a.tiles_m) * a.tiles_n >= lim) return nullptr;

    bool const dma = dma_ok;  // every tile has a direct-to-LDS kernel
    p->planned_dma = dma && (dt == dtype_t::f16   ? gemm_dma_eligible<_Float16>(a)
                             : dt == dtype_t::f32 ? gemm_dma_eligible<float>(a)
                                                  : gemm_dma_wide_eligible<double>(a, 4));
    // Too few tiles for the device and a long reduction (skinny products, e.g. one token
    // against a weight matrix): several workgroups share a tile's k range and a second
    // kernel sums their fp32 partial tiles, which live in the workspace.
    a.splits = 1;
    a.alpha = alpha;
    p->workspace_bytes = 0;
    a.lin = a.gm.n == 1 && a.gn.n == 1 && a.gk.n == 1 && a.gn.sy[0] == 1 && a.gm.sy[0] > 0 &&
            uint64_t(a.gm.sy[0]) * 256 * dtype_size(dt) < (1ull << 31);
    {
        uint64_t const in_group = 4ull * a.tiles_n;
        uint64_t const n_tiles = uint64_t(a.tiles_m) * a.tiles_n;
        a.group_magic = n_tiles * in_group < (1ull << 32) ? uint32_t((1ull << 32) / in_group) + 1
                                                          : 0;
    }
    uint64_t const tiles = uint64_t(a.tiles_m) * a.tiles_n * Bt;
    {
        const char* env = std::getenv("ES_KM_GEMM_XCD_BATCH");  // tuning and tests
        a.xcd_total = Bt > 1 && tiles < (1ull << 32) && !(env && env[0] == '0') ? uint32_t(tiles) : 0;
    }
    uint64_t const nk = K * dtype_size(dt) / 64;
    // (the partial tiles of a split product are fp32: not for f64)
    if (p->planned_dma && nk >= 16 && dt != dtype_t::f64) {
        uint64_t S = tiles <= 128 ? std::min<uint64_t>({256 / tiles, nk / 8, 64}) : 1;
        if (const char* env = std::getenv("ES_KM_GEMM_SPLITS")) {  // tuning and tests
            S = std::min<uint64_t>(uint64_t(std::max(1, std::atoi(env))), nk / 4);
        }
        if (S > 1) {
            a.splits = uint32_t(S);
            p->workspace_bytes = S * Bt * M * N * 4;
        }
    }
    a.warm_a_bytes = a.warm_b_bytes = 0;
    if (a.c_stream && dt == dtype_t::f16) {
        uint64_t const lhs = e.inn_nelem(swapped ? 1 : 0) * dtype_size(dt);
        uint64_t const rhs = e.inn_nelem(swapped ? 0 : 1) * dtype_size(dt);
        const char*    env = std::getenv("ES_KM_GEMM_WARM");  // tuning and tests
        if (lhs + rhs <= (160ull << 20) && !(env && env[0] == '0')) {
            a.warm_a_bytes = lhs;
            a.warm_b_bytes = rhs;
        }
    }
    a.shortk = 0;
    if (dt == dtype_t::f16 && p->planned_dma && p->bm == 128 && p->bn == 128 &&
        gemm::gemm_shortk_eligible(a)) {
        const char* env = std::getenv("ES_KM_GEMM_RESIDENT_A");  // tuning and tests
        a.shortk = !(env && env[0] == '0');
    }
    // Products bound by the reads of an operand that is streamed once (attention's P.V, a few
    // rows against a large matrix: the same rule that gives them the small tile) take slices
    // of whole cache lines, two stages and two workgroups per compute unit: P.V of 128 heads
    // of 2048 x 2048 runs in 0.227 instead of 0.253 ms (three stages: 0.242), 40000 x 1024
    // times 1024 x 72 in 22 instead of 28 us.  Not with split-K: a 16384 x 16384 matrix
    // times 128 columns in two shares takes 0.172 against 0.167 ms, eight rows against
    // 8192 x 8192 in four shares 32 against 29 us.
    a.wide_slices = 0;
    {
        double const elem = double(dtype_size(dt));
        double const intensity = 2.0 * double(M) * double(N) * double(K) /
                                 ((double(M) * K + double(N) * K + double(M) * N) * elem);
        bool const can = dt == dtype_t::f16 && p->planned_dma && p->bm == 128 && p->bn == 128 &&
                         !a.shortk && a.a_mode == 0;
        // (a reduction of a few slices has nothing to pipeline with two stages: 2048 x 2048 x
        // 128 per head went from 90 to 107 us)
        if (can && intensity < 150.0 && a.splits <= 1 && K >= 512) a.wide_slices = 2;
        // fp32, at most one tile per compute unit (LDS is then no constraint): four stages of
        // 128-byte slices halve the barriers per k; 2048^3 with B along n 105.7 -> 121.3
        // TFLOP/s, with B along k 123.3 -> 125.4.  With more tiles than compute units two
        // workgroups share one and only two stages fit: 4096^3 141.4 -> 142.8, not taken.
        bool const can32 = dt == dtype_t::f32 && p->planned_dma && p->bm == 128 && p->bn == 128 &&
                           a.a_mode == 0;
        if (can32 && a.splits <= 1 && K >= 512 &&
            uint64_t(a.tiles_m) * a.tiles_n * uint64_t(a.batch) <= 256) {
            a.wide_slices = 4;
        }
        if (const char* env = std::getenv("ES_KM_GEMM_WIDE_SLICES")) {  // tuning and tests
            int const v = std::atoi(env);
            a.wide_slices = ((can && (v == 2 || v == 3)) || (can32 && v >= 2 && v <= 4)) ? v : 0;
        }
        if (a.wide_slices &&
            !(dt == dtype_t::f16
                  ? gemm::gemm_dma_wide_eligible<_Float16>(a, uint32_t(a.wide_slices))
                  : gemm::gemm_dma_wide_eligible<float>(a, uint32_t(a.wide_slices)))) {
            a.wide_slices = 0;
        }
    }
    a.wave8 = 0;
    a.persistent = 0;
    a.workgroups = 0;
    if (dt == dtype_t::f16 && p->planned_dma && a.a_mode <= 1 && a.b_mode <= 1 && !a.shortk &&
        !a.wide_slices && (p->bm == 256 || p->bn == 256) &&
        gemm::gemm_dma_wide_eligible<_Float16>(a, p->bm == 256 && p->bn == 256 ? 2u : 3u)) {
        const char* env = std::getenv("ES_KM_GEMM_WAVES");  // tuning and tests: 4 keeps the old kernel
        a.wave8 = !(env && env[0] == '4');
        // Both operands along k, whole tiles' worth of work for every compute unit: the
        // persistent kernels (ES_KM_GEMM_WAVES=8 keeps the eight-wavefront kernel: tests)
        a.persistent = 0;
        bool const along_k = a.a_mode == 0 && a.b_mode == 0 && a.splits <= 1;
        if (a.wave8 && along_k && !(env && env[0] == '8')) {
            if (p->bm == 256 && p->bn == 256 && gemm::w4::gemm_w4_eligible<2>(a)) {
                a.persistent = 1;
            } else if (p->bm != p->bn && gemm::pc::gemm_pc_eligible(a)) {
                a.persistent = 2;
            }
        }
    }
    if (a.persistent || a.shortk) {
        // one workgroup per compute unit
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
            cus <= 0) {
            a.persistent = 0;
            a.shortk = 0;
            cus = 0;
        }
        a.workgroups = uint32_t(cus);
    }
    static const char* mode_name[] = {"k", "mn", "elem"};
    p->description = std::string("contraction_mfma_") + dtype_name(dt) + " tile=" +
                     std::to_string(p->bm) + "x" + std::to_string(p->bn) + " A=" +
                     mode_name[a.a_mode] + " B=" + mode_name[a.b_mode] + " C=" +
                     (a.c_mode == 3 ? "wide" : (a.c_mode == 0 ? "vec" : "elem")) +
                     (swapped ? " swapped" : "") + (dma ? " load=direct_to_lds" : "") +
                     " M=" + std::to_string(M) + " N=" + std::to_string(N) + " K=" +
                     std::to_string(K) + " batch=" + std::to_string(Bt) +
                     (a.splits > 1 ? " split_k=" + std::to_string(a.splits) : "") +
                     (a.shortk ? " resident_a" : "") + (a.warm_a_bytes ? " warm_operands" : "") +
                     (a.wide_slices ? " slices=128B" : "") +
                     (a.persistent == 1   ? " slices=128B waves=4 persistent"
                      : a.persistent == 2 ? " slices=128B waves=4+4 persistent"
                      : a.wave8           ? " slices=128B waves=8"
                                          : "") +
                     (alpha != 1.0 ? " scaled" : "");
    return p;
}

}  // namespace es
