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
// fp16 inputs accumulate in fp32 (v_mfma_f32_32x32x16_f16), fp32 uses v_mfma_f32_32x32x2_f32,
// f64 uses v_mfma_f64_16x16x4_f64.
#include "kernel_manager.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>

namespace es
{
namespace
{

constexpr int MAXG = 4;  // modes per group

// One group of modes, innermost first.  Unused slots have size 1 and stride 0.
struct group_t {
    uint32_t n;
    uint32_t size[MAXG];
    int64_t  sx[MAXG];  // stride in the first tensor that holds the group
    int64_t  sy[MAXG];  // stride in the second tensor that holds the group
    int64_t  sz[MAXG];  // batch only: stride in C
};

struct gemm_args_t {
    const void* A;
    const void* B;
    void*       C;
    uint32_t    M, N, K, batch;
    uint32_t    tiles_m, tiles_n;
    group_t     gm;  // sx: A, sy: C
    group_t     gn;  // sx: B, sy: C
    group_t     gk;  // sx: A, sy: B
    group_t     gb;  // sx: A, sy: B, sz: C
    int         a_mode, b_mode;  // 0: 16-byte vectors along k, 1: along m / n, 2: elementwise
    int         c_mode;          // 0: four consecutive n per store, 2: elementwise
};

__device__ __forceinline__ void group_offsets(group_t const& g, uint32_t i, int64_t& ox,
                                              int64_t& oy)
{
    if (g.n == 1) {
        ox = int64_t(i) * g.sx[0];
        oy = int64_t(i) * g.sy[0];
        return;
    }
    ox = 0;
    oy = 0;
#pragma unroll
    for (int d = 0; d != MAXG; ++d) {
        uint32_t q = i / g.size[d];
        uint32_t r = i - q * g.size[d];
        ox += int64_t(r) * g.sx[d];
        oy += int64_t(r) * g.sy[d];
        i = q;
    }
}

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float    float16_t __attribute__((ext_vector_type(16)));
typedef float    float4_t __attribute__((ext_vector_type(4)));
typedef double   double4_t __attribute__((ext_vector_type(4)));

struct alignas(16) chunk_t {
    uint32_t w[4];
};

template <typename T>
struct traits_t;

template <>
struct traits_t<_Float16> {
    static constexpr int MI = 32;    // rows/cols of one MFMA tile
    static constexpr int VL = 8;     // elements in a 16-byte chunk
    static constexpr int KG = 2;     // lane groups along k (64 / MI)
    static constexpr int NACC = 16;  // accumulator elements per lane per tile
    using acc_elem = float;
    using acc_t = float16_t;
    __device__ static __forceinline__ void mma(acc_t& acc, chunk_t const& row, chunk_t const& col)
    {
        half8_t r, c;
        __builtin_memcpy(&r, &row, 16);
        __builtin_memcpy(&c, &col, 16);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(r, c, acc, 0, 0, 0);
    }
    // n of accumulator element i in lane l
    __device__ static __forceinline__ int acc_row(int i, int lane)
    {
        return (i / 4) * 8 + (lane / 32) * 4 + (i % 4);
    }
    static constexpr bool QUAD = true;  // registers 4q..4q+3 hold four consecutive rows
};

template <>
struct traits_t<float> {
    static constexpr int MI = 32;
    static constexpr int VL = 4;
    static constexpr int KG = 2;
    static constexpr int NACC = 16;
    using acc_elem = float;
    using acc_t = float16_t;
    __device__ static __forceinline__ void mma(acc_t& acc, chunk_t const& row, chunk_t const& col)
    {
        float r[4], c[4];
        __builtin_memcpy(r, &row, 16);
        __builtin_memcpy(c, &col, 16);
#pragma unroll
        for (int j = 0; j != 4; ++j) {
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(r[j], c[j], acc, 0, 0, 0);
        }
    }
    __device__ static __forceinline__ int acc_row(int i, int lane)
    {
        return (i / 4) * 8 + (lane / 32) * 4 + (i % 4);
    }
    static constexpr bool QUAD = true;  // registers 4q..4q+3 hold four consecutive rows
};

template <>
struct traits_t<double> {
    static constexpr int MI = 16;
    static constexpr int VL = 2;
    static constexpr int KG = 4;
    static constexpr int NACC = 4;
    using acc_elem = double;
    using acc_t = double4_t;
    __device__ static __forceinline__ void mma(acc_t& acc, chunk_t const& row, chunk_t const& col)
    {
        double r[2], c[2];
        __builtin_memcpy(r, &row, 16);
        __builtin_memcpy(c, &col, 16);
#pragma unroll
        for (int j = 0; j != 2; ++j) {
            acc = __builtin_amdgcn_mfma_f64_16x16x4f64(r[j], c[j], acc, 0, 0, 0);
        }
    }
    // v_mfma_f64_16x16x4_f64 interleaves rows across registers: register i of lane l holds
    // row 4 * i + l / 16, so a lane's four values are four rows apart
    __device__ static __forceinline__ int acc_row(int i, int lane) { return 4 * i + lane / 16; }
    static constexpr bool QUAD = false;
};

constexpr int ROW_BYTES = 128;  // bytes of k per tile row per stage
constexpr int ROW_PITCH = 144;  // padded LDS row
constexpr int CHUNKS_PER_ROW = ROW_BYTES / 16;

// Loads one BR x (128 byte) operand slice into registers (NV chunks per thread).
//   mode 0: the slice is [row][k] in memory with k contiguous
//   mode 1: the slice is [k][row] in memory with row contiguous
//   mode 2: arbitrary strides, element by element
// `row_off[v]` / `row_ok[v]` describe the thread's rows (mode 0, 2) or its row-vector (mode 1).
template <typename T, int BR, int NV>
struct operand_loader_t {
    using tr = traits_t<T>;
    static constexpr int VL = tr::VL;
    static constexpr int BK = ROW_BYTES / int(sizeof(T));

    T const*       base;        // tensor + batch offset
    group_t const* grow;        // m or n group
    group_t const* gk;
    bool           use_sy_k;    // k strides: sx for A, sy for B
    int            mode;
    uint32_t       R, K;        // extents
    uint32_t       row0;        // first row of the tile
    // mode 0 / 2: per-chunk row offsets
    int64_t        row_off[NV];
    bool           row_ok[NV];

    __device__ __forceinline__ int64_t k_off(uint32_t k) const
    {
        int64_t a, b;
        group_offsets(*gk, k, a, b);
        return use_sy_k ? b : a;
    }

    __device__ __forceinline__ int64_t r_off(uint32_t r) const
    {
        int64_t a, b;
        group_offsets(*grow, r, a, b);
        return a;
    }

    __device__ void init(int tid)
    {
        if (mode == 1) {
            // chunk v: k-row kk = v / (BR / VL), row vector rv = v % (BR / VL)
#pragma unroll
            for (int i = 0; i != NV; ++i) {
                int      v = tid + 256 * i;
                uint32_t r = row0 + uint32_t(v % (BR / VL)) * VL;
                row_ok[i] = r < R;
                row_off[i] = row_ok[i] ? r_off(r) : 0;
            }
        } else {
#pragma unroll
            for (int i = 0; i != NV; ++i) {
                int      v = tid + 256 * i;
                uint32_t r = row0 + uint32_t(v / CHUNKS_PER_ROW);
                row_ok[i] = r < R;
                row_off[i] = row_ok[i] ? r_off(r) : 0;
            }
        }
    }

    __device__ __forceinline__ void load(int tid, uint32_t k0, chunk_t (&regs)[NV]) const
    {
        if (mode == 0) {
            uint32_t k = k0 + uint32_t(tid % CHUNKS_PER_ROW) * VL;
            bool     kok = k < K;
            int64_t  ko = kok ? k_off(k) : 0;
#pragma unroll
            for (int i = 0; i != NV; ++i) {
                chunk_t c = {{0, 0, 0, 0}};
                if (kok && row_ok[i]) {
                    c = *reinterpret_cast<chunk_t const*>(base + row_off[i] + ko);
                }
                regs[i] = c;
            }
        } else if (mode == 1) {
#pragma unroll
            for (int i = 0; i != NV; ++i) {
                int      v = tid + 256 * i;
                uint32_t k = k0 + uint32_t(v / (BR / VL));
                chunk_t  c = {{0, 0, 0, 0}};
                if (k < K && row_ok[i]) {
                    c = *reinterpret_cast<chunk_t const*>(base + row_off[i] + k_off(k));
                }
                regs[i] = c;
            }
        } else {
            uint32_t kb = k0 + uint32_t(tid % CHUNKS_PER_ROW) * VL;
#pragma unroll
            for (int i = 0; i != NV; ++i) {
                T e[VL];
#pragma unroll
                for (int j = 0; j != VL; ++j) {
                    uint32_t k = kb + uint32_t(j);
                    e[j] = (k < K && row_ok[i]) ? base[row_off[i] + k_off(k)] : T(0);
                }
                __builtin_memcpy(&regs[i], e, 16);
            }
        }
    }

    // registers -> LDS slice laid out [row][k] with ROW_PITCH bytes per row
    __device__ __forceinline__ void store(int tid, char* lds, chunk_t const (&regs)[NV]) const
    {
        if (mode == 1) {
#pragma unroll
            for (int i = 0; i != NV; ++i) {
                int v = tid + 256 * i;
                int kk = v / (BR / VL);
                int r = (v % (BR / VL)) * VL;
                T   e[VL];
                __builtin_memcpy(e, &regs[i], 16);
#pragma unroll
                for (int j = 0; j != VL; ++j) {
                    *reinterpret_cast<T*>(lds + (r + j) * ROW_PITCH + kk * int(sizeof(T))) = e[j];
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i != NV; ++i) {
                int v = tid + 256 * i;
                int r = v / CHUNKS_PER_ROW;
                int c = v % CHUNKS_PER_ROW;
                *reinterpret_cast<chunk_t*>(lds + r * ROW_PITCH + c * 16) = regs[i];
            }
        }
    }
};

template <typename T, int BM, int BN>
__global__ __launch_bounds__(256) void gemm_kernel(gemm_args_t a)
{
    using tr = traits_t<T>;
    constexpr int MI = tr::MI;
    constexpr int VL = tr::VL;
    constexpr int BK = ROW_BYTES / int(sizeof(T));
    constexpr int WM = BM / 2, WN = BN / 2;  // wave tile
    constexpr int TM = WM / MI, TN = WN / MI;
    constexpr int NVA = BM * CHUNKS_PER_ROW / 256;
    constexpr int NVB = BN * CHUNKS_PER_ROW / 256;
    constexpr int STEPS = BK / (tr::KG * VL);

    extern __shared__ __attribute__((aligned(16))) char lds[];
    constexpr int A_BYTES = BM * ROW_PITCH;
    constexpr int STAGE = (BM + BN) * ROW_PITCH;

    int const tid = threadIdx.x;
    int const lane = tid & 63;
    int const wave = tid >> 6;
    int const wm = wave >> 1, wn = wave & 1;

    // tile coordinates; consecutive blocks walk down m first so that they share the B panel
    uint32_t const tile = blockIdx.x;
    uint32_t const tm = tile % a.tiles_m;
    uint32_t const tn = tile / a.tiles_m;
    uint32_t const bz = blockIdx.y;

    int64_t boa, bob, boc;
    {
        int64_t x, y;
        group_offsets(a.gb, bz, x, y);
        boa = x;
        bob = y;
        // C strides of the batch group
        boc = 0;
        uint32_t i = bz;
#pragma unroll
        for (int d = 0; d != MAXG; ++d) {
            uint32_t q = i / a.gb.size[d];
            boc += int64_t(i - q * a.gb.size[d]) * a.gb.sz[d];
            i = q;
        }
    }

    operand_loader_t<T, BM, NVA> la;
    la.base = static_cast<T const*>(a.A) + boa;
    la.grow = &a.gm;
    la.gk = &a.gk;
    la.use_sy_k = false;
    la.mode = a.a_mode;
    la.R = a.M;
    la.K = a.K;
    la.row0 = tm * BM;
    la.init(tid);

    operand_loader_t<T, BN, NVB> lb;
    lb.base = static_cast<T const*>(a.B) + bob;
    lb.grow = &a.gn;
    lb.gk = &a.gk;
    lb.use_sy_k = true;
    lb.mode = a.b_mode;
    lb.R = a.N;
    lb.K = a.K;
    lb.row0 = tn * BN;
    lb.init(tid);

    typename tr::acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i != TM; ++i) {
#pragma unroll
        for (int j = 0; j != TN; ++j) {
#pragma unroll
            for (int e = 0; e != tr::NACC; ++e) acc[i][j][e] = 0;
        }
    }

    chunk_t ra[NVA], rb[NVB];
    uint32_t const nk = (a.K + BK - 1) / BK;

    la.load(tid, 0, ra);
    lb.load(tid, 0, rb);
    la.store(tid, lds, ra);
    lb.store(tid, lds + A_BYTES, rb);
    __syncthreads();

    // fragment addresses of this lane inside a stage
    int const frow = lane % MI;
    int const fk = (lane / MI) * 16;

    for (uint32_t kt = 0; kt != nk; ++kt) {
        char const* cur = lds + (kt & 1) * STAGE;
        char*       nxt = lds + ((kt + 1) & 1) * STAGE;
        bool const  more = kt + 1 != nk;
        if (more) {
            la.load(tid, (kt + 1) * BK, ra);
            lb.load(tid, (kt + 1) * BK, rb);
        }
#pragma unroll
        for (int s = 0; s != STEPS; ++s) {
            chunk_t fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i != TM; ++i) {
                fa[i] = *reinterpret_cast<chunk_t const*>(
                    cur + (wm * WM + i * MI + frow) * ROW_PITCH + s * tr::KG * 16 + fk);
            }
#pragma unroll
            for (int j = 0; j != TN; ++j) {
                fb[j] = *reinterpret_cast<chunk_t const*>(
                    cur + A_BYTES + (wn * WN + j * MI + frow) * ROW_PITCH + s * tr::KG * 16 + fk);
            }
#pragma unroll
            for (int i = 0; i != TM; ++i) {
#pragma unroll
                for (int j = 0; j != TN; ++j) tr::mma(acc[i][j], fb[j], fa[i]);
            }
        }
        if (more) {
            la.store(tid, nxt, ra);
            lb.store(tid, nxt + A_BYTES, rb);
        }
        __syncthreads();
    }

    // epilogue: lane holds, per tile, NACC values: n = acc_row(e, lane), m = lane % MI
    T* const C = static_cast<T*>(a.C) + boc;
#pragma unroll
    for (int i = 0; i != TM; ++i) {
        uint32_t m = tm * BM + wm * WM + i * MI + lane % MI;
        if (m >= a.M) continue;
        int64_t mo_a, mo_c;
        group_offsets(a.gm, m, mo_a, mo_c);
#pragma unroll
        for (int j = 0; j != TN; ++j) {
            uint32_t nb = tn * BN + wn * WN + j * MI;
#pragma unroll
            for (int e0 = 0; e0 < tr::NACC; e0 += 4) {
                if (tr::QUAD && a.c_mode == 0) {
                    uint32_t n = nb + uint32_t(tr::acc_row(e0, lane));
                    if (n < a.N) {
                        int64_t no_b, no_c;
                        group_offsets(a.gn, n, no_b, no_c);
                        struct alignas(4 * sizeof(T)) quad_t {
                            T v[4];
                        } q;
#pragma unroll
                        for (int t = 0; t != 4; ++t) q.v[t] = T(acc[i][j][e0 + t]);
                        *reinterpret_cast<quad_t*>(C + mo_c + no_c) = q;
                    }
                } else {
#pragma unroll
                    for (int t = 0; t != 4; ++t) {
                        uint32_t n = nb + uint32_t(tr::acc_row(e0 + t, lane));
                        if (n < a.N) {
                            int64_t no_b, no_c;
                            group_offsets(a.gn, n, no_b, no_c);
                            C[mo_c + no_c] = T(acc[i][j][e0 + t]);
                        }
                    }
                }
            }
        }
    }
}

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

// Adjacent modes of a group that are also adjacent (same order, dense) in every tensor that
// holds them were already fused by merge_adjacent_dims; what is left is genuinely strided.
struct contraction_plan_t : plan_t {
    gemm_args_t args;
    dtype_t     dtype;
    bool        swapped;
    int         bm, bn;

    void run(hipStream_t stream, void* out, void const* const* inns, void*, uint64_t) const override
    {
        gemm_args_t a = args;
        a.A = swapped ? inns[1] : inns[0];
        a.B = swapped ? inns[0] : inns[1];
        a.C = out;
        // vector paths need 16-byte aligned operands
        auto mis = [](void const* p) { return reinterpret_cast<uintptr_t>(p) % 16 != 0; };
        if (mis(a.A) && a.a_mode != 2) a.a_mode = 2;
        if (mis(a.B) && a.b_mode != 2) a.b_mode = 2;
        if (mis(a.C) && a.c_mode != 2) a.c_mode = 2;
        dim3   grid(a.tiles_m * a.tiles_n, a.batch, 1);
        size_t lds = size_t(2) * size_t(bm + bn) * ROW_PITCH;
        // more than 64 KiB of dynamic LDS has to be requested once per kernel
        static bool const raised = [lds] {
            int n = int(lds);
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<_Float16, 128, 128>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, n);
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<float, 128, 128>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, n);
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<double, 128, 128>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, n);
            return true;
        }();
        (void)raised;
        switch (dtype) {
            case dtype_t::f16:
                hipLaunchKernelGGL((gemm_kernel<_Float16, 128, 128>), grid, dim3(256), lds, stream,
                                   a);
                break;
            case dtype_t::f32:
                hipLaunchKernelGGL((gemm_kernel<float, 128, 128>), grid, dim3(256), lds, stream, a);
                break;
            case dtype_t::f64:
                hipLaunchKernelGGL((gemm_kernel<double, 128, 128>), grid, dim3(256), lds, stream,
                                   a);
                break;
            default:
                break;
        }
        hipError_t err = hipGetLastError();
        if (err != hipSuccess) {
            throw km_error(km_status::device,
                           std::string("contraction launch: ") + hipGetErrorString(err));
        }
    }
};

}  // namespace

std::shared_ptr<plan_t> plan_contraction(einsummable_t const& e, int)
{
    if (!e.is_contraction()) return nullptr;
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
    a.tiles_m = uint32_t((M + p->bm - 1) / p->bm);
    a.tiles_n = uint32_t((N + p->bn - 1) / p->bn);
    if (uint64_t(a.tiles_m) * a.tiles_n >= lim) return nullptr;

    int const VL = 16 / int(dtype_size(dt));
    auto vec_ok = [&](std::vector<mode_info_t> const& g, int64_t mode_info_t::*s, int q) {
        return !g.empty() && g[0].*s == 1 && g[0].size % uint64_t(q) == 0;
    };
    a.a_mode = vec_ok(js, sA, VL) ? 0 : (vec_ok(gm, sA, VL) ? 1 : 2);
    a.b_mode = vec_ok(js, sB, VL) ? 0 : (vec_ok(gn, sB, VL) ? 1 : 2);
    a.c_mode = vec_ok(gn, sC, 4) ? 0 : 2;

    p->workspace_bytes = 0;
    static const char* mode_name[] = {"k", "mn", "elem"};
    p->description = std::string("contraction_mfma_") + dtype_name(dt) + " tile=128x128 A=" +
                     mode_name[a.a_mode] + " B=" + mode_name[a.b_mode] + " C=" +
                     (a.c_mode == 0 ? "vec" : "elem") + (swapped ? " swapped" : "") +
                     " M=" + std::to_string(M) + " N=" + std::to_string(N) + " K=" +
                     std::to_string(K) + " batch=" + std::to_string(Bt);
    return p;
}

}  // namespace es
