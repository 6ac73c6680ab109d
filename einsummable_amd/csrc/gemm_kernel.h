// Device side of the contraction path: the strided-batched MFMA GEMM kernel template and its
// argument block.  Included by the planner (contraction.hip) and by the per-dtype translation
// units that instantiate the kernel (gemm_f16.hip, gemm_f32.hip, gemm_f64.hip).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

namespace es
{
namespace gemm
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
    int         c_mode;          // 0: four consecutive n per store, 2: elementwise,
                                 // 3: 16-byte row segments through LDS (tuned kernel)
    int         offsets_fit_32;  // every byte offset into A and B (per batch entry) < 2^32
    int         c_stream;        // C exceeds the caches: store it non-temporally
    // Split-K (direct-to-LDS kernel): `splits` workgroups per tile, one per grid z, each
    // over its own range of k slices, leave fp32 partial tiles in `ws`
    // ([split][batch][M][N]); gemm_fold_kernel sums them into C.
    uint32_t    splits;
    float*      ws;
    // m, n and k are single modes, C is contiguous along n and 256 rows of C span less than
    // 2^31 bytes: every in-tile offset is a 32-bit multiple of a stride
    // Bytes of the two operands when C is streamed past the caches and both operands together
    // fit the memory-side cache with room to spare, else 0: they are then read once, by a
    // kernel of their own, right before the product (gemm_warm_operands).
    uint64_t    warm_a_bytes, warm_b_bytes;
    // tiles_m * tiles_n * batch when the batch has more than one entry and the product fits
    // 32 bits (the XCD renumbering then runs across batch entries), else 0
    uint32_t    xcd_total;
    int         lin;
    // planned for the kernel that keeps A in registers and walks along n (K = 128, fp16)
    int         shortk;
    // floor(2^32 / (4 * tiles_n)) + 1 when tile index * 4 * tiles_n < 2^32 (then the high
    // half of tile * magic is the exact quotient), else 0
    uint32_t    group_magic;
    // 0, or the number of stages (2 or 3) of the direct-to-LDS kernel with 128-byte slices:
    // planned for f16 products bound by the reads of a large operand
    int         wide_slices;
    // f16, both operands along k, compute bound: eight wavefronts per workgroup on slices of
    // 128 bytes (launch_gemm_f16)
    int         wave8;
    // 0, or which of the persistent kernels runs it (f16, both operands along k, compute
    // bound): 1 four wavefronts on 256 x 256 (gemm_w4_kernel), 2 four multiplying and four
    // loading wavefronts on 128 x 256 / 256 x 128 (gemm_pc_kernel); `workgroups`: how many
    // of them walk the tiles (the device's compute units)
    int         persistent;
    uint32_t    workgroups;
    // every sum is multiplied by this before it is rounded to the output type (1 for a plain
    // product); split-K partial tiles stay unscaled, the fold applies it
    double      alpha;
    // Several products of one plan in one launch (gemm_pc_kernel): batch entry g reads and
    // writes at these element offsets from A, B and C instead of the batch strides -- the
    // same operand for all (offset 0 throughout) or buffers that lie anywhere
    uint32_t    grouped;
    int64_t     group_off[3][8];  // [A, B, C][entry]
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

// Workgroups go to the eight XCDs (each with its own L2) round robin in the order of their
// linear index (x fastest, then the batch in y).  The tiles are renumbered so that one XCD
// works on a contiguous run of them -- across batch entries when xcd_total is set: with the
// run inside one batch entry only, every XCD holds a piece of every entry and fetches that
// entry's operands for itself.
__device__ __forceinline__ void xcd_renumber(gemm_args_t const& a, uint32_t n_tiles,
                                             uint32_t& tile, uint32_t& bz)
{
    if (a.xcd_total) {
        uint32_t const linear = tile + n_tiles * bz;
        uint32_t const per_xcd = a.xcd_total / 8;
        if (linear < per_xcd * 8) {
            uint32_t const run = (linear % 8) * per_xcd + linear / 8;
            bz = run / n_tiles;
            tile = run - bz * n_tiles;
        }
    } else {
        uint32_t const per_xcd = n_tiles / 8;
        if (tile < per_xcd * 8) tile = (tile % 8) * per_xcd + tile / 8;
    }
}

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float    float16_t __attribute__((ext_vector_type(16)));
typedef float    float4_t __attribute__((ext_vector_type(4)));
typedef double   double4_t __attribute__((ext_vector_type(4)));
typedef double   double2_t __attribute__((ext_vector_type(2)));

// 16 bytes of an operand row; a native vector so that it lives in registers
typedef uint32_t chunk_t __attribute__((ext_vector_type(4)));

// A 16-byte store that does not allocate in the caches (a C larger than the caches would
// otherwise evict the operand tiles the other workgroups are re-reading).  Written as an
// instruction: with __builtin_nontemporal_store in one arm of a branch and a plain store of
// the same value to the same address in the other, the optimiser merges the two into one
// plain store and the hint is silently lost.
__device__ __forceinline__ void store_16_streaming(void* dst, chunk_t const& v)
{
    asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 1" : : "v"(dst), "v"(v) : "memory");
}

template <typename T>
struct elems_of;
template <>
struct elems_of<_Float16> {
    typedef _Float16 type __attribute__((ext_vector_type(8)));
};
template <>
struct elems_of<float> {
    typedef float type __attribute__((ext_vector_type(4)));
};
template <>
struct elems_of<double> {
    typedef double type __attribute__((ext_vector_type(2)));
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
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, row),
                                                     __builtin_bit_cast(half8_t, col), acc, 0, 0,
                                                     0);
    }
    // n of accumulator element i in lane l
    __device__ static __forceinline__ int acc_row(int i, int lane)
    {
        return (i / 4) * 8 + (lane / 32) * 4 + (i % 4);
    }
    static constexpr bool QUAD = true;  // registers 4q..4q+3 hold four consecutive rows
    // matrix instructions per 16-byte operand chunk, and the t-th of them
    static constexpr int SUB = 1;
    __device__ static __forceinline__ void mma_sub(acc_t& acc, chunk_t const& row,
                                                   chunk_t const& col, int)
    {
        mma(acc, row, col);
    }
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
        float4_t r = __builtin_bit_cast(float4_t, row);
        float4_t c = __builtin_bit_cast(float4_t, col);
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
    static constexpr int SUB = 4;
    __device__ static __forceinline__ void mma_sub(acc_t& acc, chunk_t const& row,
                                                   chunk_t const& col, int t)
    {
        float4_t r = __builtin_bit_cast(float4_t, row);
        float4_t c = __builtin_bit_cast(float4_t, col);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(r[t], c[t], acc, 0, 0, 0);
    }
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
        double2_t r = __builtin_bit_cast(double2_t, row);
        double2_t c = __builtin_bit_cast(double2_t, col);
#pragma unroll
        for (int j = 0; j != 2; ++j) {
            acc = __builtin_amdgcn_mfma_f64_16x16x4f64(r[j], c[j], acc, 0, 0, 0);
        }
    }
    // v_mfma_f64_16x16x4_f64 interleaves rows across registers: register i of lane l holds
    // row 4 * i + l / 16, so a lane's four values are four rows apart
    __device__ static __forceinline__ int acc_row(int i, int lane) { return 4 * i + lane / 16; }
    static constexpr bool QUAD = false;
    // a 16-byte chunk holds two k elements: two matrix instructions
    static constexpr int SUB = 2;
    __device__ static __forceinline__ void mma_sub(acc_t& acc, chunk_t const& row,
                                                   chunk_t const& col, int t)
    {
        double2_t r = __builtin_bit_cast(double2_t, row);
        double2_t c = __builtin_bit_cast(double2_t, col);
        acc = __builtin_amdgcn_mfma_f64_16x16x4f64(r[t], c[t], acc, 0, 0, 0);
    }
};

constexpr int ROW_BYTES = 128;  // bytes of k per tile row per stage
constexpr int ROW_PITCH = 144;  // padded LDS row
constexpr int CHUNKS_PER_ROW = ROW_BYTES / 16;

// Loads one BR x (128 byte) operand slice into registers (NV chunks per thread).
//   mode 0: the slice is [row][k] in memory with k contiguous
//   mode 1: the slice is [k][row] in memory with row contiguous
//   mode 2: arbitrary strides, element by element
// `row_off[v]` / `row_ok[v]` describe the thread's rows (mode 0, 2) or its row-vector (mode 1).
template <typename T, int BR, int NV, int MODE, bool IS_A>
struct operand_loader_t {
    using tr = traits_t<T>;
    static constexpr int VL = tr::VL;
    static constexpr int BK = ROW_BYTES / int(sizeof(T));

    T const*       base;        // tensor + batch offset
    int            mode_rt;     // used when MODE < 0
    uint32_t       R, K;        // extents
    uint32_t       row0;        // first row of the tile
    // mode 0 / 2: per-chunk row offsets
    int64_t        row_off[NV];
    bool           row_ok[NV];

    __device__ __forceinline__ int mode() const { return MODE >= 0 ? MODE : mode_rt; }

    // the groups are read straight from the kernel argument block (scalar registers)
    __device__ __forceinline__ int64_t k_off(gemm_args_t const& g, uint32_t k) const
    {
        int64_t a, b;
        group_offsets(g.gk, k, a, b);
        return IS_A ? a : b;
    }

    __device__ __forceinline__ int64_t r_off(gemm_args_t const& g, uint32_t r) const
    {
        int64_t a, b;
        group_offsets(IS_A ? g.gm : g.gn, r, a, b);
        return a;
    }

    __device__ __forceinline__ void init(gemm_args_t const& g, int tid)
    {
        if (mode() == 1) {
            // chunk v: k-row kk = v / (BR / VL), row vector rv = v % (BR / VL)
#pragma unroll
            for (int i = 0; i != NV; ++i) {
                int      v = tid + 256 * i;
                uint32_t r = row0 + uint32_t(v % (BR / VL)) * VL;
                row_ok[i] = r < R;
                row_off[i] = row_ok[i] ? r_off(g, r) : 0;
            }
        } else {
#pragma unroll
            for (int i = 0; i != NV; ++i) {
                int      v = tid + 256 * i;
                uint32_t r = row0 + uint32_t(v / CHUNKS_PER_ROW);
                row_ok[i] = r < R;
                row_off[i] = row_ok[i] ? r_off(g, r) : 0;
            }
        }
    }

    __device__ __forceinline__ void load(gemm_args_t const& g, int tid, uint32_t k0,
                                         chunk_t (&regs)[NV]) const
    {
        if (mode() == 0) {
            uint32_t k = k0 + uint32_t(tid % CHUNKS_PER_ROW) * VL;
            bool     kok = k < K;
            int64_t  ko = kok ? k_off(g, k) : 0;
#pragma unroll
            for (int i = 0; i != NV; ++i) {
                chunk_t c = {0, 0, 0, 0};
                if (kok && row_ok[i]) {
                    c = *reinterpret_cast<chunk_t const*>(base + row_off[i] + ko);
                }
                regs[i] = c;
            }
        } else if (mode() == 1) {
#pragma unroll
            for (int i = 0; i != NV; ++i) {
                int      v = tid + 256 * i;
                uint32_t k = k0 + uint32_t(v / (BR / VL));
                chunk_t  c = {0, 0, 0, 0};
                if (k < K && row_ok[i]) {
                    c = *reinterpret_cast<chunk_t const*>(base + row_off[i] + k_off(g, k));
                }
                regs[i] = c;
            }
        } else {
            uint32_t kb = k0 + uint32_t(tid % CHUNKS_PER_ROW) * VL;
#pragma unroll
            for (int i = 0; i != NV; ++i) {
                typename elems_of<T>::type e;
#pragma unroll
                for (int j = 0; j != VL; ++j) {
                    uint32_t k = kb + uint32_t(j);
                    e[j] = (k < K && row_ok[i]) ? base[row_off[i] + k_off(g, k)] : T(0);
                }
                regs[i] = __builtin_bit_cast(chunk_t, e);
            }
        }
    }

    // registers -> LDS slice laid out [row][k] with ROW_PITCH bytes per row
    __device__ __forceinline__ void store(int tid, char* lds, chunk_t const (&regs)[NV]) const
    {
        if (mode() == 1) {
#pragma unroll
            for (int i = 0; i != NV; ++i) {
                int v = tid + 256 * i;
                int kk = v / (BR / VL);
                int r = (v % (BR / VL)) * VL;
                typename elems_of<T>::type e = __builtin_bit_cast(typename elems_of<T>::type, regs[i]);
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

// AM / BM_: load path of A / B fixed at compile time (0: vectors along k, 1: vectors along
// m / n), or -1 to take it from the argument block (the general kernel, which also covers the
// element-wise path).
template <typename T, int BM, int BN, int AM, int BM_>
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

    // Tile coordinates.  Workgroups are handed to the 8 XCDs round-robin and every XCD has
    // its own L2, so block b is first sent to the XCD-contiguous position
    // (b % 8) * (tiles / 8) + b / 8: each XCD then owns one contiguous run of the tile order.
    // The order itself walks bands of GROUP_M tile rows column by column, so the tiles an XCD
    // runs at the same time form a compact rectangle that shares its A and B panels in L2.
    uint32_t const n_tiles = a.tiles_m * a.tiles_n;
    uint32_t       tile = blockIdx.x;
    uint32_t       bz = blockIdx.y;
    xcd_renumber(a, n_tiles, tile, bz);
    constexpr uint32_t GROUP_M = 8;
    uint32_t const     in_group = GROUP_M * a.tiles_n;
    uint32_t const     first_m = (tile / in_group) * GROUP_M;
    uint32_t const     rows = (a.tiles_m - first_m) < GROUP_M ? (a.tiles_m - first_m) : GROUP_M;
    uint32_t const     tm = first_m + (tile % in_group) % rows;
    uint32_t const     tn = (tile % in_group) / rows;

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

    operand_loader_t<T, BM, NVA, AM, true> la;
    la.base = static_cast<T const*>(a.A) + boa;
    la.mode_rt = a.a_mode;
    la.R = a.M;
    la.K = a.K;
    la.row0 = tm * BM;
    la.init(a, tid);

    operand_loader_t<T, BN, NVB, BM_, false> lb;
    lb.base = static_cast<T const*>(a.B) + bob;
    lb.mode_rt = a.b_mode;
    lb.R = a.N;
    lb.K = a.K;
    lb.row0 = tn * BN;
    lb.init(a, tid);

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

    la.load(a, tid, 0, ra);
    lb.load(a, tid, 0, rb);
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
            la.load(a, tid, (kt + 1) * BK, ra);
            lb.load(a, tid, (kt + 1) * BK, rb);
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
    typename tr::acc_elem const alpha = typename tr::acc_elem(a.alpha);
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
                if (tr::QUAD && a.c_mode != 2) {
                    uint32_t n = nb + uint32_t(tr::acc_row(e0, lane));
                    if (n < a.N) {
                        int64_t no_b, no_c;
                        group_offsets(a.gn, n, no_b, no_c);
                        struct alignas(4 * sizeof(T)) quad_t {
                            T v[4];
                        } q;
#pragma unroll
                        for (int t = 0; t != 4; ++t) q.v[t] = T(acc[i][j][e0 + t] * alpha);
                        *reinterpret_cast<quad_t*>(C + mo_c + no_c) = q;
                    }
                } else {
#pragma unroll
                    for (int t = 0; t != 4; ++t) {
                        uint32_t n = nb + uint32_t(tr::acc_row(e0 + t, lane));
                        if (n < a.N) {
                            int64_t no_b, no_c;
                            group_offsets(a.gn, n, no_b, no_c);
                            C[mo_c + no_c] = T(acc[i][j][e0 + t] * alpha);
                        }
                    }
                }
            }
        }
    }
}


// ---------------------------------------------------------------------------------------
// The tuned kernel for the vector load paths (A: 16-byte vectors along k; B: along k or n).
// Same tiling and LDS layout as gemm_kernel, with the inner loop written for one resident
// wavefront per SIMD:
//   * loads never branch: out-of-range rows are clamped to the last valid row (their products
//     land in rows of C that are never stored) and a k tail is zeroed with a select;
//   * fragments are double buffered and the instruction order is pinned: each matrix
//     instruction is followed by a 16-byte LDS read of the next k-step;
//   * the next slice goes to LDS during the second-to-last k-step, the workgroup barrier sits
//     before the last k-step, and the last k-step already reads the next slice's first
//     fragments and issues the global loads of the slice after it.
template <typename T, int BM, int BN, int BMODE>
__global__ __launch_bounds__(256) void gemm_fast_kernel(gemm_args_t a)
{
    using tr = traits_t<T>;
    constexpr int MI = tr::MI;
    constexpr int VL = tr::VL;
    constexpr int BK = ROW_BYTES / int(sizeof(T));
    constexpr int WM = BM / 2, WN = BN / 2;
    constexpr int TM = WM / MI, TN = WN / MI;
    constexpr int NVA = BM * CHUNKS_PER_ROW / 256;
    constexpr int NVB = BN * CHUNKS_PER_ROW / 256;
    constexpr int STEPS = BK / (tr::KG * VL);
    constexpr int A_BYTES = BM * ROW_PITCH;
    constexpr int STAGE = (BM + BN) * ROW_PITCH;
    // B kept as [k][n] (BMODE 1): BK rows of BN elements, padded by 16 bytes
    constexpr int PITCH_KN = BN * int(sizeof(T)) + 16;
    static_assert(BK * PITCH_KN <= BN * ROW_PITCH, "the [k][n] layout fits the B region");

    extern __shared__ __attribute__((aligned(16))) char lds[];

    int const tid = threadIdx.x;
    int const lane = tid & 63;
    int const wave = tid >> 6;
    int const wm = wave >> 1, wn = wave & 1;

    uint32_t const n_tiles = a.tiles_m * a.tiles_n;
    uint32_t       tile = blockIdx.x;
    uint32_t       bz = blockIdx.y;
    xcd_renumber(a, n_tiles, tile, bz);
    constexpr uint32_t GROUP_M = 8;
    uint32_t const     in_group = GROUP_M * a.tiles_n;
    uint32_t const     first_m = (tile / in_group) * GROUP_M;
    uint32_t const     rows = (a.tiles_m - first_m) < GROUP_M ? (a.tiles_m - first_m) : GROUP_M;
    uint32_t const     tm = first_m + (tile % in_group) % rows;
    uint32_t const     tn = (tile % in_group) / rows;

    int64_t boa, bob, boc;
    {
        group_offsets(a.gb, bz, boa, bob);
        boc = 0;
        uint32_t i = bz;
#pragma unroll
        for (int d = 0; d != MAXG; ++d) {
            uint32_t q = i / a.gb.size[d];
            boc += int64_t(i - q * a.gb.size[d]) * a.gb.sz[d];
            i = q;
        }
    }
    T const* const A = static_cast<T const*>(a.A) + boa;
    T const* const B = static_cast<T const*>(a.B) + bob;

    // A: chunk i of this thread is row (tid / 8 + 32 i), k-chunk tid % 8
    int64_t a_row[NVA];
#pragma unroll
    for (int i = 0; i != NVA; ++i) {
        uint32_t r = tm * BM + uint32_t(tid / CHUNKS_PER_ROW) + uint32_t(i) * (256 / CHUNKS_PER_ROW);
        r = r < a.M ? r : a.M - 1;
        int64_t x, y;
        group_offsets(a.gm, r, x, y);
        a_row[i] = x;
    }
    // B along k: same shape as A.  B along n: chunk i is k-row (tid / (BN/VL) + i * 256/(BN/VL)),
    // n-vector tid % (BN/VL)
    int64_t b_row[BMODE == 0 ? NVB : 1];
    if constexpr (BMODE == 0) {
#pragma unroll
        for (int i = 0; i != NVB; ++i) {
            uint32_t r = tn * BN + uint32_t(tid / CHUNKS_PER_ROW) + uint32_t(i) * (256 / CHUNKS_PER_ROW);
            r = r < a.N ? r : a.N - 1;
            int64_t x, y;
            group_offsets(a.gn, r, x, y);
            b_row[i] = x;
        }
    } else {
        uint32_t r = tn * BN + uint32_t(tid % (BN / VL)) * VL;
        r = r < a.N ? r : a.N - VL;  // N is a multiple of VL on this path
        int64_t x, y;
        group_offsets(a.gn, r, x, y);
        b_row[0] = x;
    }

    // Loads are unconditional (k beyond K is clamped to 0); whether a chunk is real is decided
    // again when it is written to LDS, so nothing waits on a load before the matrix work.
    auto load_a = [&](uint32_t k0, chunk_t(&regs)[NVA]) {
        uint32_t k = k0 + uint32_t(tid % CHUNKS_PER_ROW) * VL;
        int64_t  x, y;
        group_offsets(a.gk, k < a.K ? k : 0, x, y);
#pragma unroll
        for (int i = 0; i != NVA; ++i) {
            regs[i] = *reinterpret_cast<chunk_t const*>(A + a_row[i] + x);
        }
    };
    auto load_b = [&](uint32_t k0, chunk_t(&regs)[NVB]) {
        if constexpr (BMODE == 0) {
            uint32_t k = k0 + uint32_t(tid % CHUNKS_PER_ROW) * VL;
            int64_t  x, y;
            group_offsets(a.gk, k < a.K ? k : 0, x, y);
#pragma unroll
            for (int i = 0; i != NVB; ++i) {
                regs[i] = *reinterpret_cast<chunk_t const*>(B + b_row[i] + y);
            }
        } else {
#pragma unroll
            for (int i = 0; i != NVB; ++i) {
                uint32_t k = k0 + uint32_t(tid / (BN / VL)) + uint32_t(i) * (256 / (BN / VL));
                int64_t  x, y;
                group_offsets(a.gk, k < a.K ? k : 0, x, y);
                regs[i] = *reinterpret_cast<chunk_t const*>(B + b_row[0] + y);
            }
        }
    };
    // LDS store of chunk q of the thread's A / B registers
    auto store_a1 = [&](char* stage, uint32_t k0, chunk_t const(&regs)[NVA], int q) {
        int  r = tid / CHUNKS_PER_ROW + q * (256 / CHUNKS_PER_ROW);
        bool ok = k0 + uint32_t(tid % CHUNKS_PER_ROW) * VL < a.K;
        *reinterpret_cast<chunk_t*>(stage + r * ROW_PITCH + (tid % CHUNKS_PER_ROW) * 16) =
            ok ? regs[q] : chunk_t{0, 0, 0, 0};
    };
    auto store_b1 = [&](char* stage, uint32_t k0, chunk_t const(&regs)[NVB], int q) {
        if constexpr (BMODE == 0) {
            int  r = tid / CHUNKS_PER_ROW + q * (256 / CHUNKS_PER_ROW);
            bool ok = k0 + uint32_t(tid % CHUNKS_PER_ROW) * VL < a.K;
            *reinterpret_cast<chunk_t*>(stage + A_BYTES + r * ROW_PITCH +
                                        (tid % CHUNKS_PER_ROW) * 16) =
                ok ? regs[q] : chunk_t{0, 0, 0, 0};
        } else {
            // B arrives as rows of consecutive n: kept that way in LDS ([k][n], PITCH_KN bytes
            // per k row); the fragment reads do the transposition
            int  kk = tid / (BN / VL) + q * (256 / (BN / VL));
            bool ok = k0 + uint32_t(kk) < a.K;
            *reinterpret_cast<chunk_t*>(stage + A_BYTES + kk * PITCH_KN + (tid % (BN / VL)) * 16) =
                ok ? regs[q] : chunk_t{0, 0, 0, 0};
        }
    };

    typename tr::acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i != TM; ++i) {
#pragma unroll
        for (int j = 0; j != TN; ++j) {
#pragma unroll
            for (int e = 0; e != tr::NACC; ++e) acc[i][j][e] = 0;
        }
    }

    chunk_t        ra[NVA], rb[NVB];
    uint32_t const nk = (a.K + BK - 1) / BK;

    int const frag = (lane % MI) * ROW_PITCH + (lane / MI) * 16;
    int const fa_base = wm * WM * ROW_PITCH + frag;
    int const fb_base = A_BYTES + wn * WN * ROW_PITCH + frag;

    // fragment q of k-step s: q < TM is an A fragment, the rest are B fragments
    auto read_frag = [&](char const* cur, int s, int q, chunk_t(&fa)[TM], chunk_t(&fb)[TN]) {
        if (q < TM) {
            fa[q] = *reinterpret_cast<chunk_t const*>(cur + fa_base + q * MI * ROW_PITCH +
                                                      s * tr::KG * 16);
        } else if constexpr (BMODE == 0) {
            fb[q - TM] = *reinterpret_cast<chunk_t const*>(cur + fb_base + (q - TM) * MI * ROW_PITCH +
                                                           s * tr::KG * 16);
        } else if constexpr (sizeof(T) == 2) {
            // ds_read_b64_tr_b16: within 16 lanes, lane i supplies the address of 4
            // consecutive n of k-row i / 4 (column group i % 4) and receives, for its own n,
            // the 4 consecutive k: two reads give the 8 k of the MFMA operand.
            typedef short tr_t __attribute__((ext_vector_type(4)));
            int const i16 = lane & 15, blk = lane >> 4;
            int const n0 = wn * WN + (q - TM) * MI + (blk & 1) * 16 + 4 * (i16 & 3);
            int const k0 = s * tr::KG * VL + (blk >> 1) * VL + (i16 >> 2);
            char const* p = cur + A_BYTES + k0 * PITCH_KN + n0 * 2;
            tr_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) tr_t*)(p));
            tr_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) tr_t*)(p + 4 * PITCH_KN));
            typedef short tr8_t __attribute__((ext_vector_type(8)));
            tr8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            fb[q - TM] = __builtin_bit_cast(chunk_t, both);
        } else {
            // 4-byte elements: the operand is one element per lane per instruction, so the
            // [k][n] rows are read directly, lanes along n
            int const n0 = wn * WN + (q - TM) * MI + lane % MI;
            int const k0 = s * tr::KG * VL + (lane / MI) * VL;
            char const* p = cur + A_BYTES + k0 * PITCH_KN + n0 * int(sizeof(T));
            chunk_t v;
#pragma unroll
            for (int t = 0; t != VL; ++t) {
                v[t] = *reinterpret_cast<uint32_t const*>(p + t * PITCH_KN);
            }
            fb[q - TM] = v;
        }
    };
    constexpr int PAIRS = TM * TN;          // matrix-instruction groups per k-step
    constexpr int READS = TM + TN;          // fragment reads per k-step
    constexpr int STORES = NVA + NVB;       // LDS stores per slice
    constexpr int READS_PER_PAIR = (READS + PAIRS - 1) / PAIRS;
    constexpr int STORES_PER_PAIR = (STORES + PAIRS - 1) / PAIRS;
    static_assert(STEPS >= 2, "the pipeline needs two k-steps per slice");

    chunk_t fa[2][TM], fb[2][TN];

    // prologue: slice 0 into stage 0, slice 1 on its way, first fragments in registers
    load_a(0, ra);
    load_b(0, rb);
#pragma unroll
    for (int q = 0; q != NVA; ++q) store_a1(lds, 0, ra, q);
#pragma unroll
    for (int q = 0; q != NVB; ++q) store_b1(lds, 0, rb, q);
    __syncthreads();
    load_a(BK, ra);
    load_b(BK, rb);
#pragma unroll
    for (int q = 0; q != READS; ++q) read_frag(lds, 0, q, fa[0], fb[0]);

    // One slice kt.  Program order is the issue order of the resident wave, so every matrix
    // instruction is followed by its share of the side work, which runs in its shadow:
    //   steps 0 .. STEPS-3 : fragment reads of the next step
    //   step  STEPS-2      : fragment reads of the last step + LDS stores of slice kt+1
    //   barrier            : slice kt+1 is complete in the other stage
    //   step  STEPS-1      : first fragments of slice kt+1, global loads of slice kt+2
    // so the matrix cores never wait for LDS at a slice boundary.
    auto slice = [&](uint32_t kt, auto has_next_tag) {
        constexpr bool HAS_NEXT = decltype(has_next_tag)::value;
        char const*    cur = lds + (kt & 1) * STAGE;
        char*          nxt = lds + ((kt + 1) & 1) * STAGE;
#pragma unroll
        for (int s = 0; s != STEPS; ++s) {
            if (HAS_NEXT && s == STEPS - 1) {
                __syncthreads();
                load_a((kt + 2) * BK, ra);
                load_b((kt + 2) * BK, rb);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int p = 0; p != PAIRS; ++p) {
                tr::mma(acc[p / TN][p % TN], fb[s & 1][p % TN], fa[s & 1][p / TN]);
                if (s + 1 != STEPS) {
#pragma unroll
                    for (int r = 0; r != READS_PER_PAIR; ++r) {
                        int q = p * READS_PER_PAIR + r;
                        if (q < READS) read_frag(cur, s + 1, q, fa[(s + 1) & 1], fb[(s + 1) & 1]);
                    }
                } else if (HAS_NEXT) {
#pragma unroll
                    for (int r = 0; r != READS_PER_PAIR; ++r) {
                        int q = p * READS_PER_PAIR + r;
                        if (q < READS) read_frag(nxt, 0, q, fa[0], fb[0]);
                    }
                }
                if (HAS_NEXT && s == STEPS - 2) {
#pragma unroll
                    for (int r = 0; r != STORES_PER_PAIR; ++r) {
                        int q = p * STORES_PER_PAIR + r;
                        if (q < NVA) {
                            store_a1(nxt, (kt + 1) * BK, ra, q);
                        } else if (q < STORES) {
                            store_b1(nxt, (kt + 1) * BK, rb, q - NVA);
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    static_assert(STEPS % 2 == 0, "fragment buffers alternate per k-step");
    for (uint32_t kt = 0; kt + 1 < nk; ++kt) slice(kt, std::true_type{});
    slice(nk - 1, std::false_type{});

    T* const C = static_cast<T*>(a.C) + boc;
    typename tr::acc_elem const alpha = typename tr::acc_elem(a.alpha);
    if (a.c_mode == 3) {
        // Wide epilogue: each wave turns MI rows of its tile through a private LDS strip so
        // that the global stores are 16 bytes per lane and whole row segments per wavefront
        // (the accumulator layout alone gives 8-byte stores scattered over 32 rows).
        constexpr int STRIP_PITCH = WN * int(sizeof(T)) + 16;
        constexpr int CPR = WN * int(sizeof(T)) / 16;  // 16-byte chunks per strip row
        __syncthreads();                                // every wave is done with the stages
        char* const strip = lds + wave * (MI * STRIP_PITCH);
        typedef T quad_t __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int i = 0; i != TM; ++i) {
#pragma unroll
            for (int j = 0; j != TN; ++j) {
#pragma unroll
                for (int e0 = 0; e0 < tr::NACC; e0 += 4) {
                    quad_t q;
#pragma unroll
                    for (int t = 0; t != 4; ++t) q[t] = T(acc[i][j][e0 + t] * alpha);
                    int n = j * MI + tr::acc_row(e0, lane);
                    *reinterpret_cast<quad_t*>(strip + (lane % MI) * STRIP_PITCH +
                                               n * int(sizeof(T))) = q;
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int c = 0; c != MI * CPR / 64; ++c) {
                int      idx = c * 64 + lane;
                int      r = idx / CPR, ch = idx % CPR;
                uint32_t m = tm * BM + wm * WM + i * MI + uint32_t(r);
                uint32_t n = tn * BN + wn * WN + uint32_t(ch) * VL;
                chunk_t  v = *reinterpret_cast<chunk_t const*>(strip + r * STRIP_PITCH + ch * 16);
                if (m < a.M && n < a.N) {
                    int64_t mo_a, mo_c, no_b, no_c;
                    group_offsets(a.gm, m, mo_a, mo_c);
                    group_offsets(a.gn, n, no_b, no_c);
                    *reinterpret_cast<chunk_t*>(C + mo_c + no_c) = v;
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
        return;
    }
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
                if (a.c_mode != 2) {
                    uint32_t n = nb + uint32_t(tr::acc_row(e0, lane));
                    if (n < a.N) {
                        int64_t no_b, no_c;
                        group_offsets(a.gn, n, no_b, no_c);
                        typedef T quad_t __attribute__((ext_vector_type(4)));
                        quad_t q;
#pragma unroll
                        for (int t = 0; t != 4; ++t) q[t] = T(acc[i][j][e0 + t] * alpha);
                        *reinterpret_cast<quad_t*>(C + mo_c + no_c) = q;
                    }
                } else {
#pragma unroll
                    for (int t = 0; t != 4; ++t) {
                        uint32_t n = nb + uint32_t(tr::acc_row(e0 + t, lane));
                        if (n < a.N) {
                            int64_t no_b, no_c;
                            group_offsets(a.gn, n, no_b, no_c);
                            C[mo_c + no_c] = T(acc[i][j][e0 + t] * alpha);
                        }
                    }
                }
            }
        }
    }
}

// Host launcher implemented once per dtype.  am / bm_ select a compile-time load path when
// such an instantiation exists; the general kernel is used otherwise.
void launch_gemm_f16(int bm, int bn, gemm_args_t const& a, hipStream_t stream);
void launch_gemm_f32(int bm, int bn, gemm_args_t const& a, hipStream_t stream);
void launch_gemm_f64(int bm, int bn, gemm_args_t const& a, hipStream_t stream);
double probe_mfma_f16(void const* operands, void* scratch, int blocks, int iters,
                      hipStream_t stream);

// Reads `bytes` at `p` and keeps nothing: the lines end up in the L2 and in the memory-side
// cache behind it.  Used ahead of a product whose output is written at HBM speed: operand
// reads that have to go to HBM in the middle of that write stream cost far more than their
// size suggests (attention scores, 128 MiB of operands against 1 GiB of output: 0.35 ms
// with cold operands, 0.21 ms with warm ones plus 0.03 ms for warming them).
void gemm_warm_operands(void const* p, uint64_t bytes_p, void const* q, uint64_t bytes_q,
                        hipStream_t stream);

// The fp16 kernel for reductions of exactly 128 elements (gemm_shortk_kernel.h)
bool gemm_shortk_eligible(gemm_args_t const& a);
void launch_gemm_shortk(gemm_args_t const& a, hipStream_t stream);

// the same problem cut into bm x bn tiles
inline gemm_args_t with_tile(gemm_args_t a, int bm, int bn)
{
    a.tiles_m = (a.M + uint32_t(bm) - 1) / uint32_t(bm);
    a.tiles_n = (a.N + uint32_t(bn) - 1) / uint32_t(bn);
    a.group_magic = 0;  // belongs to the tile counts it was computed for
    uint64_t const total = uint64_t(a.tiles_m) * a.tiles_n * a.batch;
    a.xcd_total = a.xcd_total && total < (1ull << 32) ? uint32_t(total) : 0;
    return a;
}

template <typename T, int BM, int BN, int AM, int BM_>
void launch_gemm_kernel(gemm_args_t const& a, hipStream_t stream)
{
    constexpr size_t lds = size_t(2) * size_t(BM + BN) * ROW_PITCH;
    // more than 64 KiB of dynamic LDS has to be requested once per kernel
    static bool const raised = [] {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<T, BM, BN, AM, BM_>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));
        return true;
    }();
    (void)raised;
    dim3 grid(a.tiles_m * a.tiles_n, a.batch, 1);
    hipLaunchKernelGGL((gemm_kernel<T, BM, BN, AM, BM_>), grid, dim3(256), lds, stream, a);
}

template <typename T, int BM, int BN, int BMODE>
void launch_gemm_fast_kernel(gemm_args_t const& a, hipStream_t stream)
{
    constexpr size_t lds = size_t(2) * size_t(BM + BN) * ROW_PITCH;
    static bool const raised = [] {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_fast_kernel<T, BM, BN, BMODE>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));
        return true;
    }();
    (void)raised;
    dim3 grid(a.tiles_m * a.tiles_n, a.batch, 1);
    hipLaunchKernelGGL((gemm_fast_kernel<T, BM, BN, BMODE>), grid, dim3(256), lds, stream, a);
}

// dispatch of one dtype over tiles and compile-time load paths
template <typename T, int BM, int BN>
bool launch_gemm_fast(gemm_args_t const& a, hipStream_t stream)
{
    if (a.a_mode == 0 && a.b_mode == 0) {
        launch_gemm_fast_kernel<T, BM, BN, 0>(a, stream);
        return true;
    }
    if (a.a_mode == 0 && a.b_mode == 1) {
        launch_gemm_fast_kernel<T, BM, BN, 1>(a, stream);
        return true;
    }
    return false;
}

}  // namespace gemm
}  // namespace es
