// 256 x 256 macro-tile GEMM whose operand slices go from global memory straight into LDS
// (global_load_lds_dwordx4), for problems where each operand is contiguous along k or along
// its own m / n mode (all four matmul transposes and their batched / multi-mode relatives).
//
// Why a second kernel: with 128 x 128 tiles every flop costs twice the LDS and L1 traffic of a
// 256 x 256 tile, and both are what limits the register-staged kernel.  A 256 x 256 tile per
// workgroup of four wavefronts needs 256 accumulator registers per lane, which leaves no room
// for register staging of the next slice; the direct-to-LDS loads need none.
//
//   * WGM x WGN wavefronts, each owning (BM/WGM) x (BN/WGN) of C: 2 x 2 (128 x 128 = 4 x 4 MFMA
//     tiles = 256 accumulators for the 256 x 256 tile), or eight of them, 2 x 4 or 4 x 2, two
//     per SIMD, for the compute-bound f16 products (launch_gemm_f16 says which and why).
//   * LDS: NS stages of (BM + BN) rows x 64 bytes.  Loads run NS - 1 slices ahead of the
//     matrix work; one workgroup barrier per slice.
//   * One load instruction moves 16 rows x 64 bytes; a wavefront's 64 x 16 bytes land
//     contiguously in LDS (lane l at +16 l), so rows cannot be padded.  Instead the four
//     16-byte chunks of a row are XOR-swizzled with bits 2..3 of the row number, applied on
//     the global address of the load and again on the fragment read: sixteen consecutive rows
//     of one k-chunk then cover all 64 banks once.
//   * The loads are written as inline assembly so that the compiler does not serialise the
//     pipeline with a full vmcnt wait in front of every LDS read; the waits are explicit
//     (each lane issues 8 loads per slice, so "slice kt+1 has landed" is vmcnt <= 8 x the
//     number of younger slices in flight).
//   * K must be a multiple of the slice (64 bytes) and at least four slices (>= NS); rows beyond M / N
//     are clamped on load (their results are never stored).
#pragma once
#include "gemm_kernel.h"

namespace es
{
namespace gemm
{

constexpr int DMA_ROW = 64;  // bytes of k per row per stage

// 64 lanes x 16 bytes from `base + voff` (per lane) to LDS at `lds_addr + 16 * lane`
__device__ __forceinline__ void load_to_lds_16(void const* base, uint32_t voff, uint32_t lds_addr)
{
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %1, %2"
        :
        : "s"(lds_addr), "v"(voff), "s"(base)
        : "memory");  // m0 is not kept live by the compiler across statements
}

// 64 lanes x 4 bytes from `base + voff` (per lane) to LDS at `lds_addr + 4 * lane`
__device__ __forceinline__ void load_to_lds_4(void const* base, uint32_t voff, uint32_t lds_addr)
{
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dword %1, %2"
        :
        : "s"(lds_addr), "v"(voff), "s"(base)
        : "memory");
}

template <int VM>
__device__ __forceinline__ void wait_loads_and_lds()
{
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" : : "n"(VM) : "memory");
}

// RB: bytes of k per row per slice, 64 or 128.  With 128 a slice is a whole cache line per
// row (products that stream a large operand once read it at 5.9 instead of 3.6 TB/s in a
// stand-alone walk of the same pattern), eight rows per load instruction instead of sixteen,
// and four k-steps per slice instead of two.
template <typename T, int BM, int BN, int NS, int AMODE, int BMODE, int RB = DMA_ROW, int WGM = 2,
          int WGN = 2>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_dma_kernel(gemm_args_t a)
{
    using tr = traits_t<T>;
    constexpr int NW = WGM * WGN;  // wavefronts, WGM x WGN over the tile
    constexpr int MI = tr::MI;
    constexpr int VL = tr::VL;
    constexpr int BK = RB / int(sizeof(T));
    constexpr int CPRW = RB / 16;       // 16-byte chunks per row of a slice
    constexpr int ROWS_PI = 1024 / RB;  // rows per load instruction (operand along k)
    constexpr int STAGE = (BM + BN) * RB;
    constexpr int A_BYTES = BM * RB;
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int TM = WM / MI, TN = WN / MI;
    constexpr int STEPS = BK / (tr::KG * VL);
    // load instructions per thread per slice: one moves 1 KiB per wavefront
    constexpr int NLA = BM * RB / (NW * 1024), NLB = BN * RB / (NW * 1024);
    static_assert(NLA >= 1 && NLB >= 1 && (NW == 4 || NW == 8), "whole load instructions");
    // 32 x 32 matrix tiles with two lane groups along k (f16, f32) or 16 x 16 tiles with four
    // (f64: v_mfma_f64_16x16x4_f64); a lane group reads one 16-byte chunk per k-step
    static_assert(((MI == 32 && tr::KG == 2) || (MI == 16 && tr::KG == 4)) &&
                      (STEPS == 2 || STEPS == 4) && (RB == 64 || RB == 128),
                  "fragment layout");
    static_assert(BM % 64 == 0 && BN % 64 == 0, "");
    // An operand contiguous along m / n (mode 1) stays [k][m] / [k][n] in LDS: BK rows of
    // BM / BN elements
    constexpr int RAM = BM * int(sizeof(T));  // bytes of one k row of A
    constexpr int RPIA = 1024 / RAM;          // k rows per load instruction
    constexpr int RBN = BN * int(sizeof(T));
    constexpr int RPI = 1024 / RBN;
    static_assert(AMODE == 0 || (RAM <= 1024 && 1024 % RAM == 0), "");
    static_assert(BMODE == 0 || (RBN <= 1024 && 1024 % RBN == 0), "");

    extern __shared__ __attribute__((aligned(16))) char lds[];
    uint32_t const lds_base =
        uint32_t(uintptr_t((__attribute__((address_space(3))) char*)lds));

    int const tid = threadIdx.x;
    int const lane = tid & 63;
    int const wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int const wm = wave / WGN, wn = wave % WGN;

    // one XCD (one L2) works on a contiguous run of tiles, across batch entries: attention's
    // P.V, 16 tiles per head, moved 1.67 GiB out of the L2s for 1.06 GiB of operands while the
    // run stayed inside one batch entry
    uint32_t const n_tiles = a.tiles_m * a.tiles_n;
    uint32_t       tile = blockIdx.x;
    uint32_t       bz = blockIdx.y;
    xcd_renumber(a, n_tiles, tile, bz);
    constexpr uint32_t GROUP_M = 4;
    uint32_t const     in_group = GROUP_M * a.tiles_n;
    // all of this is uniform: a multiply-high and shifts stay on the scalar unit, while a
    // division is a long vector sequence that every workgroup would pay before its first load
    uint32_t const group = a.group_magic ? __umulhi(tile, a.group_magic) : tile / in_group;
    uint32_t const in_g = tile - group * in_group;
    uint32_t const first_m = group * GROUP_M;
    uint32_t const rows = (a.tiles_m - first_m) < GROUP_M ? (a.tiles_m - first_m) : GROUP_M;
    uint32_t       tm, tn;
    if (rows == GROUP_M) {
        tm = first_m + in_g % GROUP_M;
        tn = in_g / GROUP_M;
    } else {
        tm = first_m + in_g % rows;
        tn = in_g / rows;
    }

    int64_t boa, bob, boc;
    {
        group_offsets(a.gb, bz, boa, bob);
        if (a.gb.n == 1) {
            boc = int64_t(bz) * a.gb.sz[0];
        } else {
            boc = 0;
            uint32_t i = bz;
#pragma unroll
            for (int d = 0; d != MAXG; ++d) {
                uint32_t q = i / a.gb.size[d];
                boc += int64_t(i - q * a.gb.size[d]) * a.gb.sz[d];
                i = q;
            }
        }
    }
    // the bases go into scalar registers of the load instructions
    auto uniform = [](T const* p) {
        uint64_t const v = reinterpret_cast<uint64_t>(p);
        uint32_t const lo = __builtin_amdgcn_readfirstlane(uint32_t(v));
        uint32_t const hi = __builtin_amdgcn_readfirstlane(uint32_t(v >> 32));
        return reinterpret_cast<T const*>((uint64_t(hi) << 32) | lo);
    };
    T const* const A = uniform(static_cast<T const*>(a.A) + boa);
    T const* const B = uniform(static_cast<T const*>(a.B) + bob);

    // Load instruction i of this wavefront covers rows (NW i + wave) * 16 + lane / 4 of the
    // tile; the lane's LDS slot is chunk lane % 4 of that row and holds global chunk
    // (lane % 4) ^ bits 2..3 of the row = (lane % 4) ^ ((lane / 16) % 4).
    // 128-byte rows: rows (NW i + wave) * 8 + lane / 8, slot lane % 8, and the swizzle is bits
    // 1..3 of the row = (wave % 2) * 4 + lane / 16: sixteen consecutive rows of one k-chunk
    // (two rows per 64 banks) again cover all banks once.
    uint32_t const load_chunk =
        RB == 64 ? uint32_t((lane & 3) ^ ((lane >> 4) & 3))
                 : uint32_t((lane & 7) ^ (((lane >> 4) & 3) | ((wave & 1) << 2)));
    uint32_t       voa[NLA], vob[NLB];
    // [k][m] / [k][n] rows: the 16-byte chunks of a row are permuted so that the fragment
    // reads (which walk down k for a fixed m / n) spread over the banks; bits of the k row
    // select which 64-byte (2-byte elements: rows k..k+3 are read together) or 128-byte
    // (4-byte elements: rows k and k+4) segment a chunk lands in
    // (8-byte elements: a lane group reads rows k and k + 1, the four groups rows 0, 2, 4, 6
    // of a k-step: bit 1 of the row picks the half)
    auto kn_swizzle = [](uint32_t r) {
        return sizeof(T) == 2 ? (r & 3) << 2 : (sizeof(T) == 4 ? ((r >> 2) & 1) << 3 : ((r >> 1) & 1) << 3);
    };
#pragma unroll
    for (int i = 0; i != NLA; ++i) {
        int64_t x, y;
        if constexpr (AMODE == 0) {
            uint32_t r = tm * BM + uint32_t((NW * i + wave) * ROWS_PI + lane / CPRW);
            r = r < a.M ? r : a.M - 1;
            group_offsets(a.gm, r, x, y);
            voa[i] = uint32_t(x) * uint32_t(sizeof(T));
        } else {
            // this lane's slot: k row r of the slice, chunk c of that row
            uint32_t const r = uint32_t(NW * i + wave) * RPIA + uint32_t(lane * 16) / RAM;
            uint32_t const c = (uint32_t(lane * 16) % RAM) / 16;
            uint32_t       m = tm * BM + (c ^ kn_swizzle(r)) * VL;
            m = m < a.M ? m : a.M - VL;  // M is a multiple of VL on this path
            group_offsets(a.gm, m, x, y);
            voa[i] = (uint32_t(x) + r * uint32_t(a.gk.sx[0])) * uint32_t(sizeof(T));
        }
    }
#pragma unroll
    for (int i = 0; i != NLB; ++i) {
        int64_t x, y;
        if constexpr (BMODE == 0) {
            uint32_t r = tn * BN + uint32_t((NW * i + wave) * ROWS_PI + lane / CPRW);
            r = r < a.N ? r : a.N - 1;
            group_offsets(a.gn, r, x, y);
            vob[i] = uint32_t(x) * uint32_t(sizeof(T));
        } else {
            // this lane's slot: k row r of the slice, chunk c of that row
            uint32_t const r = uint32_t(NW * i + wave) * RPI + uint32_t(lane * 16) / RBN;
            uint32_t const c = (uint32_t(lane * 16) % RBN) / 16;
            uint32_t       n = tn * BN + (c ^ kn_swizzle(r)) * VL;
            n = n < a.N ? n : a.N - VL;  // N is a multiple of VL on this path
            group_offsets(a.gn, n, x, y);
            vob[i] = (uint32_t(x) + r * uint32_t(a.gk.sy[0])) * uint32_t(sizeof(T));
        }
    }
    // Byte offsets of the lane's 16-byte chunk within a row of A / of B, slice after slice:
    // next_k_offsets hands out those of the next slice in line (every slice's loads are
    // issued in order).  With several k modes the digits of the slice's first k element are
    // carried along and stepped by BK -- as long as the innermost mode holds whole slices, the
    // usual case (a head dimension of 64 or 128) -- instead of decomposing every lane's k by
    // division: those were some hundred vector instructions per slice in front of the
    // matrix instructions (out-projection adbe,cde->abc: 0.082 -> 0.070 ms).
    bool const k_walk = AMODE == 0 && BMODE == 0 && a.gk.n != 1 && a.gk.size[0] % BK == 0;
    uint32_t   k_next = 0;  // slice index (within this workgroup's share) handed out next
    uint32_t   k_dig[MAXG] = {0, 0, 0, 0};
    uint32_t   k_wa = 0, k_wb = 0;        // element offsets of the slice's first k element
    uint32_t   k_la = 0, k_lb = 0;        // the lane's own part, bytes
    auto seek_k = [&](uint32_t first_slice) {
        if (!k_walk) return;
        int64_t x, y;
        group_offsets(a.gk, first_slice * BK, x, y);
        k_wa = uint32_t(x);
        k_wb = uint32_t(y);
        uint32_t i = first_slice * BK;
#pragma unroll
        for (int d = 0; d != MAXG; ++d) {
            uint32_t const q = i / a.gk.size[d];
            k_dig[d] = i - q * a.gk.size[d];
            i = q;
        }
        k_la = load_chunk * VL * uint32_t(a.gk.sx[0]) * uint32_t(sizeof(T));
        k_lb = load_chunk * VL * uint32_t(a.gk.sy[0]) * uint32_t(sizeof(T));
    };
    auto next_k_offsets = [&](uint32_t first_slice, uint32_t& ka, uint32_t& kb) {
        uint32_t const kt = first_slice + k_next;
        ++k_next;
        uint32_t const k = kt * BK + load_chunk * VL;
        if constexpr (AMODE == 1 || BMODE == 1) {  // one k mode (checked by the launcher)
            ka = AMODE == 1 ? kt * BK * uint32_t(a.gk.sx[0]) * uint32_t(sizeof(T))
                            : k * uint32_t(sizeof(T));
            kb = BMODE == 1 ? kt * BK * uint32_t(a.gk.sy[0]) * uint32_t(sizeof(T))
                            : k * uint32_t(sizeof(T));
        } else if (a.gk.n == 1) {  // contiguous in both operands on this path
            ka = kb = k * uint32_t(sizeof(T));
        } else if (k_walk) {
            ka = k_wa * uint32_t(sizeof(T)) + k_la;
            kb = k_wb * uint32_t(sizeof(T)) + k_lb;
            // step to the next slice: all of this is uniform
            k_dig[0] += BK;
            k_wa += BK * uint32_t(a.gk.sx[0]);
            k_wb += BK * uint32_t(a.gk.sy[0]);
#pragma unroll
            for (int d = 0; d + 1 != MAXG; ++d) {
                if (k_dig[d] == a.gk.size[d]) {
                    k_dig[d] = 0;
                    k_dig[d + 1] += 1;
                    k_wa += uint32_t(a.gk.sx[d + 1]) - a.gk.size[d] * uint32_t(a.gk.sx[d]);
                    k_wb += uint32_t(a.gk.sy[d + 1]) - a.gk.size[d] * uint32_t(a.gk.sy[d]);
                }
            }
        } else {
            int64_t x, y;
            group_offsets(a.gk, k, x, y);
            ka = uint32_t(x) * uint32_t(sizeof(T));
            kb = uint32_t(y) * uint32_t(sizeof(T));
        }
    };
    // load q of slice kt: A rows for q < NLA, B rows after that
    auto issue = [&](uint32_t kt, int q, uint32_t ka, uint32_t kb) {
        uint32_t const st = kt % NS;
        if (q < NLA) {
            load_to_lds_16(A, voa[q] + ka,
                           lds_base + st * STAGE + uint32_t(NW * q + wave) * 1024);
        } else {
            load_to_lds_16(B, vob[q - NLA] + kb,
                           lds_base + st * STAGE + A_BYTES + uint32_t(NW * (q - NLA) + wave) * 1024);
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

    // Fragment of k-step s for MFMA tile row r0 + lane % MI: k-chunk KG s + lane / MI, found
    // in slot chunk ^ bits 2..3 (64-byte rows) or 1..3 (128-byte rows) of the row
    int const f_sw = RB == 64 ? (lane >> 2) & 3 : ((lane % MI) >> 1) & 7;
    int       f_off[STEPS];
#pragma unroll
    for (int s = 0; s != STEPS; ++s) {
        f_off[s] = (lane % MI) * RB + (((tr::KG * s + lane / MI) ^ f_sw) * 16);
    }
    int const fa_base = wm * WM * RB;
    int const fb_base = A_BYTES + wn * WN * RB;
    // [k][m] A / [k][n] B: byte offset of the lane's first element of MFMA tile i / j at
    // k-step 0.  ds_read_b64_tr_b16: within 16 lanes, lane i addresses 4 consecutive m (n) of
    // k row i / 4 (column group i % 4) and receives, for its own m (n), 4 consecutive k.
    int f_km[TM];
    if constexpr (AMODE == 1) {
#pragma unroll
        for (int i = 0; i != TM; ++i) {
            if constexpr (sizeof(T) == 2) {
                int const i16 = lane & 15, blk = lane >> 4;
                int const m0 = wm * WM + i * MI + (blk & 1) * 16 + 4 * (i16 & 3);
                int const k0 = (blk >> 1) * VL + (i16 >> 2);
                f_km[i] = k0 * RAM + ((m0 * 2) ^ int(kn_swizzle(uint32_t(k0)) * 16));
            } else {
                int const m0 = wm * WM + i * MI + lane % MI;
                int const k0 = (lane / MI) * VL;
                f_km[i] = k0 * RAM + ((m0 * int(sizeof(T))) ^ int(kn_swizzle(uint32_t(k0)) * 16));
            }
        }
    }
    int f_kn[TN];
    if constexpr (BMODE == 1) {
#pragma unroll
        for (int j = 0; j != TN; ++j) {
            if constexpr (sizeof(T) == 2) {
                // ds_read_b64_tr_b16: within 16 lanes, lane i addresses 4 consecutive n of k
                // row i / 4 (column group i % 4) and receives, for its own n, 4 consecutive k
                int const i16 = lane & 15, blk = lane >> 4;
                int const n0 = wn * WN + j * MI + (blk & 1) * 16 + 4 * (i16 & 3);
                int const k0 = (blk >> 1) * VL + (i16 >> 2);
                f_kn[j] = k0 * RBN + ((n0 * 2) ^ int(kn_swizzle(uint32_t(k0)) * 16));
            } else {
                int const n0 = wn * WN + j * MI + lane % MI;
                int const k0 = (lane / MI) * VL;
                f_kn[j] = k0 * RBN + ((n0 * int(sizeof(T))) ^ int(kn_swizzle(uint32_t(k0)) * 16));
            }
        }
    }

    chunk_t fa[2][TM], fb[2][TN];
    // a fragment of an operand kept [k][row] in LDS: transposing read (2-byte elements) or
    // one element per k row (4-byte elements); rows k..k+3 and k+4..k+7 share their low two
    // bits, rows k0..k0+3 of one lane share bit 2, hence their swizzle
    auto read_transposed = [&](char const* p, int row_bytes) {
        if constexpr (sizeof(T) == 2) {
            typedef short tr_t __attribute__((ext_vector_type(4)));
            typedef short tr8_t __attribute__((ext_vector_type(8)));
            tr_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) tr_t*)(p));
            tr_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) tr_t*)(p + 4 * row_bytes));
            tr8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            return __builtin_bit_cast(chunk_t, both);
        } else if constexpr (sizeof(T) == 4) {
            chunk_t v;
#pragma unroll
            for (int t = 0; t != VL; ++t) {
                v[t] = *reinterpret_cast<uint32_t const*>(p + t * row_bytes);
            }
            return v;
        } else {
            typedef uint32_t pair_t __attribute__((ext_vector_type(2)));
            pair_t const lo = *reinterpret_cast<pair_t const*>(p);
            pair_t const hi = *reinterpret_cast<pair_t const*>(p + row_bytes);
            return chunk_t{lo[0], lo[1], hi[0], hi[1]};
        }
    };
    auto read_a = [&](char const* stage, int s, int i) {
        if constexpr (AMODE == 0) {
            return *reinterpret_cast<chunk_t const*>(stage + fa_base + i * MI * RB + f_off[s]);
        } else {
            return read_transposed(stage + f_km[i] + s * tr::KG * VL * RAM, RAM);
        }
    };
    auto read_b = [&](char const* stage, int s, int j) {
        if constexpr (BMODE == 0) {
            return *reinterpret_cast<chunk_t const*>(stage + fb_base + j * MI * RB + f_off[s]);
        } else {
            return read_transposed(stage + A_BYTES + f_kn[j] + s * tr::KG * VL * RBN, RBN);
        }
    };
    // read order: what the first matrix instructions of a step need comes first
    auto read_frag = [&](char const* stage, int s, int q, chunk_t(&xa)[TM], chunk_t(&xb)[TN]) {
        if (q == 0) {
            xa[0] = read_a(stage, s, 0);
        } else if (q <= TN) {
            xb[q - 1] = read_b(stage, s, q - 1);
        } else {
            xa[q - TN] = read_a(stage, s, q - TN);
        }
    };
    constexpr int READS = TM + TN;
    constexpr int PAIRS = TM * TN;
    constexpr int LOADS = NLA + NLB;
    // side work per matrix instruction: step 0 spreads the reads over all of them, step 1
    // over all but the first (which is followed by the barrier)
    // A 16-byte chunk feeds tr::SUB matrix instructions (4 for 4-byte elements).  They go
    // round the accumulator tiles, so that consecutive instructions never depend on each
    // other, and each carries its share of the side work.
    constexpr int MMAS = PAIRS * tr::SUB;
    constexpr int R0 = (READS + MMAS - 1) / MMAS;
    constexpr int R1 = (READS + MMAS - 2) / (MMAS - 1);

    // k slices of this workgroup: all of them, or this split's share (the first K/BK mod
    // splits shares are one slice longer); every share has at least NS slices
    uint32_t k_begin = 0;
    uint32_t nk = a.K / BK;  // >= NS, no remainder (checked by the launcher)
    if (a.splits > 1) {
        uint32_t const q = nk / a.splits, r = nk % a.splits, z = blockIdx.z;
        k_begin = z * q + (z < r ? z : r);
        nk = q + (z < r ? 1 : 0);
    }

    // prologue: NS slices in flight, the first one landed
    seek_k(k_begin);
#pragma unroll
    for (int s = 0; s != NS; ++s) {
        uint32_t ka, kb;
        next_k_offsets(k_begin, ka, kb);
#pragma unroll
        for (int q = 0; q != LOADS; ++q) issue(uint32_t(s), q, ka, kb);
    }
    wait_loads_and_lds<LOADS*(NS - 1)>();
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int q = 0; q != READS; ++q) read_frag(lds, 0, q, fa[0], fb[0]);

    // One slice.  YOUNGER = slices issued after slice kt+1 that may still be in flight when
    // slice kt+1 is needed (-1: there is no slice kt+1); ISSUE: refill this stage with slice
    // kt+NS.  The loads of a slice are not issued in one burst: its first 1/STEPS goes out
    // after the barrier in the last k-step of slice kt, the other parts during the first
    // STEPS-1 k-steps of slice kt+1 (`prev`: slice kt-1+NS exists and this is not the first
    // slice, whose predecessor's loads the prologue issued).  Eight wavefronts that each push
    // all their loads of a slice right after the barrier fill the queue of the texture
    // addresser, and a wavefront that cannot get a load accepted cannot issue matrix
    // instructions either (8192^3, 256x256 tile: 72 % of the cycles had a matrix instruction
    // in flight against 85 % without the loads and 87 % in a run whose loads all hit one line).
    // (With two stages a load has one slice's time to land, and every part issued later
    // cuts into it: 8192^3 on eight wavefronts runs 3 % slower in four parts than in one and
    // 2 % faster in two; the four-wavefront kernels on two stages keep the single burst.)
    constexpr bool SPREAD = true;
    constexpr int  PARTS = NS >= 3 ? STEPS : (NW == 8 ? 2 : 1);
    auto part_lo = [](int p) { return (p < PARTS ? p : PARTS) * LOADS / PARTS; };
    uint32_t ka = 0, kb = 0;  // k offsets of the slice that is being issued
    auto slice = [&](uint32_t kt, auto younger_tag, auto issue_tag, bool prev) {
        constexpr int  YOUNGER = decltype(younger_tag)::value;
        constexpr bool ISSUE = decltype(issue_tag)::value;
        char const*    cur = lds + (kt % NS) * STAGE;
        char const*    nxt = lds + ((kt + 1) % NS) * STAGE;
        if (!SPREAD) prev = false;
        // ka, kb: still those of slice kt-1+NS, whose first part the slice before this one issued
#pragma unroll
        for (int s = 0; s != STEPS - 1; ++s) {
            int const lo = part_lo(s + 1), n = part_lo(s + 2) - part_lo(s + 1);
#pragma unroll
            for (int q = 0; q != MMAS; ++q) {
                int const p = q % PAIRS;
                tr::mma_sub(acc[p / TN][p % TN], fb[s & 1][p % TN], fa[s & 1][p / TN], q / PAIRS);
#pragma unroll
                for (int r = q * R0; r != (q + 1) * R0; ++r) {
                    if (r < READS) read_frag(cur, s + 1, r, fa[(s + 1) & 1], fb[(s + 1) & 1]);
                }
                if (prev) {
#pragma unroll
                    for (int r = lo + q * n / MMAS; r != lo + (q + 1) * n / MMAS; ++r) {
                        issue(kt - 1 + NS, r, ka, kb);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (ISSUE) next_k_offsets(k_begin, ka, kb);  // slice kt+NS
        constexpr int N0 = LOADS / PARTS;  // part 0
#pragma unroll
        for (int q = 0; q != MMAS; ++q) {
            int const p = q % PAIRS;
            tr::mma_sub(acc[p / TN][p % TN], fb[1][p % TN], fa[1][p / TN], q / PAIRS);
            if (YOUNGER >= 0) {
                if (q == 0) {
                    // this wave's part of slice kt+1 has landed and its reads of this stage
                    // are complete; after the barrier that holds for the whole workgroup
                    wait_loads_and_lds<(YOUNGER < 0 ? 0 : YOUNGER) * LOADS>();
                    __builtin_amdgcn_s_barrier();
                } else {
#pragma unroll
                    for (int r = (q - 1) * R1; r != q * R1; ++r) {
                        if (r < READS) read_frag(nxt, 0, r, fa[0], fb[0]);
                    }
#pragma unroll
                    for (int r = (q - 1) * N0 / (MMAS - 1); r != q * N0 / (MMAS - 1); ++r) {
                        if (ISSUE) issue(kt + NS, r, ka, kb);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    {
        using std::integral_constant;
        uint32_t kt = 0;
        for (; kt + NS < nk; ++kt) {
            slice(kt, integral_constant<int, NS - 2>{}, std::true_type{}, kt != 0);
        }
        // the last NS slices refill nothing and have ever fewer loads behind them
        auto tail = [&](auto const& self, auto j_tag) {
            constexpr int J = decltype(j_tag)::value;
            slice(kt, integral_constant<int, NS - 2 - J>{}, std::false_type{}, J == 0 && kt != 0);
            ++kt;
            if constexpr (J + 1 < NS) self(self, integral_constant<int, J + 1>{});
        };
        tail(tail, integral_constant<int, 0>{});
    }

    // Epilogue: each wave turns MI rows of its tile through a private LDS strip so that the
    // global stores are 16 bytes per lane and whole row segments per wavefront.
    if (a.splits > 1) {
        // partial tile, fp32: every lane holds four consecutive n of one m per register quad
        float* const part = a.ws + (size_t(blockIdx.z) * a.batch + bz) * a.M * size_t(a.N);
#pragma unroll
        for (int i = 0; i != TM; ++i) {
            uint32_t const m = tm * BM + wm * WM + i * MI + uint32_t(lane % MI);
#pragma unroll
            for (int j = 0; j != TN; ++j) {
#pragma unroll
                for (int e0 = 0; e0 < tr::NACC; e0 += 4) {
                    uint32_t const n = tn * BN + wn * WN + j * MI + uint32_t(tr::acc_row(e0, lane));
                    if (m < a.M && n < a.N) {  // N is a multiple of 4 on this path
                        float4_t q = {float(acc[i][j][e0]), float(acc[i][j][e0 + 1]),
                                      float(acc[i][j][e0 + 2]), float(acc[i][j][e0 + 3])};
                        *reinterpret_cast<float4_t*>(part + size_t(m) * a.N + n) = q;
                    }
                }
            }
        }
        return;
    }
    T* const C = static_cast<T*>(a.C) + boc;
    typename tr::acc_elem const alpha = typename tr::acc_elem(a.alpha);
    constexpr int STRIP_PITCH = WN * int(sizeof(T)) + 16;
    constexpr int CPR = WN * int(sizeof(T)) / 16;
    wait_loads_and_lds<0>();
    __builtin_amdgcn_s_barrier();
    char* const strip = lds + wave * (MI * STRIP_PITCH);
    typedef T quad_t __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int i = 0; i != TM; ++i) {
#pragma unroll
        for (int j = 0; j != TN; ++j) {
#pragma unroll
            for (int e0 = 0; e0 < tr::NACC; e0 += 4) {
                if constexpr (tr::QUAD) {
                    quad_t q;
#pragma unroll
                    for (int t = 0; t != 4; ++t) q[t] = T(acc[i][j][e0 + t] * alpha);
                    int n = j * MI + tr::acc_row(e0, lane);
                    *reinterpret_cast<quad_t*>(strip + (lane % MI) * STRIP_PITCH +
                                               n * int(sizeof(T))) = q;
                } else {
#pragma unroll
                    for (int t = 0; t != 4; ++t) {
                        int n = j * MI + tr::acc_row(e0 + t, lane);
                        *reinterpret_cast<T*>(strip + (lane % MI) * STRIP_PITCH +
                                              n * int(sizeof(T))) = T(acc[i][j][e0 + t] * alpha);
                    }
                }
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
                chunk_t* const dst = reinterpret_cast<chunk_t*>(C + mo_c + no_c);
                if (a.c_stream) {
                    store_16_streaming(dst, v);
                } else {
                    *dst = v;
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

// Whether the direct-to-LDS kernel can run this problem (both operands 16-byte vectors along
// k, wide epilogue, K a whole number of at least four slices, operand offsets within 32 bits).
template <typename T>
bool gemm_dma_eligible(gemm_args_t const& a)
{
    constexpr uint32_t BK = DMA_ROW / sizeof(T);
    // an operand contiguous along m / n needs a single k mode (its k rows are addressed by
    // one stride)
    bool const a_ok = a.a_mode == 0 || (a.a_mode == 1 && a.gk.n == 1);
    bool const b_ok = a.b_mode == 0 || (a.b_mode == 1 && a.gk.n == 1);
    return a_ok && b_ok && a.c_mode == 3 && a.K % BK == 0 && a.K / BK >= 4 &&
           a.offsets_fit_32 != 0;
}

// The same with slices of 128 bytes per row: K a whole number of such slices, and every
// split-K share (the kernel cuts K into shares of its own slices) at least `stages` of them.
template <typename T>
bool gemm_dma_wide_eligible(gemm_args_t const& a, uint32_t stages)
{
    constexpr uint32_t BK = 128 / sizeof(T);
    uint32_t const     splits = a.splits > 1 ? a.splits : 1;
    return gemm_dma_eligible<T>(a) && a.K % BK == 0 && a.K / BK / splits >= stages;
}

template <typename T, int BM, int BN, int NS, int AMODE, int BMODE, int RB = DMA_ROW, int WGM = 2,
          int WGN = 2>
void launch_gemm_dma_kernel_mode(gemm_args_t const& a, hipStream_t stream)
{
    static_assert(NS >= 2 && NS <= 4, "eligibility guarantees four slices");
    constexpr int lds = NS * (BM + BN) * RB;
    static bool const raised = [] {
        (void)hipFuncSetAttribute(
            reinterpret_cast<const void*>(
                &gemm_dma_kernel<T, BM, BN, NS, AMODE, BMODE, RB, WGM, WGN>),
            hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        return true;
    }();
    (void)raised;
    dim3 grid(a.tiles_m * a.tiles_n, a.batch, a.splits > 1 ? a.splits : 1);
    hipLaunchKernelGGL((gemm_dma_kernel<T, BM, BN, NS, AMODE, BMODE, RB, WGM, WGN>), grid,
                       dim3(64 * WGM * WGN), lds, stream, a);
}

// Second pass of a split-K contraction: C = sum over the splits' partial tiles, in split
// order (deterministic), converted to T.  One thread per four consecutive n.
template <typename T>
__global__ __launch_bounds__(256) void gemm_fold_kernel(gemm_args_t a)
{
    uint64_t const quads_per_row = a.N / 4;
    uint64_t const total = uint64_t(a.batch) * a.M * quads_per_row;
    uint64_t const id = uint64_t(blockIdx.x) * 256 + threadIdx.x;
    if (id >= total) return;
    uint32_t const n = uint32_t(id % quads_per_row) * 4;
    uint64_t const rest = id / quads_per_row;
    uint32_t const m = uint32_t(rest % a.M);
    uint32_t const bz = uint32_t(rest / a.M);
    size_t const   plane = size_t(a.batch) * a.M * size_t(a.N);
    float const*   p = a.ws + (size_t(bz) * a.M + m) * a.N + n;
    float4_t       sum = {0, 0, 0, 0};
    for (uint32_t z = 0; z != a.splits; ++z) {
        sum += *reinterpret_cast<float4_t const*>(p + size_t(z) * plane);
    }
    int64_t boc = 0;
    {
        uint32_t i = bz;
#pragma unroll
        for (int d = 0; d != MAXG; ++d) {
            uint32_t q = i / a.gb.size[d];
            boc += int64_t(i - q * a.gb.size[d]) * a.gb.sz[d];
            i = q;
        }
    }
    int64_t mo_a, mo_c, no_b, no_c;
    group_offsets(a.gm, m, mo_a, mo_c);
    group_offsets(a.gn, n, no_b, no_c);
    typedef T quad_t __attribute__((ext_vector_type(4)));
    float const alpha = float(a.alpha);
    quad_t out = {T(sum[0] * alpha), T(sum[1] * alpha), T(sum[2] * alpha), T(sum[3] * alpha)};
    *reinterpret_cast<quad_t*>(static_cast<T*>(a.C) + boc + mo_c + no_c) = out;
}

template <typename T>
void launch_gemm_fold(gemm_args_t const& a, hipStream_t stream)
{
    uint64_t const total = uint64_t(a.batch) * a.M * (a.N / 4);
    hipLaunchKernelGGL((gemm_fold_kernel<T>), dim3(unsigned((total + 255) / 256)), dim3(256), 0,
                       stream, a);
}

template <typename T, int BM, int BN, int NS>
void launch_gemm_dma_kernel(gemm_args_t const& a, hipStream_t stream)
{
    if (a.a_mode == 0) {
        if (a.b_mode == 0) {
            launch_gemm_dma_kernel_mode<T, BM, BN, NS, 0, 0>(a, stream);
        } else {
            launch_gemm_dma_kernel_mode<T, BM, BN, NS, 0, 1>(a, stream);
        }
    } else {
        if (a.b_mode == 0) {
            launch_gemm_dma_kernel_mode<T, BM, BN, NS, 1, 0>(a, stream);
        } else {
            launch_gemm_dma_kernel_mode<T, BM, BN, NS, 1, 1>(a, stream);
        }
    }
    if (a.splits > 1) launch_gemm_fold<T>(a, stream);
}

}  // namespace gemm
}  // namespace es
