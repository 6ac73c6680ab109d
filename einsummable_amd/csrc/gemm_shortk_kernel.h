// fp16 contractions with a reduction of exactly 128 elements (attention scores: K is the head
// dimension) and many output tiles.  Such a product does 256 flop per output byte pair and is
// bound by writing C; a tile has only eight matrix-instruction steps of work, so a kernel
// that starts a workgroup per tile spends its time in set-up, in waiting for the first
// operands and in an epilogue that nothing overlaps.  Here a workgroup keeps its 128 rows of
// A in registers for its whole life and walks along n:
//
//   * waves 4 and 5 only load: 128 x 128 tiles of B go from global memory straight into a
//     ring of LDS buffers (global_load_lds_dwordx4; 256-byte rows whose sixteen 16-byte
//     chunks are XOR-swizzled with the row number so that fragment reads are free of bank
//     conflicts), each wave half a tile, one tile ahead of the multiplication; they wait
//     until the next tile has landed and join the workgroup barrier;
//   * waves 0..3 (2 x 2, 64 x 64 each) multiply the current B buffer with their A
//     fragments and leave the tile, converted to fp16, in one of two LDS staging tiles;
//   * waves 6 and 7 only store: they read the staging tile of the previous step as whole
//     256-byte row segments and write them to C.  A store instruction stalls its wave until
//     the memory pipeline takes it; on these waves that costs nothing, while the same
//     stall on a multiplying wave (measured: the time to write C simply added to the time
//     of everything else) keeps the matrix cores and the loads idle.
//
// One workgroup barrier per tile orders the three roles: a B buffer is refilled after
// everyone has read it, a staging tile is rewritten after it has been read out.
#pragma once
#include "gemm_dma_kernel.h"

#include <algorithm>
#include <cstdlib>

namespace es
{
namespace gemm
{

constexpr int SK_K = 128;                         // elements along k
constexpr int SK_RB = SK_K * 2;                   // bytes of one operand row
constexpr int SK_BM = 128, SK_BN = 128;           // tile
constexpr int SK_BUF = SK_BN * SK_RB;             // one B buffer
constexpr int SK_NBUF = 2;                        // ring of B buffers
constexpr int SK_OUT_PITCH = SK_BN * 2 + 16;      // staging row: 128 outputs + pad
constexpr int SK_OUT = SK_BM * SK_OUT_PITCH;      // one staging tile
constexpr int SK_LDS = SK_NBUF * SK_BUF + 2 * SK_OUT + 512;  // + scratch of the prefetches
constexpr int SK_PF_DIST = 4;                     // tiles the L2 prefetch runs ahead
constexpr int SK_PF_LOADS = 2;                    // 128-byte lines per row of B
constexpr int SK_THREADS = 512;                   // 4 multiplying, 2 loading, 2 storing waves

__global__ __launch_bounds__(SK_THREADS) void gemm_shortk_kernel(gemm_args_t a,
                                                                 uint32_t tiles_per_block,
                                                                 uint32_t chunks_n)
{

    using T = _Float16;
    using tr = traits_t<T>;
    extern __shared__ __attribute__((aligned(16))) char lds[];
    uint32_t const lds_base = uint32_t(uintptr_t((__attribute__((address_space(3))) char*)lds));

    int const tid = threadIdx.x;
    int const lane = tid & 63;
    int const wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // consecutive logical workgroups (same batch entry, neighbouring rows of tiles: they
    // share B) run on one XCD, i.e. behind one L2
    uint32_t const per_batch = a.tiles_m * chunks_n;
    uint32_t       id = blockIdx.x;
    {
        uint32_t const per_xcd = gridDim.x / 8;
        if (id < per_xcd * 8) id = (id % 8) * per_xcd + id / 8;
    }
    uint32_t const bz = id / per_batch;
    uint32_t const rem = id - bz * per_batch;
    uint32_t const chunk = rem / a.tiles_m;
    uint32_t const tm = rem - chunk * a.tiles_m;
    uint32_t const t0 = chunk * tiles_per_block;
    uint32_t const t1 = t0 + tiles_per_block < a.tiles_n ? t0 + tiles_per_block : a.tiles_n;

    int64_t boa, bob, boc;
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
    uint32_t const lda = uint32_t(a.gm.sx[0]), ldb = uint32_t(a.gn.sx[0]);
    uint32_t const ldc = uint32_t(a.gm.sy[0]);

    if (wave == 4 || wave == 5) {
        // ---- the loading waves.  Load instruction q of a tile covers rows 4 q + lane / 16
        // (wave 4: q < 16, wave 5: the rest); the lane's LDS slot (lane % 16) receives
        // global chunk slot ^ (row % 16).
        T const* const B = static_cast<T const*>(a.B) + bob;
        uint32_t const lr = uint32_t(lane) >> 4, slot = uint32_t(lane) & 15;
        int const      half = wave - 4;
        constexpr int  PER_WAVE = SK_BN / 4 / 2;  // load instructions per tile per wave
        auto tile_loads = [&](uint32_t tn) {
            uint32_t const buf = (tn - t0) % SK_NBUF;
            static_assert(SK_NBUF == 2, "the waits below assume one tile of lookahead");
            uint32_t const n0 = tn * SK_BN;
            uint32_t const last = a.N - 1 - n0;  // rows past the end re-read the last one
            // the base goes into a scalar register pair of the load instructions (the
            // builtin returns a signed int: widen each half as unsigned)
            uint64_t const p = reinterpret_cast<uint64_t>(B + int64_t(n0) * ldb);
            uint32_t const lo = uint32_t(__builtin_amdgcn_readfirstlane(uint32_t(p)));
            uint32_t const hi = uint32_t(__builtin_amdgcn_readfirstlane(uint32_t(p >> 32)));
            T const* const base = reinterpret_cast<T const*>((uint64_t(hi) << 32) | lo);
#pragma unroll
            for (int q0 = 0; q0 != PER_WAVE; ++q0) {
                uint32_t const q = uint32_t(half * PER_WAVE + q0);
                uint32_t const row = 4 * q + lr;
                uint32_t const src = row < last ? row : last;
                uint32_t const voff = src * ldb * 2 + ((slot ^ (row & 15)) << 4);
                load_to_lds_16(base, voff, lds_base + buf * SK_BUF + q * 1024);
            }
        };
        // Brings tile `tn` into the L2 only (one dword per 128-byte line into a scratch
        // corner of LDS that nobody reads).  The tile needed next must not wait for HBM: with
        // C being written at full speed a read that misses the L2 takes microseconds, and
        // the lookahead of the buffer ring alone is one tile.
        auto prefetch = [&](T const* Bx, uint32_t tn) {
            uint32_t const n0 = tn * SK_BN;
            uint32_t const last = a.N - 1 - n0;
            uint64_t const p = reinterpret_cast<uint64_t>(Bx + int64_t(n0) * ldb);
            uint32_t const lo = uint32_t(__builtin_amdgcn_readfirstlane(uint32_t(p)));
            uint32_t const hi = uint32_t(__builtin_amdgcn_readfirstlane(uint32_t(p >> 32)));
            T const* const base = reinterpret_cast<T const*>((uint64_t(hi) << 32) | lo);
            uint32_t const row = uint32_t(half) * 64 + uint32_t(lane);
            uint32_t const src = row < last ? row : last;
#pragma unroll
            for (int u = 0; u != SK_PF_LOADS; ++u) {
                load_to_lds_4(base, src * ldb * 2 + uint32_t(u) * 128,
                              lds_base + SK_NBUF * SK_BUF + 2 * SK_OUT + uint32_t(half) * 256);
            }
        };
        tile_loads(t0);
        uint32_t ahead = 0;  // prefetch instructions younger than the tile loads
        for (uint32_t p = 1; p <= SK_PF_DIST && t0 + p < t1; ++p) {
            prefetch(B, t0 + p);
            ahead += SK_PF_LOADS;
        }
        // The workgroup that will follow this one on the compute unit (the XCD's 32 units take
        // consecutive logical workgroups in turn): its rows of A and its first tile of B.
        // Its own first loads then hit the L2 instead of waiting for HBM.
        {
            uint32_t const per_xcd = gridDim.x / 8;
            uint32_t const next = id + 32;
            if (blockIdx.x < per_xcd * 8 && blockIdx.x / 8 + 32 < per_xcd) {
                uint32_t const nbz = next / per_batch;
                uint32_t const nrem = next - nbz * per_batch;
                uint32_t const nchunk = nrem / a.tiles_m;
                uint32_t const ntm = nrem - nchunk * a.tiles_m;
                int64_t        nboa, nbob;
                group_offsets(a.gb, nbz, nboa, nbob);
                // rows of A: 128 rows of 256 bytes, this wave's half
                {
                    T const* const An = static_cast<T const*>(a.A) + nboa;
                    uint32_t const m_first = ntm * SK_BM;
                    uint32_t const last = a.M - 1 - m_first;
                    uint64_t const p = reinterpret_cast<uint64_t>(An + int64_t(m_first) * lda);
                    uint32_t const lo = uint32_t(__builtin_amdgcn_readfirstlane(uint32_t(p)));
                    uint32_t const hi = uint32_t(__builtin_amdgcn_readfirstlane(uint32_t(p >> 32)));
                    T const* const base = reinterpret_cast<T const*>((uint64_t(hi) << 32) | lo);
                    uint32_t const row = uint32_t(half) * 64 + uint32_t(lane);
                    uint32_t const src = row < last ? row : last;
#pragma unroll
                    for (int u = 0; u != SK_PF_LOADS; ++u) {
                        load_to_lds_4(base, src * lda * 2 + uint32_t(u) * 128,
                                      lds_base + SK_NBUF * SK_BUF + 2 * SK_OUT + uint32_t(half) * 256);
                    }
                }
                prefetch(static_cast<T const*>(a.B) + nbob, nchunk * tiles_per_block);
                ahead += 2 * SK_PF_LOADS;
            }
        }
        // the tile has landed; the prefetches behind it may still be in flight
        switch (ahead / SK_PF_LOADS) {
            case 0: wait_loads_and_lds<0>(); break;
            case 1: wait_loads_and_lds<1 * SK_PF_LOADS>(); break;
            case 2: wait_loads_and_lds<2 * SK_PF_LOADS>(); break;
            case 3: wait_loads_and_lds<3 * SK_PF_LOADS>(); break;
            case 4: wait_loads_and_lds<4 * SK_PF_LOADS>(); break;
            case 5: wait_loads_and_lds<5 * SK_PF_LOADS>(); break;
            default: wait_loads_and_lds<6 * SK_PF_LOADS>(); break;
        }
        __builtin_amdgcn_s_barrier();
        for (uint32_t t = t0; t != t1; ++t) {
            // the buffer of tile t + 1 is the one tile t - 1 was read from
            if (t + 1 < t1) tile_loads(t + 1);
            bool const pf = t + 1 + SK_PF_DIST < t1;
            if (pf) prefetch(B, t + 1 + SK_PF_DIST);
            if (t + 1 < t1) {
                if (pf) {
                    wait_loads_and_lds<SK_PF_LOADS>();
                } else {
                    wait_loads_and_lds<0>();
                }
            }
            __builtin_amdgcn_s_barrier();
        }
        return;
    }

    T* const C = static_cast<T*>(a.C) + boc;
    if (wave >= 6) {
        // ---- the storing waves: rows 64 (wave - 6) .. + 63 of every tile; instruction c
        // covers rows 4 c + lane / 16 with 16 lanes per 256-byte row segment
        int const      half = wave - 6;
        uint32_t const lr = uint32_t(lane) >> 4, lch = uint32_t(lane) & 15;
        uint32_t const mrow = tm * SK_BM + uint32_t(half) * 64;  // first row of this wave
        uint32_t const lane_off = (lr * ldc + lch * 8) * 2;
        int const      lds_off = int(uint32_t(half) * 64 + lr) * SK_OUT_PITCH + int(lch) * 16;
        constexpr int  NST = 16;
        __builtin_amdgcn_s_barrier();
        for (uint32_t t = t0; t != t1; ++t) {
            __builtin_amdgcn_s_barrier();  // tile t is staged
            char const* const out = lds + SK_NBUF * SK_BUF + ((t - t0) & 1) * SK_OUT + lds_off;
            uint32_t const    n0 = t * SK_BN;
            chunk_t           v[NST];
#pragma unroll
            for (int c = 0; c != NST; ++c) {
                v[c] = *reinterpret_cast<chunk_t const*>(out + c * 4 * SK_OUT_PITCH);
            }
            char* const corner = reinterpret_cast<char*>(C + int64_t(mrow) * ldc + n0);
            if (mrow + 64 <= a.M && n0 + SK_BN <= a.N) {  // uniform: no lane masking
#pragma unroll
                for (int c = 0; c != NST; ++c) {
                    chunk_t* const dst = reinterpret_cast<chunk_t*>(
                        corner + uint64_t(uint32_t(c * 4) * ldc) * 2 + lane_off);
                    if (a.c_stream) {
                        store_16_streaming(dst, v[c]);
                    } else {
                        *dst = v[c];
                    }
                }
            } else {
#pragma unroll
                for (int c = 0; c != NST; ++c) {
                    if (mrow + uint32_t(c * 4) + lr < a.M && n0 + lch * 8 < a.N) {
                        chunk_t* const dst = reinterpret_cast<chunk_t*>(
                            corner + uint64_t(uint32_t(c * 4) * ldc) * 2 + lane_off);
                        *dst = v[c];
                    }
                }
            }
        }
        return;
    }

    // ---- the multiplying waves
    int const wm = wave >> 1, wn = wave & 1;
    uint32_t const m0 = tm * SK_BM + uint32_t(wm) * 64;
    // A fragments: tile row i, k-step s: row lane % 32, k chunk 2 s + lane / 32
    chunk_t fa[2][8];
    float const alpha = float(a.alpha);
    {
        T const* const A = static_cast<T const*>(a.A) + boa;
#pragma unroll
        for (int i = 0; i != 2; ++i) {
            uint32_t r = m0 + uint32_t(i * 32 + lane % 32);
            r = r < a.M ? r : a.M - 1;
            T const* const row = A + int64_t(r) * lda + (lane / 32) * 8;
#pragma unroll
            for (int s = 0; s != 8; ++s) {
                fa[i][s] = *reinterpret_cast<chunk_t const*>(row + s * 16);
            }
        }
    }
    // B fragments: tile row j * 32 + lane % 32 of this wave's half, chunk 2 s + lane / 32 in
    // slot chunk ^ (row % 16); row % 16 is lane % 16 for every j
    int fb_row[2];
#pragma unroll
    for (int j = 0; j != 2; ++j) fb_row[j] = (wn * 64 + j * 32 + lane % 32) * SK_RB;
    int fb_slot[8];
#pragma unroll
    for (int s = 0; s != 8; ++s) fb_slot[s] = ((2 * s + lane / 32) ^ (lane & 15)) << 4;

    typedef T quad_t __attribute__((ext_vector_type(4)));

    __builtin_amdgcn_s_barrier();
    for (uint32_t t = t0; t != t1; ++t) {
        char const* const buf = lds + ((t - t0) % SK_NBUF) * SK_BUF;
        tr::acc_t acc[2][2];
#pragma unroll
        for (int i = 0; i != 2; ++i) {
#pragma unroll
            for (int j = 0; j != 2; ++j) {
#pragma unroll
                for (int e = 0; e != tr::NACC; ++e) acc[i][j][e] = 0;
            }
        }
        chunk_t fb[2][2];
#pragma unroll
        for (int j = 0; j != 2; ++j) {
            fb[0][j] = *reinterpret_cast<chunk_t const*>(buf + fb_row[j] + fb_slot[0]);
        }
#pragma unroll
        for (int s = 0; s != 8; ++s) {
            if (s + 1 != 8) {
#pragma unroll
                for (int j = 0; j != 2; ++j) {
                    fb[(s + 1) & 1][j] =
                        *reinterpret_cast<chunk_t const*>(buf + fb_row[j] + fb_slot[s + 1]);
                }
            }
#pragma unroll
            for (int i = 0; i != 2; ++i) {
#pragma unroll
                for (int j = 0; j != 2; ++j) tr::mma(acc[i][j], fb[s & 1][j], fa[i][s]);
            }
        }
        // every lane holds, per register quad, four consecutive n of row lane % 32
        char* const out = lds + SK_NBUF * SK_BUF + ((t - t0) & 1) * SK_OUT;
#pragma unroll
        for (int i = 0; i != 2; ++i) {
#pragma unroll
            for (int j = 0; j != 2; ++j) {
#pragma unroll
                for (int e0 = 0; e0 < tr::NACC; e0 += 4) {
                    quad_t q;
#pragma unroll
                    for (int u = 0; u != 4; ++u) q[u] = T(acc[i][j][e0 + u] * alpha);
                    int const m = wm * 64 + i * 32 + lane % 32;
                    int const n = wn * 64 + j * 32 + tr::acc_row(e0, lane);
                    *reinterpret_cast<quad_t*>(out + m * SK_OUT_PITCH + n * 2) = q;
                }
            }
        }
        wait_loads_and_lds<0>();  // the staged tile is complete before the barrier says so
        __builtin_amdgcn_s_barrier();
    }
}

// Tiles along n that one workgroup walks, or 0 when the kernel that takes a workgroup per
// tile is the better choice.  Measured with cold caches on b x s x s x 128 products, time of
// the per-tile kernel / time of this one, walks of 16 tiles: 1.09-1.23 from 1024 workgroups
// on (128 x 2048, 64 x 2048, 32 x 4096, 4 x 8192), 1.02 for 128 x 1024; below that, and for
// rows of four tiles, 0.86-0.97 (8 .. 32 x 2048, 8 x 4096, 256 x 512).
inline uint32_t shortk_walk(gemm_args_t const& a)
{
    uint64_t const tiles_m = (a.M + SK_BM - 1) / SK_BM, tiles_n = (a.N + SK_BN - 1) / SK_BN;
    if (tiles_n < 8 || tiles_m * tiles_n * a.batch >= (1ull << 31)) return 0;
    static uint64_t const min_walks = [] {
        const char* env = std::getenv("ES_KM_GEMM_RESIDENT_MIN");  // tuning and tests
        return uint64_t(env ? std::max(1, std::atoi(env)) : 1024);
    }();
    uint64_t const walks = tiles_m * a.batch * ((tiles_n + 15) / 16);
    return walks >= min_walks ? 16 : 0;
}

// Both operands contiguous along a single k mode of exactly 128 elements, single m and n
// modes, C contiguous along n, strides small enough for 32-bit in-tile offsets, and enough
// rows of tiles for several workgroups per compute unit.
bool gemm_shortk_eligible(gemm_args_t const& a)
{
    if (!a.lin || a.K != SK_K || a.a_mode != 0 || a.b_mode != 0 || a.c_mode != 3) return false;
    if (a.splits > 1 || a.N % 8 != 0 || a.gm.sy[0] % 8 != 0) return false;
    if (a.gk.sx[0] != 1 || a.gk.sy[0] != 1) return false;
    if (a.gm.sx[0] <= 0 || a.gn.sx[0] <= 0) return false;
    if (uint64_t(a.gm.sx[0]) * 256 * 2 >= (1ull << 31)) return false;
    if (uint64_t(a.gn.sx[0]) * 256 * 2 >= (1ull << 31)) return false;
    return shortk_walk(a) != 0;
}

void launch_gemm_shortk(gemm_args_t const& a0, hipStream_t stream)
{
    gemm_args_t a = with_tile(a0, SK_BM, SK_BN);
    uint32_t const walk = shortk_walk(a);
    uint32_t const tpb = a.tiles_n < walk ? a.tiles_n : walk;
    uint32_t const chunks = (a.tiles_n + tpb - 1) / tpb;
    static bool const raised = [] {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_shortk_kernel),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, SK_LDS);
        return true;
    }();
    (void)raised;
    dim3 grid(a.tiles_m * chunks * a.batch);
    hipLaunchKernelGGL(gemm_shortk_kernel, grid, dim3(SK_THREADS), SK_LDS, stream, a, tpb, chunks);
}

}  // namespace gemm
}  // namespace es
