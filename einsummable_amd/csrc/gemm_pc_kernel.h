// fp16 GEMM on 128 x 256 (256 x 128) tiles with wave roles: four wavefronts multiply, four
// only load, one of each on every SIMD.
//
// A 128 x 256 x 64 slice is 48 KiB of operands for 1024 cycles of matrix instructions, and
// the load path of a compute unit takes 64 bytes per cycle: it is busy three quarters of the
// time.  A wave that issues a load while that path is full stands there, and matrix
// instructions behind the load wait with it (the persistent four-wave kernel on this tile
// takes 1480 cycles per slice against 1024 of matrix work).  Here the waves that multiply
// never issue a load: their loop is matrix instructions, LDS reads and one barrier per slice.
// The loading waves stand at the load path instead, three slices ahead, and also do the
// part of the epilogue that waits for memory: the multiplying waves convert 32 rows of their
// accumulators, leave them in an LDS strip and convert the next 32 rows while the loading
// wave of their SIMD reads the strip and stores whole row segments.  128 accumulators per
// wave leave room for two waves per SIMD (256 registers each).
//
// Barriers: every one is executed by all eight waves.  Per slice g one barrier says both
// "the multiplying waves have read all of slice g" (its stage may be overwritten) and "slice
// g + 1 has landed".  Per tile 2 (BM / 64) - 1 more hand the strips to and fro.  Both roles count
// them from the same uniform numbers.
#pragma once
#include "gemm_w4_kernel.h"

#include <cstddef>

namespace es
{
namespace gemm
{
namespace pc
{
using namespace w4;

// The offsets of a grouped launch, read through the kernel-argument pointer (the arguments
// are the kernel's first parameter): a run-time index into the by-value struct would have the
// compiler copy the whole block into private memory first.
__device__ __forceinline__ int64_t const __attribute__((address_space(4))) * group_table()
{
    typedef char const __attribute__((address_space(4))) const_byte_t;
    typedef int64_t const __attribute__((address_space(4))) const_off_t;
    return (const_off_t*)((const_byte_t*)__builtin_amdgcn_kernarg_segment_ptr() +
                          offsetof(gemm_args_t, group_off));
}

// Fragment read i of R goes behind matrix instruction i (N - 1) / R of a k-step's N: the index of
// the read behind instruction q, or -1
constexpr int spread_read(int q, int n, int r)
{
    for (int i = 0; i != r; ++i) {
        if (i * (n - 1) / r == q) return i;
    }
    return -1;
}

template <int BM, int BN, bool KW>
__global__ __launch_bounds__(512) void gemm_pc_kernel(gemm_args_t a, uint32_t total_tiles)
{
    using T = _Float16;
    using std::integral_constant;
    constexpr int NS = 3;
    constexpr int MI = 16, VL = 8, WGN = 2;
    constexpr int KS = BK / 32;  // k-steps (16 x 16 x 32 matrix instructions along k) per slice
    constexpr int BAND = 32;     // rows per turn of the epilogue
    constexpr int TMB = BM / 2 / BAND;
    constexpr int WM = BM / 2, WN = BN / 2;
    constexpr int TM = WM / MI, TN = WN / MI;
    constexpr int NT = TM * TN;  // accumulator tiles per multiplying wave
    constexpr int STAGE = (BM + BN) * RB;
    constexpr int A_BYTES = BM * RB;
    constexpr int NLA = BM / 32, NLB = BN / 32;  // load instructions per loading wave per slice
    constexpr int LP = NLA + NLB;
    constexpr int READS = TM + TN;
    static_assert(NT * 4 <= 128 && READS < NT && KS == 2, "");
    constexpr int STRIP_PITCH = WN * int(sizeof(T)) + 16;
    constexpr int CPR = WN * int(sizeof(T)) / 16;  // 16-byte chunks per strip row
    constexpr int CPL = BAND * CPR / 64;           // chunks per lane per band
    static_assert(4 * BAND * STRIP_PITCH <= STAGE, "");

    extern __shared__ __attribute__((aligned(16))) char lds[];
    uint32_t const lds_base = uint32_t(uintptr_t((__attribute__((address_space(3))) char*)lds));

#ifdef ES_W4_STAMP
    uint64_t const stamp_entry = __builtin_amdgcn_s_memtime();
#endif
    int const tid = threadIdx.x;
    int const lane = tid & 63;
    int const wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int const role_wave = wave & 3;  // index among the waves of its role
    int const wm = role_wave / WGN, wn = role_wave % WGN;

    claim_accumulators_128();

    uint32_t const n_tiles = a.tiles_m * a.tiles_n;
    uint32_t const nk = a.K / BK;  // >= NS (checked by the launcher)
    uint32_t const G = gridDim.x;
    uint32_t const my_tiles = (total_tiles - blockIdx.x + G - 1) / G;

    struct tile_t {
        uint32_t tm, tn, bz;
    };
    auto locate = [&](uint32_t L) ES_INLINE {
        uint32_t bz = L / n_tiles;
        uint32_t tile = L - bz * n_tiles;
        xcd_renumber(a, n_tiles, tile, bz);
        constexpr uint32_t GROUP_M = 4;
        uint32_t const     in_group = GROUP_M * a.tiles_n;
        uint32_t const group = a.group_magic ? __umulhi(tile, a.group_magic) : tile / in_group;
        uint32_t const in_g = tile - group * in_group;
        uint32_t const first_m = group * GROUP_M;
        uint32_t const rows =
            (a.tiles_m - first_m) < GROUP_M ? (a.tiles_m - first_m) : GROUP_M;
        tile_t t;
        t.tm = first_m + in_g % rows;
        t.tn = in_g / rows;
        t.bz = bz;
        return t;
    };

    if (wave < 4) {
        // ================================================================ multiplying waves
        static_for<NT * 4>([](auto r) ES_INLINE { acc_clear<decltype(r)::value>(); });
        // k-step s, MFMA tile row r0 + lane % 16: k-chunk 4 s + lane / 16, found in slot
        // chunk ^ bits 1..3 of the row
        int const f_sw = ((lane % MI) >> 1) & 7;
        int       f_off[KS];
#pragma unroll
        for (int s = 0; s != KS; ++s) {
            f_off[s] = (lane % MI) * RB + (((4 * s + lane / MI) ^ f_sw) * 16);
        }
        int const fa_base = wm * WM * RB;
        int const fb_base = A_BYTES + wn * WN * RB;
        chunk_t   fa[2][TM], fb[2][TN];
        auto read_frag = [&](char const* stage, auto s_tag, auto q_tag, chunk_t(&xa)[TM],
                             chunk_t(&xb)[TN]) ES_INLINE {
            constexpr int s = decltype(s_tag)::value, q = decltype(q_tag)::value;
            if constexpr (q == 0) {
                xa[0] = *reinterpret_cast<chunk_t const*>(stage + fa_base + f_off[s]);
            } else if constexpr (q <= TN) {
                xb[q - 1] = *reinterpret_cast<chunk_t const*>(stage + fb_base + (q - 1) * MI * RB +
                                                              f_off[s]);
            } else {
                xa[q - TN] = *reinterpret_cast<chunk_t const*>(stage + fa_base +
                                                               (q - TN) * MI * RB + f_off[s]);
            }
        };
        // The four multiplying waves share one LDS port of 128 bytes a cycle and a fragment
        // read is 1 KiB per wave, a matrix instruction 16 cycles: one read per instruction
        // from every wave asks for twice what the port gives, and the instructions behind
        // the full queue wait.  Read i of a k-step goes behind instruction i (NT - 1) / READS.
        uint32_t st = 0;  // stage of the slice being computed
        auto slice = [&]() ES_INLINE {
            uint32_t const nx = st + 1 == NS ? 0 : st + 1;
            char const*    cur = lds + st * STAGE;
            char const*    nxt = lds + nx * STAGE;
            static_for<KS - 1>([&](auto s_tag) ES_INLINE {
                constexpr int s = decltype(s_tag)::value;
                static_for<NT>([&](auto q_tag) ES_INLINE {
                    constexpr int q = decltype(q_tag)::value;
                    mma16<q>(fb[s & 1][q % TN], fa[s & 1][q / TN]);
                    if constexpr (spread_read(q, NT, READS) >= 0) {
                        read_frag(cur, integral_constant<int, s + 1>{},
                                  integral_constant<int, spread_read(q, NT, READS)>{}, fa[(s + 1) & 1],
                                  fb[(s + 1) & 1]);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                });
            });
            static_for<NT>([&](auto q_tag) ES_INLINE {
                constexpr int q = decltype(q_tag)::value;
                mma16<q>(fb[(KS - 1) & 1][q % TN], fa[(KS - 1) & 1][q / TN]);
                if constexpr (q == 0) {
                    // all of this stage has been read; behind the barrier the next has landed
                    asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
                    __builtin_amdgcn_s_barrier();
                } else if constexpr (spread_read(q - 1, NT, READS) >= 0) {
                    read_frag(nxt, integral_constant<int, 0>{},
                              integral_constant<int, spread_read(q - 1, NT, READS)>{}, fa[0], fb[0]);
                }
                __builtin_amdgcn_sched_barrier(0);
            });
            st = nx;
        };
        // 32 rows of this wave's part of C, converted: band I holds the accumulator tiles of rows
        // 32 I .. 32 I + 31 (quad g: row 16 (g / TN) + lane % 16 of the band, the four
        // consecutive n from 16 (g % TN) + lane / 16 * 4 on); the accumulators are cleared on
        // the way
        float const alpha = float(a.alpha);
        typedef T   quad_t __attribute__((ext_vector_type(4)));
        constexpr int QB = (BAND / MI) * TN;  // quads per band
        quad_t      band[QB];
        auto convert = [&](auto i_tag) ES_INLINE {
            constexpr int i = decltype(i_tag)::value;
            static_for<QB>([&](auto g_tag) ES_INLINE {
                constexpr int g = decltype(g_tag)::value;
                constexpr int R = (i * QB + g) * 4;
                quad_t        q;
                q[0] = T(acc_read<R>() * alpha);
                q[1] = T(acc_read<R + 1>() * alpha);
                q[2] = T(acc_read<R + 2>() * alpha);
                q[3] = T(acc_read<R + 3>() * alpha);
                acc_clear<R>();
                acc_clear<R + 1>();
                acc_clear<R + 2>();
                acc_clear<R + 3>();
                band[g] = q;
            });
        };

        __builtin_amdgcn_s_barrier();  // slice 0 has landed
        static_for<READS>([&](auto q_tag) ES_INLINE {
            read_frag(lds, integral_constant<int, 0>{}, q_tag, fa[0], fb[0]);
        });
        for (uint32_t it = 0; it != my_tiles; ++it) {
#ifdef ES_W4_STAMP
            uint64_t const stamp0 = __builtin_amdgcn_s_memtime();
#endif
            for (uint32_t kt = 0; kt + 1 < nk; ++kt) slice();
            uint32_t const freed = st;
            slice();
            char* const strip = lds + freed * STAGE + role_wave * (BAND * STRIP_PITCH);
#ifdef ES_W4_STAMP
            uint64_t const stamp1 = __builtin_amdgcn_s_memtime();
#endif
            settle();
            convert(integral_constant<int, 0>{});
            static_for<TMB>([&](auto i_tag) ES_INLINE {
                constexpr int i = decltype(i_tag)::value;
                if constexpr (i > 0) __builtin_amdgcn_s_barrier();  // the strips have been read
                static_for<QB>([&](auto g_tag) ES_INLINE {
                    constexpr int g = decltype(g_tag)::value;
                    int const     n = (g % TN) * MI + (lane / MI) * 4;
                    *reinterpret_cast<quad_t*>(strip + ((g / TN) * MI + lane % MI) * STRIP_PITCH +
                                               n * int(sizeof(T))) = band[g];
                });
                asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
                __builtin_amdgcn_s_barrier();  // the strips are written
                if constexpr (i + 1 < TMB) convert(integral_constant<int, i + 1>{});
            });
#ifdef ES_W4_STAMP
            {
                uint64_t const stamp2 = __builtin_amdgcn_s_memtime();
                asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
                if (tid == 0 && it < 8) {
                    uint64_t* dst =
                        reinterpret_cast<uint64_t*>(a.ws) + (size_t(blockIdx.x) * 8 + it) * 4;
                    dst[0] = stamp0;
                    dst[1] = stamp1;
                    dst[2] = stamp2;
                    dst[3] = stamp_entry;
                }
            }
#endif
        }
        return;
    }

    // ===================================================================== loading waves
    // Load instruction i of this wave covers rows (4 i + p) * 8 + lane / 8 of the tile's A (or
    // B) rows (p: the wave's index among the loading waves); the lane's LDS slot is chunk
    // lane % 8 of that row and holds global chunk (lane % 8) ^ bits 1..3 of the row.
    uint32_t const lds_wave = lds_base + uint32_t(role_wave) * 1024;
    uint32_t const load_chunk =
        uint32_t((lane & 7) ^ (((lane >> 4) & 3) | ((role_wave & 1) << 2)));
    uint32_t voa[NLA], vob[NLB];  // byte offsets of the lane's chunk within slice 0
    T const *A_ld = nullptr, *B_ld = nullptr;
    T const *A_tile = nullptr, *B_tile = nullptr;
    uint32_t L_ld = blockIdx.x, kt_ld = 0;
    uint32_t k_dig[MAXG] = {0, 0, 0, 0};
    int64_t  k_wa = 0, k_wb = 0;
    auto uniform = [](T const* p) ES_INLINE {
        uint64_t const v = reinterpret_cast<uint64_t>(p);
        uint32_t const lo = __builtin_amdgcn_readfirstlane(uint32_t(v));
        uint32_t const hi = __builtin_amdgcn_readfirstlane(uint32_t(v >> 32));
        return reinterpret_cast<T const*>((uint64_t(hi) << 32) | lo);
    };
    auto seek_tile = [&](uint32_t L) ES_INLINE {
        tile_t const t = locate(L);
        int64_t      boa, bob;
        if (a.grouped) {
            boa = group_table()[t.bz];
            bob = group_table()[8 + t.bz];
        } else {
            group_offsets(a.gb, t.bz, boa, bob);
        }
        A_tile = uniform(static_cast<T const*>(a.A) + boa);
        B_tile = uniform(static_cast<T const*>(a.B) + bob);
        uint32_t const lane_a = load_chunk * VL * uint32_t(a.gk.sx[0]) * uint32_t(sizeof(T));
        uint32_t const lane_b = load_chunk * VL * uint32_t(a.gk.sy[0]) * uint32_t(sizeof(T));
#pragma unroll
        for (int i = 0; i != NLA; ++i) {
            int64_t  x, y;
            uint32_t r = t.tm * BM + uint32_t((4 * i + role_wave) * 8 + lane / 8);
            r = r < a.M ? r : a.M - 1;
            group_offsets(a.gm, r, x, y);
            voa[i] = uint32_t(x) * uint32_t(sizeof(T)) + lane_a;
        }
#pragma unroll
        for (int i = 0; i != NLB; ++i) {
            int64_t  x, y;
            uint32_t r = t.tn * BN + uint32_t((4 * i + role_wave) * 8 + lane / 8);
            r = r < a.N ? r : a.N - 1;
            group_offsets(a.gn, r, x, y);
            vob[i] = uint32_t(x) * uint32_t(sizeof(T)) + lane_b;
        }
        A_ld = A_tile;
        B_ld = B_tile;
        kt_ld = 0;
        if constexpr (KW) {
            k_wa = k_wb = 0;
#pragma unroll
            for (int d = 0; d != MAXG; ++d) k_dig[d] = 0;
        }
    };
    int64_t const step_a = BK * a.gk.sx[0], step_b = BK * a.gk.sy[0];
    uint32_t      st_ld = 0;        // stage the next slice goes to
    uint32_t      to_issue = my_tiles * nk;  // slices not yet issued
    // the loader's slice into its stage, then on to the next slice (of this tile or of this
    // workgroup's next one)
    auto issue_slice = [&]() ES_INLINE {
        if (to_issue == 0) return;
        --to_issue;
        uint32_t const stage = lds_wave + st_ld * STAGE;
        static_for<LP>([&](auto q_tag) ES_INLINE {
            constexpr int q = decltype(q_tag)::value;
            if constexpr (q < NLA) {
                load_lds<4 * q * 1024>(A_ld, voa[q], stage);
            } else {
                load_lds<A_BYTES + 4 * (q - NLA) * 1024>(B_ld, vob[q - NLA], stage);
            }
        });
        st_ld = st_ld + 1 == NS ? 0 : st_ld + 1;
        ++kt_ld;
        if (kt_ld == nk) {
            L_ld += G;
            if (L_ld < total_tiles) seek_tile(L_ld);
            return;
        }
        if constexpr (!KW) {
            A_ld += step_a;
            B_ld += step_b;
        } else {
            k_dig[0] += BK;
            k_wa += step_a;
            k_wb += step_b;
#pragma unroll
            for (int d = 0; d + 1 != MAXG; ++d) {
                if (k_dig[d] == a.gk.size[d]) {
                    k_dig[d] = 0;
                    k_dig[d + 1] += 1;
                    k_wa += a.gk.sx[d + 1] - int64_t(a.gk.size[d]) * a.gk.sx[d];
                    k_wb += a.gk.sy[d + 1] - int64_t(a.gk.size[d]) * a.gk.sy[d];
                }
            }
            A_ld = A_tile + k_wa;
            B_ld = B_tile + k_wb;
        }
    };

    seek_tile(L_ld);
    static_for<NS>([&](auto) ES_INLINE { issue_slice(); });  // nk >= NS: all in the first tile
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"((NS - 1) * LP) : "memory");
    __builtin_amdgcn_s_barrier();  // slice 0 has landed
    uint32_t to_land = my_tiles * nk - 1;  // slices after the one being computed
    uint32_t st_c = 0;                     // stage of the slice being computed
    for (uint32_t it = 0; it != my_tiles; ++it) {
        for (uint32_t kt = 0; kt != nk; ++kt) {
            // slice g is being computed; before the barrier slice g + 1 must have landed:
            // everything but the youngest slice in flight, if there is one
            if (to_land >= 2) {
                asm volatile("s_waitcnt vmcnt(%0)" : : "n"(LP) : "memory");
            } else {
                asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
            }
            if (to_land) --to_land;
            __builtin_amdgcn_s_barrier();
            // the stage of slice g is free -- unless the tile ends here: then it is the
            // epilogue's first
            if (kt + 1 != nk) {
                issue_slice();
                st_c = st_c + 1 == NS ? 0 : st_c + 1;
            }
        }
        // ---- this wave's share of the epilogue: the strip of the multiplying wave with the
        // same index, 32 rows at a time, as whole 16-byte chunks
        uint32_t const freed = st_c;  // the stage of the tile's last slice
        st_c = st_c + 1 == NS ? 0 : st_c + 1;
        tile_t const   t = locate(blockIdx.x + it * G);
        int64_t        boc;
        if (a.grouped) {
            boc = group_table()[16 + t.bz];
        } else if (a.gb.n == 1) {
            boc = int64_t(t.bz) * a.gb.sz[0];
        } else {
            boc = 0;
            uint32_t i = t.bz;
#pragma unroll
            for (int d = 0; d != MAXG; ++d) {
                uint32_t q = i / a.gb.size[d];
                boc += int64_t(i - q * a.gb.size[d]) * a.gb.sz[d];
                i = q;
            }
        }
        T* const          C = static_cast<T*>(a.C) + boc;
        char const* const strip = lds + freed * STAGE + role_wave * (BAND * STRIP_PITCH);
        static_for<TMB>([&](auto i_tag) ES_INLINE {
            constexpr int i = decltype(i_tag)::value;
            __builtin_amdgcn_s_barrier();  // the strips are written
            chunk_t v[CPL];
#pragma unroll
            for (int c = 0; c != CPL; ++c) {
                int const idx = c * 64 + lane;
                v[c] = *reinterpret_cast<chunk_t const*>(strip + (idx / CPR) * STRIP_PITCH +
                                                         (idx % CPR) * 16);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
            if constexpr (i + 1 < TMB) __builtin_amdgcn_s_barrier();  // the strips have been read
#pragma unroll
            for (int c = 0; c != CPL; ++c) {
                int const      idx = c * 64 + lane;
                uint32_t const m = t.tm * BM + wm * WM + i * BAND + uint32_t(idx / CPR);
                uint32_t const n = t.tn * BN + wn * WN + uint32_t(idx % CPR) * VL;
                if (m < a.M && n < a.N) {
                    int64_t mo_a, mo_c, no_b, no_c;
                    group_offsets(a.gm, m, mo_a, mo_c);
                    group_offsets(a.gn, n, no_b, no_c);
                    chunk_t* const dst = reinterpret_cast<chunk_t*>(C + mo_c + no_c);
                    if (a.c_stream) {
                        store_16_streaming(dst, v[c]);
                    } else {
                        *dst = v[c];
                    }
                }
            }
        });
        issue_slice();  // the slice the freed stage was waiting for
    }
    // nothing may still be on its way into this workgroup's LDS when it ends
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
}

inline bool gemm_pc_eligible(gemm_args_t const& a)
{
    return w4::gemm_w4_eligible<3>(a);
}

template <int BM, int BN, bool KW>
void launch_gemm_pc_kw(gemm_args_t const& a, uint32_t workgroups, hipStream_t stream)
{
    constexpr int lds = 3 * (BM + BN) * RB;
    static bool const raised = [] {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_pc_kernel<BM, BN, KW>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        return true;
    }();
    (void)raised;
    uint64_t const total = uint64_t(a.tiles_m) * a.tiles_n * a.batch;
    uint32_t const grid = uint32_t(total < workgroups ? total : workgroups);
    hipLaunchKernelGGL((gemm_pc_kernel<BM, BN, KW>), dim3(grid), dim3(512), lds, stream, a,
                       uint32_t(total));
}

template <int BM, int BN>
void launch_gemm_pc(gemm_args_t const& a, uint32_t workgroups, hipStream_t stream)
{
    if (a.gk.n == 1) {
        launch_gemm_pc_kw<BM, BN, false>(a, workgroups, stream);
    } else {
        launch_gemm_pc_kw<BM, BN, true>(a, workgroups, stream);
    }
}

}  // namespace pc
}  // namespace gemm
}  // namespace es
