// Persistent fp16 GEMM for the compute-bound products: four wavefronts, one per SIMD, each
// owning a quarter of a 256 x 256 (or 128 x 256 / 256 x 128) tile of C, operand slices of 128
// bytes per row straight from global memory into LDS, and every workgroup walking through
// several tiles with the next tile's first slices already in flight while the current tile
// is written out.
//
// What this kernel does that gemm_dma_kernel does not, and why:
//   * The accumulators live in named accumulation registers.  A wave with 128 x 128 of C
//     holds 256 of them, all of a[0:255]; left to the register allocator they are split
//     between a and v registers, moved to and fro around every matrix instruction and
//     spilled.  Here the matrix instructions, the clearing and the reads are assembly
//     statements on fixed registers (a[4 t : 4 t + 3] is accumulator tile t of 16 x 16), so
//     the main loop is matrix instructions, LDS reads and load issues and nothing else.  With
//     one wave per SIMD a wave reads 0.25 LDS vectors per matrix instruction where two waves
//     of 128 x 64 read 0.375.
//   * The load path of a compute unit takes 64 bytes per cycle and a 256 x 256 x 64 slice is
//     64 KiB: half of the time the matrix instructions of the slice take.  Four waves that
//     issue all their loads of a slice behind one barrier fill the queue and then stand at
//     the issue of the next load, and a wave that stands cannot issue matrix instructions
//     either (per-slice cycle stamps: 2810 cycles against 2048 of matrix work; 2440 with the
//     loads of a slice issued one per two matrix instructions over two k-steps).
//   * A tile's set-up, the latency of its first loads and its epilogue cost 11 + 22 thousand
//     cycles when every tile is a workgroup of its own (a tenth of a 256 x 256 x 8192 tile,
//     a fifth at K = 4096).  A persistent workgroup computes the next tile's addresses and
//     issues its first slices before the current tile's last slice is done, so only the
//     epilogue's own instructions remain between two tiles.
//
// Hazards the compiler does not see (it does not know the statements are matrix
// instructions): between two uses of one accumulator tile the loop goes round all tiles (the
// same-opcode back-to-back case needs no idle slots anyway); before the epilogue reads an
// accumulator and before the first matrix instruction after clearing, settle() idles.
#pragma once
#include <utility>

#define ES_INLINE __attribute__((always_inline))

#include "gemm_dma_kernel.h"

namespace es
{
namespace gemm
{
namespace w4
{

template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>)
{
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// Accumulator tile T (a[4 T .. 4 T + 3]) += x * y with the 16 x 16 x 32 instruction: x holds, per lane,
// eight k elements (k = lane / 16 * 8 ..) of row lane % 16 of the 16 rows of the result, y
// the same of its 16 columns; the lane gets rows lane / 16 * 4 .. + 3 of column lane % 16.
// Per flop it moves half the accumulator registers of the 32 x 32 x 16 instruction, and under
// the board's power limit that is worth a tenth of the clock: the same kernel, instruction
// exchanged, ran 8192^3 at 1449 instead of 1311 TFLOP/s.
template <int T>
__device__ __forceinline__ void mma16(chunk_t const& x, chunk_t const& y)
{
    asm volatile("v_mfma_f32_16x16x32_f16 a[%0:%1], %2, %3, a[%0:%1]"
                 :
                 : "n"(4 * T), "n"(4 * T + 3), "v"(x), "v"(y));
}

template <int R>
__device__ __forceinline__ float acc_read()
{
    float v;
    asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(v) : "n"(R));
    return v;
}

template <int R>
__device__ __forceinline__ void acc_clear()
{
    asm volatile("v_accvgpr_write_b32 a[%0], 0" : : "n"(R));
}

// An 8-pass matrix instruction's result may be read by another unit 11 issue slots after it
// was issued at the earliest; a cleared accumulator may be an operand 2 slots after the write.
__device__ __forceinline__ void settle()
{
    asm volatile("s_nop 15\n\ts_nop 7" : : : "memory");
}

// Tells the compiler that the kernel uses a[0:255]: they count for the kernel's register
// allocation, and nothing of the compiler's own is kept in them across this statement (the
// compiler has no reason to use one afterwards: the kernel needs far fewer than 256 v
// registers).
#define ES_A10(n) "a" #n "0", "a" #n "1", "a" #n "2", "a" #n "3", "a" #n "4", "a" #n "5", "a" #n "6", "a" #n "7", "a" #n "8", "a" #n "9"
__device__ __forceinline__ void claim_accumulators()
{
    asm volatile(""
                 :
                 :
                 : "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", ES_A10(1),
                   ES_A10(2), ES_A10(3), ES_A10(4), ES_A10(5), ES_A10(6), ES_A10(7), ES_A10(8),
                   ES_A10(9), ES_A10(10), ES_A10(11), ES_A10(12), ES_A10(13), ES_A10(14),
                   ES_A10(15), ES_A10(16), ES_A10(17), ES_A10(18), ES_A10(19), ES_A10(20),
                   ES_A10(21), ES_A10(22), ES_A10(23), ES_A10(24), "a250", "a251", "a252", "a253",
                   "a254", "a255");
}
// the same for a kernel whose waves hold 128 accumulators (two waves per SIMD)
__device__ __forceinline__ void claim_accumulators_128()
{
    asm volatile(""
                 :
                 :
                 : "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", ES_A10(1),
                   ES_A10(2), ES_A10(3), ES_A10(4), ES_A10(5), ES_A10(6), ES_A10(7), ES_A10(8),
                   ES_A10(9), ES_A10(10), ES_A10(11), "a120", "a121", "a122", "a123", "a124",
                   "a125", "a126", "a127");
}
#undef ES_A10

// 64 lanes x 16 bytes from `base + voff` (per lane) to LDS at `lds_addr + OFF + 16 * lane`
template <int OFF>
__device__ __forceinline__ void load_lds(void const* base, uint32_t voff, uint32_t lds_addr)
{
    asm volatile(
        "s_add_u32 m0, %0, %3\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %1, %2"
        :
        : "s"(lds_addr), "v"(voff), "s"(base), "n"(OFF)
        : "memory", "scc");
}

template <int VM>
__device__ __forceinline__ void wait_vm_lgkm()
{
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" : : "n"(VM) : "memory");
}

constexpr int RB = 128;  // bytes of k per row per slice
constexpr int BK = 64;   // elements of k per slice

// KW: several k modes (the slice walker steps digit by digit); otherwise a slice is one stride on
template <int BM, int BN, int NS, bool KW>
__global__ __launch_bounds__(256) void gemm_w4_kernel(gemm_args_t a, uint32_t total_tiles)
{
    using T = _Float16;
    constexpr int MI = 16, VL = 8, NW = 4, WGN = 2;
    constexpr int KS = BK / 32;  // k-steps (matrix instructions along k) per slice
    constexpr int BAND = 32;     // rows per turn of the epilogue
    constexpr int WM = BM / 2, WN = BN / 2;
    constexpr int TM = WM / MI, TN = WN / MI;
    constexpr int NT = TM * TN;  // accumulator tiles per wave
    constexpr int STAGE = (BM + BN) * RB;
    constexpr int A_BYTES = BM * RB;
    constexpr int NLA = BM / 32, NLB = BN / 32;  // load instructions per wave per slice
    constexpr int LOADS = NLA + NLB;
    constexpr int READS = TM + TN;
    // the loads of a slice are issued in PARTS parts: part 0 in the last k-step of the slice
    // that frees the stage, the others in the first k-steps of the slice after it.  With two
    // stages a load must land within one slice of being issued: two parts; with three there
    // is a slice more
    constexpr int PARTS = 2;
    static_assert(NS == 2 && KS == 2, "the schedule below: two stages, two k-steps per slice");
    static_assert(NT * 4 <= 256 && READS < NT / 2 && LOADS % PARTS == 0 && NT % 2 == 0, "");

    extern __shared__ __attribute__((aligned(16))) char lds[];
    uint32_t const lds_base = uint32_t(uintptr_t((__attribute__((address_space(3))) char*)lds));

    int const tid = threadIdx.x;
    int const lane = tid & 63;
    int const wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int const wm = wave / WGN, wn = wave % WGN;
    uint32_t const lds_wave = lds_base + uint32_t(wave) * 1024;

    claim_accumulators();
    static_for<NT * 4>([](auto r) ES_INLINE { acc_clear<decltype(r)::value>(); });

    uint32_t const n_tiles = a.tiles_m * a.tiles_n;
    uint32_t const nk = a.K / BK;  // >= NS (checked by the launcher)
    uint32_t const G = gridDim.x;

    // ---- where tile number L (this workgroup computes L = blockIdx.x, + G, + 2 G, ...) lies
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

    // ---- loader: the slice whose loads are being issued.  While slice g is computed (from
    // stage g mod NS) that is slice g + NS - 1 (into the stage before it) until the k-step
    // before last, then slice g + NS (into the stage that slice g frees).
    // Load instruction i of this wave covers rows (4 i + wave) * 8 + lane / 8 of the tile's A
    // (or B) rows; the lane's LDS slot is chunk lane % 8 of that row and holds global chunk
    // (lane % 8) ^ bits 1..3 of the row: sixteen consecutive rows of one k-chunk cover all
    // banks once on the fragment read.
    uint32_t const load_chunk = uint32_t((lane & 7) ^ (((lane >> 4) & 3) | ((wave & 1) << 2)));
    uint32_t       voa[NLA], vob[NLB];  // byte offsets of the lane's chunk within slice 0
    T const *      A_ld = nullptr, *B_ld = nullptr;  // + the slice's first k element
    uint32_t       L_ld = blockIdx.x;
    // several k modes: the element offsets of the slice's first k element are stepped from
    // slice to slice (the innermost mode holds whole slices: checked by the launcher)
    uint32_t k_dig[MAXG] = {0, 0, 0, 0};
    int64_t  k_wa = 0, k_wb = 0;
    T const *A_tile = nullptr, *B_tile = nullptr;
    auto uniform = [](T const* p) ES_INLINE {
        uint64_t const v = reinterpret_cast<uint64_t>(p);
        uint32_t const lo = __builtin_amdgcn_readfirstlane(uint32_t(v));
        uint32_t const hi = __builtin_amdgcn_readfirstlane(uint32_t(v >> 32));
        return reinterpret_cast<T const*>((uint64_t(hi) << 32) | lo);
    };
    auto rewind_k = [&]() ES_INLINE {
        A_ld = A_tile;
        B_ld = B_tile;
        if constexpr (KW) {
            k_wa = k_wb = 0;
#pragma unroll
            for (int d = 0; d != MAXG; ++d) k_dig[d] = 0;
        }
    };
    auto seek_tile = [&](uint32_t L) ES_INLINE {
        tile_t const t = locate(L);
        int64_t      boa, bob;
        group_offsets(a.gb, t.bz, boa, bob);
        A_tile = uniform(static_cast<T const*>(a.A) + boa);
        B_tile = uniform(static_cast<T const*>(a.B) + bob);
        uint32_t const lane_a = load_chunk * VL * uint32_t(a.gk.sx[0]) * uint32_t(sizeof(T));
        uint32_t const lane_b = load_chunk * VL * uint32_t(a.gk.sy[0]) * uint32_t(sizeof(T));
#pragma unroll
        for (int i = 0; i != NLA; ++i) {
            int64_t  x, y;
            uint32_t r = t.tm * BM + uint32_t((NW * i + wave) * 8 + lane / 8);
            r = r < a.M ? r : a.M - 1;
            group_offsets(a.gm, r, x, y);
            voa[i] = uint32_t(x) * uint32_t(sizeof(T)) + lane_a;
        }
#pragma unroll
        for (int i = 0; i != NLB; ++i) {
            int64_t  x, y;
            uint32_t r = t.tn * BN + uint32_t((NW * i + wave) * 8 + lane / 8);
            r = r < a.N ? r : a.N - 1;
            group_offsets(a.gn, r, x, y);
            vob[i] = uint32_t(x) * uint32_t(sizeof(T)) + lane_b;
        }
        rewind_k();
    };
    // load q of the loader's slice into the stage whose first slot of this wave is `slot`: A
    // rows for q < NLA, B rows after that; the instruction's own slot is a constant
    auto issue = [&](uint32_t slot, auto q_tag) ES_INLINE {
        constexpr int q = decltype(q_tag)::value;
        if constexpr (q < NLA) {
            load_lds<NW * q * 1024>(A_ld, voa[q], slot);
        } else {
            load_lds<A_BYTES + NW * (q - NLA) * 1024>(B_ld, vob[q - NLA], slot);
        }
    };
    // on to the next slice of the loader's tile
    int64_t const step_a = BK * a.gk.sx[0], step_b = BK * a.gk.sy[0];
    auto next_slice = [&]() ES_INLINE {
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
    // On to the first slice of this workgroup's next tile.  Behind its last tile the loader
    // goes round that tile again: the loads stay what they are in every slice (so do the
    // counts the waits rely on), what they bring is never read, and the kernel ends only
    // when they have landed.
    auto next_tile = [&]() ES_INLINE {
        if (L_ld + G < total_tiles) {
            L_ld += G;
            seek_tile(L_ld);
        } else {
            rewind_k();
        }
    };

    // ---- fragments
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
    // read order: what the first matrix instructions of a step need comes first
    auto read_frag = [&](char const* stage, auto s_tag, auto q_tag, chunk_t(&xa)[TM],
                         chunk_t(&xb)[TN]) ES_INLINE {
        constexpr int s = decltype(s_tag)::value, q = decltype(q_tag)::value;
        if constexpr (q == 0) {
            xa[0] = *reinterpret_cast<chunk_t const*>(stage + fa_base + f_off[s]);
        } else if constexpr (q <= TN) {
            xb[q - 1] =
                *reinterpret_cast<chunk_t const*>(stage + fb_base + (q - 1) * MI * RB + f_off[s]);
        } else {
            xa[q - TN] =
                *reinterpret_cast<chunk_t const*>(stage + fa_base + (q - TN) * MI * RB + f_off[s]);
        }
    };
    using std::integral_constant;

    // ---- prologue: slices 0 .. NS-2 whole and part 0 of slice NS-1 in flight
    seek_tile(L_ld);
    static_for<NS - 1>([&](auto st_tag) ES_INLINE {
        static_for<LOADS>([&](auto q_tag) ES_INLINE {
            issue(lds_wave + decltype(st_tag)::value * STAGE, q_tag);
        });
        next_slice();  // nk >= NS: still inside the first tile
    });
    static_for<LOADS / PARTS>([&](auto q_tag) ES_INLINE {
        issue(lds_wave + (NS - 1) * STAGE, q_tag);
    });
    wait_vm_lgkm<(NS - 2) * LOADS + LOADS / PARTS>();
    __builtin_amdgcn_s_barrier();
    static_for<READS>([&](auto q_tag) ES_INLINE {
        read_frag(lds, integral_constant<int, 0>{}, q_tag, fa[0], fb[0]);
    });

    // One slice, computed from stage st, in two halves with the loader's step between them.
    // The four waves' fragment reads share one LDS port of 128 bytes a cycle, and a read is
    // 1 KiB per wave: more than one read per two matrix instructions (16 cycles each) fills
    // the port's queue and the matrix instructions behind it wait.  So the reads are spread:
    // k-step 0 reads the fragments of k-step 1 one per four instructions, and -- one per
    // eight, two rows of tiles ahead of their use -- the A fragments of its own k-step from
    // the fourth on (JIT), which leaves the second half of k-step 1 with the eleven reads
    // k-step 0 starts on.  The second part of the loader's slice goes to the stage before st
    // in the first half of k-step 0, a load per four matrix instructions (more would fill
    // the load path; later ones would land too late).
    constexpr int JIT = 3;             // first A fragment of k-step 0 that k-step 0 reads itself
    constexpr int EARLY = TN + JIT;    // reads of k-step 0 left to the k-step before it
    static_assert(NT == 64 && TN == 8 && READS == 16 && LOADS / PARTS == 8, "");
    uint32_t st = 0;  // stage of the slice being computed
    auto head = [&]() ES_INLINE {
        char const*    cur = lds + st * STAGE;
        uint32_t const ld_slot = lds_wave + (st == 0 ? NS - 1 : st - 1) * STAGE;
        static_for<NT>([&](auto q_tag) ES_INLINE {
            constexpr int q = decltype(q_tag)::value;
            mma16<q>(fb[0][q % TN], fa[0][q / TN]);
            if constexpr (q % 4 == 1) {
                read_frag(cur, integral_constant<int, 1>{}, integral_constant<int, q / 4>{}, fa[1],
                          fb[1]);
            }
            if constexpr (q % TN == 0 && q / TN + 2 >= JIT && q / TN + 2 < TM) {
                read_frag(cur, integral_constant<int, 0>{},
                          integral_constant<int, TN + q / TN + 2>{}, fa[0], fb[0]);
            }
            if constexpr (q % 4 == 3 && q < NT / 2) {
                issue(ld_slot, integral_constant<int, LOADS / PARTS + q / 4>{});
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    // k-step 1.  Half-way through it the next slice must have landed; this stage has been
    // read in full by then (its k-step 1 went to registers during k-step 0), so behind the
    // barrier it takes the first part of the loader's new slice -- unless this is the tile's
    // LAST slice: then the freed stage is the epilogue's first.
    auto tail = [&](auto last_tag) ES_INLINE {
        constexpr bool LAST = decltype(last_tag)::value;
        uint32_t const nx = st + 1 == NS ? 0 : st + 1;
        char const*    nxt = lds + nx * STAGE;
        uint32_t const ld_slot = lds_wave + st * STAGE;
        static_for<NT>([&](auto q_tag) ES_INLINE {
            constexpr int q = decltype(q_tag)::value;
            mma16<q>(fb[1][q % TN], fa[1][q / TN]);
            if constexpr (q == NT / 2) {
                // this wave's part of the next slice has landed and its reads of this stage
                // are complete; after the barrier that holds for the whole workgroup
                wait_vm_lgkm<(NS - 2) * LOADS>();
                __builtin_amdgcn_s_barrier();
            } else if constexpr (q > NT / 2) {
                constexpr int r = q - NT / 2 - 1;
                if constexpr (r % 3 == 0 && r / 3 < EARLY) {
                    read_frag(nxt, integral_constant<int, 0>{}, integral_constant<int, r / 3>{},
                              fa[0], fb[0]);
                }
                if constexpr (!LAST && r % 3 == 1 && r / 3 < LOADS / PARTS) {
                    issue(ld_slot, integral_constant<int, r / 3>{});
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        st = nx;
    };

    // ---- epilogue of one tile: each wave turns 32 rows of its part through an LDS strip in
    // the stage that has just been freed, so that the global stores are 16 bytes per lane
    // and whole row segments; the accumulators are cleared on the way.  All chunks of a band
    // are read back before the first store, so the LDS latency is paid once per band.
    constexpr int STRIP_PITCH = WN * int(sizeof(T)) + 16;
    constexpr int CPR = WN * int(sizeof(T)) / 16;
    constexpr int CPL = BAND * CPR / 64;  // chunks per lane per band
    static_assert(NW * BAND * STRIP_PITCH <= STAGE, "");
    float const alpha = float(a.alpha);
    auto epilogue = [&](uint32_t L, uint32_t freed_stage) ES_INLINE {
        tile_t const t = locate(L);
        int64_t      boc;
        if (a.gb.n == 1) {
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
        T* const    C = static_cast<T*>(a.C) + boc;
        char* const strip = lds + freed_stage * STAGE + wave * (BAND * STRIP_PITCH);
        typedef T   quad_t __attribute__((ext_vector_type(4)));
        // this lane's chunks of a band: rows lane / CPR + c * (64 / CPR), 16 bytes at
        // (lane % CPR) * 8 elements
        uint32_t const m0 = t.tm * BM + wm * WM + uint32_t(lane / CPR);
        uint32_t const n0 = t.tn * BN + wn * WN + uint32_t(lane % CPR) * VL;
        // C with one mode per side and unit stride along n: a row is a multiple of the
        // leading dimension away (32-bit byte offsets from the tile's first row: a.lin)
        bool const     lin = a.lin != 0;
        uint32_t const ldc_bytes = uint32_t(a.gm.sy[0]) * uint32_t(sizeof(T));
        char* const    c_lin = reinterpret_cast<char*>(C) + int64_t(t.tm * BM + wm * WM) * a.gm.sy[0] * int64_t(sizeof(T));
        uint32_t const v_lin = uint32_t(lane / CPR) * ldc_bytes + n0 * uint32_t(sizeof(T));
        settle();
        // band i: the accumulator tiles of rows 32 i .. 32 i + 31; a tile's lane holds column
        // lane % 16 of the instruction's result, i.e. row lane % 16 of C, and four
        // consecutive n from lane / 16 * 4 on
        static_for<WM / BAND>([&](auto i_tag) ES_INLINE {
            constexpr int i = decltype(i_tag)::value;
            static_for<BAND / MI>([&](auto h_tag) ES_INLINE {
                constexpr int h = decltype(h_tag)::value;
                static_for<TN>([&](auto j_tag) ES_INLINE {
                    constexpr int j = decltype(j_tag)::value;
                    constexpr int R = ((i * (BAND / MI) + h) * TN + j) * 4;
                    quad_t        q;
                    q[0] = T(acc_read<R>() * alpha);
                    q[1] = T(acc_read<R + 1>() * alpha);
                    q[2] = T(acc_read<R + 2>() * alpha);
                    q[3] = T(acc_read<R + 3>() * alpha);
                    acc_clear<R>();
                    acc_clear<R + 1>();
                    acc_clear<R + 2>();
                    acc_clear<R + 3>();
                    int const n = j * MI + (lane / MI) * 4;
                    *reinterpret_cast<quad_t*>(strip + (h * MI + lane % MI) * STRIP_PITCH +
                                               n * int(sizeof(T))) = q;
                });
            });
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            chunk_t v[CPL];
#pragma unroll
            for (int c = 0; c != CPL; ++c) {
                int const idx = c * 64 + lane;
                v[c] = *reinterpret_cast<chunk_t const*>(strip + (idx / CPR) * STRIP_PITCH +
                                                         (idx % CPR) * 16);
            }
#pragma unroll
            for (int c = 0; c != CPL; ++c) {
                uint32_t const m = m0 + uint32_t(i * BAND + c * (64 / CPR));
#ifdef ES_W4_ABL_NO_STORE
                if (m < a.M && n0 < a.N && v[c][0] == 0x12345678u) {
#else
                if (m < a.M && n0 < a.N) {
#endif
                    chunk_t* dst;
                    if (lin) {
                        dst = reinterpret_cast<chunk_t*>(
                            c_lin + (v_lin + uint32_t(i * BAND + c * (64 / CPR)) * ldc_bytes));
                    } else {
                        int64_t mo_a, mo_c, no_b, no_c;
                        group_offsets(a.gm, m, mo_a, mo_c);
                        group_offsets(a.gn, n0, no_b, no_c);
                        dst = reinterpret_cast<chunk_t*>(C + mo_c + no_c);
                    }
                    if (a.c_stream) {
                        store_16_streaming(dst, v[c]);
                    } else {
                        *dst = v[c];
                    }
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        });
    };

    // ---- the walk over this workgroup's tiles.  The loader is NS - 1 slices ahead of the
    // slice being computed and steps once per slice; in the tile's slice nk - NS it steps
    // into the next tile.
    uint32_t const my_tiles = (total_tiles - blockIdx.x + G - 1) / G;
    for (uint32_t it = 0; it != my_tiles; ++it) {
#ifdef ES_W4_STAMP
        uint64_t const stamp0 = __builtin_amdgcn_s_memtime();
#endif
        for (uint32_t kt = 0; kt + 1 < nk; ++kt) {
            head();
            if (kt + NS == nk) next_tile();
            else next_slice();
            tail(std::false_type{});
        }
        head();
        next_slice();
        uint32_t const freed = st;
        tail(std::true_type{});
#ifdef ES_W4_STAMP
        uint64_t const stamp1 = __builtin_amdgcn_s_memtime();
#endif
        epilogue(blockIdx.x + it * G, freed);
#ifdef ES_W4_STAMP
        uint64_t const stamp2 = __builtin_amdgcn_s_memtime();
#endif
        // every wave is done with its strip: the stage can take part 0 of its next slice
        asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
        __builtin_amdgcn_s_barrier();
        static_for<LOADS / PARTS>([&](auto q_tag) ES_INLINE {
            issue(lds_wave + freed * STAGE, q_tag);
        });
#ifdef ES_W4_STAMP
        {
            asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
            if (tid == 0 && it < 8) {
                uint64_t* dst = reinterpret_cast<uint64_t*>(a.ws) + (size_t(blockIdx.x) * 8 + it) * 4;
                dst[0] = stamp0;
                dst[1] = stamp1;
                dst[2] = stamp2;
                dst[3] = stamp0;
            }
        }
#endif
    }
    // nothing may still be on its way into this workgroup's LDS when it ends
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
}

// K in whole slices, at least `NS` of them, every k mode but the innermost a whole number of
// slices apart (the slice walker steps the innermost one), both operands along k.
template <int NS>
inline bool gemm_w4_eligible(gemm_args_t const& a)
{
    return gemm_dma_eligible<_Float16>(a) && a.a_mode == 0 && a.b_mode == 0 && a.splits <= 1 &&
           a.K % BK == 0 && a.K / BK >= uint32_t(NS) && (a.gk.n == 1 || a.gk.size[0] % BK == 0);
}

template <int BM, int BN, int NS, bool KW>
void launch_gemm_w4_kw(gemm_args_t const& a, uint32_t workgroups, hipStream_t stream)
{
    constexpr int lds = NS * (BM + BN) * RB;
    static bool const raised = [] {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_w4_kernel<BM, BN, NS, KW>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        return true;
    }();
    (void)raised;
    uint64_t const total = uint64_t(a.tiles_m) * a.tiles_n * a.batch;
    uint32_t const grid = uint32_t(total < workgroups ? total : workgroups);
    hipLaunchKernelGGL((gemm_w4_kernel<BM, BN, NS, KW>), dim3(grid), dim3(256), lds, stream, a,
                       uint32_t(total));
}

template <int BM, int BN, int NS>
void launch_gemm_w4(gemm_args_t const& a, uint32_t workgroups, hipStream_t stream)
{
    if (a.gk.n == 1) {
        launch_gemm_w4_kw<BM, BN, NS, false>(a, workgroups, stream);
    } else {
        launch_gemm_w4_kw<BM, BN, NS, true>(a, workgroups, stream);
    }
}

}  // namespace w4
}  // namespace gemm
}  // namespace es

