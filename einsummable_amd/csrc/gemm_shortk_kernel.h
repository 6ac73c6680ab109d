// fp16 contractions with a reduction of exactly 128 elements (attention scores: K is the head
// dimension) and many output tiles.  Such a product does 256 flop per output byte pair and is
// bound by writing C; a tile has only eight matrix-instruction steps of work, so a kernel
// that starts a workgroup per tile spends its time in set-up, in waiting for the first
// operands and in an epilogue that nothing overlaps.  Here a workgroup keeps 128 rows of A
// in registers and walks along n, one row of tiles after another, for the whole launch:
//
//   * waves 4 and 5 only load: 128 x 128 tiles of B go from global memory straight into a
//     ring of LDS buffers (global_load_lds_dwordx4; 256-byte rows whose sixteen 16-byte
//     chunks are XOR-swizzled with the row number so that fragment reads are free of bank
//     conflicts), each wave half a tile, one tile ahead of the multiplication; they wait
//     until the next tile has landed and join the workgroup barrier;
//   * waves 0..3 (2 x 2, 64 x 64 each) multiply the current B buffer with their A
//     fragments.  Converting a tile (reading 64 accumulators, scaling, packing to fp16,
//     writing an LDS staging tile) is over a hundred vector instructions of four cycles
//     each, as long as half of the tile's 32 matrix instructions; a wave that does one after
//     the other loses a third of the matrix rate.  So a wave converts one half of its
//     accumulators between the matrix instructions of the other half (a matrix instruction
//     runs for 32 cycles, in which the wave issues up to eight other instructions);
//   * waves 6 and 7 only store: they read the staging tile of the step before as whole
//     256-byte row segments and write them to C.  A store instruction stalls its wave until
//     the memory pipeline takes it; on these waves that costs nothing, while the same
//     stall on a multiplying wave (measured: the time to write C simply added to the time
//     of everything else) keeps the matrix cores and the loads idle.
//
// A staging tile has rows of 256 bytes without padding; the 16-byte chunk c of row m lies at
// chunk c ^ (m % 16) and its two 8-byte halves are exchanged when bit 3 of m is set.  With
// that the multiplying waves' 8-byte writes (32 rows per instruction) and the storing waves'
// 16-byte reads (four whole rows per instruction) are both free of bank conflicts; rows
// padded by 16 bytes cost every one of those instructions four extra cycles
// (SQ_LDS_BANK_CONFLICT: 1.1 conflict cycles per active LDS cycle of the whole kernel).
//
// One workgroup barrier per tile orders the three roles: a B buffer is refilled after
// everyone has read it, a staging tile is rewritten after it has been read out.  Step g of a
// workgroup's stream of tiles multiplies tile g, stages tile g - 1 and stores tile g - 2; one
// more step at the end stages the last tile, and the storing waves store it after the last
// barrier.
//
// What bounds it (measured, 128 heads of 2048 x 2048): C is written as 256-byte pieces of
// rows that lie 4 KiB apart; a kernel that does nothing but those stores, from two waves per
// compute unit, writes 5.2 TB/s (whole 1 KiB pieces: 5.6; torch's fill of the same GiB: 6.9).
// Under this kernel's mix of matrix work and memory traffic the device clock settles near
// 1.25 GHz, and a step then takes the multiplying waves about as long as the stores.
#pragma once
#include "gemm_w4_kernel.h"

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
constexpr int SK_OUT_PITCH = SK_BN * 2;           // staging row: 128 outputs, chunks swizzled
constexpr int SK_OUT = SK_BM * SK_OUT_PITCH;      // one staging tile
constexpr int SK_LDS = SK_NBUF * SK_BUF + 2 * SK_OUT + 512;  // + scratch of the prefetches
constexpr int SK_PF_DIST = 4;                     // tiles the L2 prefetch runs ahead
constexpr int SK_PF_LOADS = 2;                    // 128-byte lines per row of B
constexpr int SK_THREADS = 512;                   // 4 multiplying, 2 loading, 2 storing waves

// 16 bytes from `p + OFF` into the registers of `dst` (the compiler sees a statement that
// updates dst, not a load: it keeps dst where it is)
template <int OFF>
__device__ __forceinline__ void sk_load_in_place(chunk_t& dst, void const* p)
{
    asm volatile("global_load_dwordx4 %0, %1, off offset:%2" : "+v"(dst) : "v"(p), "n"(OFF) : "memory");
}
template <uint32_t C>
__device__ __forceinline__ uint32_t sk_xor(uint32_t x)
{
    uint32_t r;
    asm volatile("v_xor_b32 %0, %1, %2" : "=v"(r) : "n"(C), "v"(x));
    return r;
}
// waits for every load of the wave; what reads x afterwards is ordered behind the wait
__device__ __forceinline__ void sk_await_loads(chunk_t (&x)[8])
{
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "+v"(x[4]), "+v"(x[5]),
                   "+v"(x[6]), "+v"(x[7])
                 :
                 : "memory");
}

// SCALE: the products are multiplied by a.alpha (else a.alpha is 1).
//
// The grid is one workgroup per compute unit (a multiple of 8: workgroup b runs on XCD b % 8).
// A walk is `tiles_per_block` tiles of one row of tiles; the walks of a batch entry share B,
// so XCD x takes the consecutive walks [x * per_xcd, (x + 1) * per_xcd), its workgroups in
// turn.  A workgroup's tiles, walk after walk, form one stream: the roles run through it
// without a pause between walks (only the multiplying waves fetch new rows of A).
template <bool SCALE>
__global__ __launch_bounds__(SK_THREADS) void gemm_shortk_kernel(gemm_args_t a,
                                                                 uint32_t tiles_per_block,
                                                                 uint32_t chunks_n,
                                                                 uint32_t total_walks)
{
    using T = _Float16;
    using tr = traits_t<T>;
    using namespace w4;
    using std::integral_constant;
    extern __shared__ __attribute__((aligned(16))) char lds[];
    uint32_t const lds_base = uint32_t(uintptr_t((__attribute__((address_space(3))) char*)lds));

    int const tid = threadIdx.x;
    int const lane = tid & 63;
    int const wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    uint32_t const per_batch = a.tiles_m * chunks_n;
    uint32_t const per_xcd = (total_walks + 7) / 8;
    uint32_t const in_turn = gridDim.x / 8;  // workgroups of an XCD
    uint32_t const xcd_first = (blockIdx.x % 8) * per_xcd;
    uint32_t const lda = uint32_t(a.gm.sx[0]), ldb = uint32_t(a.gn.sx[0]);
    uint32_t const ldc = uint32_t(a.gm.sy[0]);

    // a position in this workgroup's stream of tiles
    struct cursor_t {
        uint32_t local;  // the walk's number within the XCD's range
        uint32_t tm, t;  // row of tiles, tile along n
        uint32_t t0, cnt, i;  // the walk's first tile and length, the step within the walk
        int64_t  boa, bob, boc;
        bool     valid;
    };
    auto seek = [&](cursor_t& c, uint32_t local) ES_INLINE {
        c.local = local;
        uint32_t const id = xcd_first + local;
        c.valid = local < per_xcd && id < total_walks;
        if (!c.valid) return;
        uint32_t const bz = id / per_batch;
        uint32_t const rem = id - bz * per_batch;
        uint32_t const chunk = rem / a.tiles_m;
        c.tm = rem - chunk * a.tiles_m;
        c.t0 = chunk * tiles_per_block;
        c.cnt = (c.t0 + tiles_per_block < a.tiles_n ? c.t0 + tiles_per_block : a.tiles_n) - c.t0;
        // Workgroups that run side by side start their walks at different columns and wrap
        // round.  Walking in step from the same column they would all write, at any moment,
        // the same 256 bytes of every row of C (a row is a few KiB), and those addresses
        // share few memory channels.
        c.i = 0;
        c.t = c.t0 + id % c.cnt;
        group_offsets(a.gb, bz, c.boa, c.bob);
        if (a.gb.n == 1) {
            c.boc = int64_t(bz) * a.gb.sz[0];
        } else {
            c.boc = 0;
            uint32_t i = bz;
#pragma unroll
            for (int d = 0; d != MAXG; ++d) {
                uint32_t q = i / a.gb.size[d];
                c.boc += int64_t(i - q * a.gb.size[d]) * a.gb.sz[d];
                i = q;
            }
        }
    };
    // to the next tile; true when that is the first of another walk
    auto advance = [&](cursor_t& c) ES_INLINE {
        if (++c.i != c.cnt) {
            c.t = c.t + 1 == c.t0 + c.cnt ? c.t0 : c.t + 1;
            return false;
        }
        seek(c, c.local + in_turn);
        return true;
    };
    // tiles in this workgroup's stream
    uint32_t steps = 0;
    {
        cursor_t c;
        for (seek(c, blockIdx.x / 8); c.valid; seek(c, c.local + in_turn)) steps += c.cnt;
    }
    if (steps == 0) return;
    auto uniform_ptr = [](T const* p) ES_INLINE {
        uint64_t const v = reinterpret_cast<uint64_t>(p);
        // (the builtin returns a signed int: widen each half as unsigned)
        uint32_t const lo = uint32_t(__builtin_amdgcn_readfirstlane(uint32_t(v)));
        uint32_t const hi = uint32_t(__builtin_amdgcn_readfirstlane(uint32_t(v >> 32)));
        return reinterpret_cast<T const*>((uint64_t(hi) << 32) | lo);
    };

    if (wave == 4 || wave == 5) {
        // ---- the loading waves.  Load instruction q of a tile covers rows 4 q + lane / 16
        // (wave 4: q < 16, wave 5: the rest); the lane's LDS slot (lane % 16) receives
        // global chunk slot ^ (row % 16).
        uint32_t const lr = uint32_t(lane) >> 4, slot = uint32_t(lane) & 15;
        int const      half = wave - 4;
        constexpr int  PER_WAVE = SK_BN / 4 / 2;  // load instructions per tile per wave
        uint32_t const pf_scratch = lds_base + SK_NBUF * SK_BUF + 2 * SK_OUT + uint32_t(half) * 256;
        auto tile_loads = [&](cursor_t const& c, uint32_t buf) ES_INLINE {
            uint32_t const n0 = c.t * SK_BN;
            uint32_t const last = a.N - 1 - n0;  // rows past the end re-read the last one
            // the base goes into a scalar register pair of the load instructions
            T const* const base =
                uniform_ptr(static_cast<T const*>(a.B) + c.bob + int64_t(n0) * ldb);
#pragma unroll
            for (int q0 = 0; q0 != PER_WAVE; ++q0) {
                uint32_t const q = uint32_t(half * PER_WAVE + q0);
                uint32_t const row = 4 * q + lr;
                uint32_t const src = row < last ? row : last;
                uint32_t const voff = src * ldb * 2 + ((slot ^ (row & 15)) << 4);
                load_to_lds_16(base, voff, lds_base + buf * SK_BUF + q * 1024);
            }
        };
        // Brings 128 rows of 256 bytes (a tile of B, the rows of A of a walk) into the L2 only:
        // one dword per 128-byte line into a scratch corner of LDS that nobody reads.  What is
        // needed next must not wait for HBM: with C being written at full speed a read that
        // misses the L2 takes microseconds, and the lookahead of the buffer ring is one tile.
        auto prefetch_rows = [&](T const* first_row, uint32_t ld, uint32_t rows_left) ES_INLINE {
            T const* const base = uniform_ptr(first_row);
            uint32_t const row = uint32_t(half) * 64 + uint32_t(lane);
            uint32_t const src = row < rows_left ? row : rows_left - 1;
#pragma unroll
            for (int u = 0; u != SK_PF_LOADS; ++u) {
                load_to_lds_4(base, src * ld * 2 + uint32_t(u) * 128, pf_scratch);
            }
        };
        // the tile the prefetch cursor stands on (and, at the start of a walk, its rows of A);
        // returns the number of load instructions issued
        auto prefetch = [&](cursor_t const& c, bool walk_start) ES_INLINE {
            uint32_t const n0 = c.t * SK_BN;
            prefetch_rows(static_cast<T const*>(a.B) + c.bob + int64_t(n0) * ldb, ldb, a.N - n0);
            if (!walk_start) return uint32_t(SK_PF_LOADS);
            uint32_t const m_first = c.tm * SK_BM;
            prefetch_rows(static_cast<T const*>(a.A) + c.boa + int64_t(m_first) * lda, lda,
                          a.M - m_first);
            return uint32_t(2 * SK_PF_LOADS);
        };
        // waits until at most `younger` loads (0, 2, 4, ...) are outstanding
        auto wait_but = [](uint32_t younger) ES_INLINE {
            switch (younger / SK_PF_LOADS) {
                case 0: wait_loads_and_lds<0>(); break;
                case 1: wait_loads_and_lds<1 * SK_PF_LOADS>(); break;
                case 2: wait_loads_and_lds<2 * SK_PF_LOADS>(); break;
                case 3: wait_loads_and_lds<3 * SK_PF_LOADS>(); break;
                case 4: wait_loads_and_lds<4 * SK_PF_LOADS>(); break;
                case 5: wait_loads_and_lds<5 * SK_PF_LOADS>(); break;
                case 6: wait_loads_and_lds<6 * SK_PF_LOADS>(); break;
                case 7: wait_loads_and_lds<7 * SK_PF_LOADS>(); break;
                default: wait_loads_and_lds<8 * SK_PF_LOADS>(); break;
            }
        };
        cursor_t ld, pf;  // the next tile to load, the next tile to prefetch
        seek(ld, blockIdx.x / 8);
        pf = ld;
        tile_loads(ld, 0);
        advance(ld);
        uint32_t ahead = 0;  // prefetch instructions younger than the tile loads
        bool     pf_start = advance(pf);
        for (int d = 0; d != SK_PF_DIST && pf.valid; ++d) {
            ahead += prefetch(pf, pf_start);
            pf_start = advance(pf);
        }
        static_assert(SK_PF_DIST <= 4, "wait_but() counts up to 8 pairs");
        wait_but(ahead);  // the tile has landed; the prefetches behind it may be in flight
        __builtin_amdgcn_s_barrier();
        for (uint32_t g = 0; g != steps; ++g) {
            // the buffer of tile g + 1 is the one tile g - 1 was read from
            if (g + 1 < steps) {
                tile_loads(ld, (g + 1) % SK_NBUF);
                advance(ld);
                uint32_t younger = 0;
                if (pf.valid) {
                    younger = prefetch(pf, pf_start);
                    pf_start = advance(pf);
                }
                wait_but(younger);
            }
            __builtin_amdgcn_s_barrier();
        }
        __builtin_amdgcn_s_barrier();  // the last tile is staged
        return;
    }

    if (wave >= 6) {
        // ---- the storing waves: rows 64 (wave - 6) .. + 63 of every tile; instruction c
        // covers rows 4 c + lane / 16 with 16 lanes per 256-byte row segment
        int const      half = wave - 6;
        uint32_t const lr = uint32_t(lane) >> 4, lch = uint32_t(lane) & 15;
        uint32_t const lane_off = (lr * ldc + lch * 8) * 2;
        // instruction c reads rows 4 c + lr: chunk lch of such a row lies at lch ^ (4 (c % 4) + lr)
        int const      lds_row = int(uint32_t(half) * 64 + lr) * SK_OUT_PITCH;
        int            lds_chunk[4];
#pragma unroll
        for (int k = 0; k != 4; ++k) lds_chunk[k] = int((lch ^ (4 * uint32_t(k) + lr)) * 16);
        constexpr int  NST = 16;
        cursor_t       sc;
        seek(sc, blockIdx.x / 8);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_s_barrier();  // the first tile is multiplied
        for (uint32_t g = 0; g != steps; ++g) {
            __builtin_amdgcn_s_barrier();  // tile g is staged
            char const* const out = lds + SK_NBUF * SK_BUF + (g & 1) * SK_OUT + lds_row;
            uint32_t const    n0 = sc.t * SK_BN;
            uint32_t const    mrow = sc.tm * SK_BM + uint32_t(half) * 64;  // first row of this wave
            chunk_t           v[NST];
#pragma unroll
            for (int c = 0; c != NST; ++c) {
                chunk_t const x =
                    *reinterpret_cast<chunk_t const*>(out + c * 4 * SK_OUT_PITCH + lds_chunk[c % 4]);
                // (bit 3 of the row 4 c + lr is bit 1 of c)
                v[c] = (c & 2) ? chunk_t{x[2], x[3], x[0], x[1]} : x;
            }
            char* const corner =
                reinterpret_cast<char*>(static_cast<T*>(a.C) + sc.boc + int64_t(mrow) * ldc + n0);
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
            advance(sc);
        }
        return;
    }

    // ---- the multiplying waves
    int const   wm = wave >> 1, wn = wave & 1;
    float const alpha = float(a.alpha);
    // A fragments: tile row i, k-step s: row lane % 32, k chunk 2 s + lane / 32.  They are
    // loaded by instructions the compiler does not see as loads, into the registers that hold
    // the fragments of the walk before: a load that is a branch of the step loop would
    // otherwise get 64 registers of its own.  (The matrix instructions that read the old
    // fragments were issued before; a load returns hundreds of cycles after they have read
    // their operands.)
    chunk_t fa[2][8];
    auto    load_a = [&](cursor_t const& c) ES_INLINE {
        T const* const A = static_cast<T const*>(a.A) + c.boa;
        uint32_t const m0 = c.tm * SK_BM + uint32_t(wm) * 64;
        static_for<2>([&](auto i_tag) ES_INLINE {
            constexpr int i = decltype(i_tag)::value;
            uint32_t      r = m0 + uint32_t(i * 32 + lane % 32);
            r = r < a.M ? r : a.M - 1;
            T const* const row = A + int64_t(r) * lda + (lane / 32) * 8;
            static_for<8>([&](auto s_tag) ES_INLINE {
                constexpr int s = decltype(s_tag)::value;
                sk_load_in_place<s * 32>(fa[i][s], row);
            });
        });
    };
    // the fragments have arrived (these waves have no other loads in flight)
    auto await_a = [&]() ES_INLINE {
        sk_await_loads(fa[0]);
        sk_await_loads(fa[1]);
    };
    // B fragments: tile row j * 32 + lane % 32 of this wave's half, chunk 2 s + lane / 32 in
    // slot chunk ^ (row % 16); row % 16 is lane % 16 for every j.  The byte offset of row and
    // slot is fb_lane ^ (s << 5) (+ 32 rows for j = 1): the row's offset is a multiple of 256,
    // the slot's 16 (2 s ^ lane / 32 ^ lane % 16).
    uint32_t const fb_lane = uint32_t((wn * 64 + lane % 32) * SK_RB) |
                             uint32_t(((lane / 32) ^ (lane & 15)) << 4);
    uint32_t fb_at[8];  // the k-steps' offsets in the B buffer of the current step

    // A step works through the wave's 64 x 64 in two halves along n (j = 0, 1), 16 matrix
    // instructions each, and converts one half while it multiplies the other:
    //   first half:  j = 0 of tile g;  between the instructions, j = 1 of tile g - 1 is packed
    //                and written to the staging tile, and so is the packed j = 0 of g - 1;
    //   second half: j = 1 of tile g;  j = 0 of tile g is packed and kept in registers.
    // So the whole staging tile of g - 1 is written during step g, as the barriers expect, and
    // every accumulator is free again when its half comes round: 64 accumulators, not 128.
    // acc[j][i]: a lane holds row lane % 32 of tile row i and, per register quad e0 .. e0 + 3,
    // the four consecutive n from j * 32 + (e0 / 4) * 8 + (lane / 32) * 4 on.
    tr::acc_t acc[2][2];
    uint32_t  packed[16];  // j = 0: quad q = 4 i + e0 / 4 in packed[2 q], packed[2 q + 1]
    chunk_t   fb[4];  // the fragment of k-step n of a step's 16 in fb[n % 4], read three ahead
    typedef T half2_t __attribute__((ext_vector_type(2)));
    // half quad h (0 .. 15) of half j: two accumulators, scaled and packed
    auto pack = [&](auto j_tag, auto h_tag) ES_INLINE {
        constexpr int j = decltype(j_tag)::value, h = decltype(h_tag)::value;
        constexpr int q = h / 2, i = q / 4, e = (q % 4) * 4 + (h % 2) * 2;
        float x0 = acc[j][i][e], x1 = acc[j][i][e + 1];
        if constexpr (SCALE) {
            x0 *= alpha;
            x1 *= alpha;
        }
        half2_t v;
        v[0] = T(x0);
        v[1] = T(x1);
        return __builtin_bit_cast(uint32_t, v);
    };
    // quad q of half j of the staging tile at `stage`
    // (the lane's row is wm * 64 + i * 32 + lane % 32: its low four bits are the lane's; the
    // quad's byte column wn * 128 + j * 64 + (q % 4) * 16 + (lane / 32) * 8 goes through the
    // row's swizzle, which is an XOR with a value of the lane)
    uint32_t const stage_swz = (uint32_t(wn) * 128 + uint32_t(lane / 32) * 8) ^
                               ((uint32_t(lane) & 15) << 4) ^ (((uint32_t(lane) >> 3) & 1) << 3);
    uint32_t stage_at[8];  // j * 4 + q % 4 -> the quad's address in the current staging tile, row i = 0
    auto stage_quad = [&](auto j_tag, auto q_tag, uint32_t lo, uint32_t hi) ES_INLINE {
        constexpr int j = decltype(j_tag)::value, q = decltype(q_tag)::value;
        typedef uint32_t pair_t __attribute__((ext_vector_type(2)));
        typedef __attribute__((address_space(3))) pair_t* lds_pair_ptr;
        pair_t v;
        v[0] = lo;
        v[1] = hi;
        *(lds_pair_ptr)(uintptr_t)(stage_at[j * 4 + q % 4] + (q / 4) * 32 * SK_OUT_PITCH) = v;
    };
    uint32_t const stage_row = lds_base + SK_NBUF * SK_BUF + uint32_t(wm * 64 + lane % 32) * SK_OUT_PITCH;
    auto stage_into = [&](uint32_t parity) ES_INLINE {
#pragma unroll
        for (int k = 0; k != 8; ++k) {
            stage_at[k] = stage_row + parity * SK_OUT + (uint32_t((k / 4) * 64 + (k % 4) * 16) ^ stage_swz);
        }
    };
    uint32_t    held = 0;
    // One step on the tile in B buffer `par`; with PREV, the staging tile of the tile before
    // (the other parity) is written.
    auto multiply = [&](uint32_t par, auto prev_tag) ES_INLINE {
        constexpr bool PREV = decltype(prev_tag)::value;
        static_assert(SK_BUF == 1 << 15 && SK_NBUF == 2, "");
#pragma unroll
        for (int s = 0; s != 8; ++s) {
            fb_at[s] = lds_base + ((fb_lane ^ uint32_t(s << 5)) | (par << 15));
        }
        typedef __attribute__((address_space(3))) chunk_t const* lds_chunk_ptr;
        if constexpr (PREV) stage_into(par ^ 1);
        fb[0] = *(lds_chunk_ptr)(uintptr_t)(fb_at[0]);
        fb[1] = *(lds_chunk_ptr)(uintptr_t)(fb_at[1]);
        fb[2] = *(lds_chunk_ptr)(uintptr_t)(fb_at[2]);
        static_for<2>([&](auto j_tag) ES_INLINE {
            constexpr int j = decltype(j_tag)::value;
            static_for<8>([&](auto s_tag) ES_INLINE {
                constexpr int s = decltype(s_tag)::value;
                constexpr int n = j * 8 + s;
                static_for<2>([&](auto i_tag) ES_INLINE {
                    constexpr int i = decltype(i_tag)::value;
                    constexpr int h = s * 2 + i;  // 0 .. 15 within the half
                    if constexpr (s == 0) {
                        tr::acc_t zero;
#pragma unroll
                        for (int e = 0; e != tr::NACC; ++e) zero[e] = 0;
                        acc[j][i] = zero;
                    }
                    tr::mma(acc[j][i], fb[n % 4], fa[i][s]);
                    if constexpr (i == 0 && n + 3 < 16) {
                        constexpr int s2 = (n + 3) % 8, j2 = (n + 3) / 8;
                        fb[(n + 3) % 4] = *(lds_chunk_ptr)(uintptr_t)(fb_at[s2] + j2 * 32 * SK_RB);
                    }
                    if constexpr (j == 0 && PREV) {
                        // j = 1 of the tile before, and its packed j = 0
                        uint32_t const w = pack(integral_constant<int, 1>{}, integral_constant<int, h>{});
                        if constexpr (h % 2 == 0) {
                            held = w;
                            stage_quad(integral_constant<int, 0>{}, integral_constant<int, h / 2>{},
                                       packed[h], packed[h + 1]);
                        } else {
                            stage_quad(integral_constant<int, 1>{}, integral_constant<int, h / 2>{},
                                       held, w);
                        }
                    }
                    if constexpr (j == 1) {
                        packed[h] = pack(integral_constant<int, 0>{}, integral_constant<int, h>{});
                    }
                    __builtin_amdgcn_sched_barrier(0);
                });
            });
        });
    };

    cursor_t mc;
    seek(mc, blockIdx.x / 8);
#pragma unroll
    for (int i = 0; i != 2; ++i) {
#pragma unroll
        for (int s = 0; s != 8; ++s) fa[i][s] = chunk_t{0, 0, 0, 0};
    }
    load_a(mc);
    __builtin_amdgcn_s_barrier();
    for (uint32_t g = 0; g != steps; ++g) {
        await_a();
        if (g == 0) {
            multiply(0u, std::false_type{});
        } else {
            multiply(g & 1, std::true_type{});
        }
        // the rows of A of the next walk: asked for behind the walk's last matrix instruction
        if (advance(mc) && mc.valid) load_a(mc);
        // the staged tile is complete, and this B buffer read, before the barrier says so
        asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
        __builtin_amdgcn_s_barrier();
    }
    // the last tile
    {
        stage_into((steps - 1) & 1);
        static_for<16>([&](auto h_tag) ES_INLINE {
            constexpr int  h = decltype(h_tag)::value;
            uint32_t const w = pack(integral_constant<int, 1>{}, h_tag);
            if constexpr (h % 2 == 0) {
                held = w;
                stage_quad(integral_constant<int, 0>{}, integral_constant<int, h / 2>{}, packed[h],
                           packed[h + 1]);
            } else {
                stage_quad(integral_constant<int, 1>{}, integral_constant<int, h / 2>{}, held, w);
            }
        });
    }
    asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
    __builtin_amdgcn_s_barrier();
}

// Tiles along n of one walk, or 0 when the kernel that takes a workgroup per tile is the
// better choice.  Measured on b x s x s x 128 products, each launch after a fill that
// empties the caches, time of the per-tile kernel / time of this one, walks of 16 tiles:
// 1.15-1.23 for 2048 walks (128 x 2048, 32 x 4096) and 2 x 8192, 1.06-1.13 for 512 and 256
// walks (32 x 2048, 8 x 4096, 4 x 4096, 32 x 1024), 0.98-1.00 for 16 x 2048 and 64 x 1024;
// with fewer walks than compute units 0.95 (8 x 2048).
inline uint32_t shortk_walk(gemm_args_t const& a)
{
    uint64_t const tiles_m = (a.M + SK_BM - 1) / SK_BM, tiles_n = (a.N + SK_BN - 1) / SK_BN;
    if (tiles_n < 8 || tiles_m * tiles_n * a.batch >= (1ull << 31)) return 0;
    const char*    env = std::getenv("ES_KM_GEMM_RESIDENT_MIN");  // tuning and tests
    uint64_t const min_walks = uint64_t(env ? std::max(1, std::atoi(env)) : 256);
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
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_shortk_kernel<false>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, SK_LDS);
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_shortk_kernel<true>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, SK_LDS);
        return true;
    }();
    (void)raised;
    uint32_t const walks = a.tiles_m * chunks * a.batch;
    // one workgroup per compute unit, a multiple of 8 (workgroup b runs on XCD b % 8)
    uint32_t cus = a.workgroups ? a.workgroups : 256;
    if (const char* env = std::getenv("ES_KM_GEMM_RESIDENT_GRID")) {  // tuning and tests
        cus = uint32_t(std::max(1, std::atoi(env)));
    }
    dim3 grid(cus < 8 ? 8 : cus / 8 * 8);
    if (float(a.alpha) == 1.0f) {
        hipLaunchKernelGGL(gemm_shortk_kernel<false>, grid, dim3(SK_THREADS), SK_LDS, stream, a, tpb,
                           chunks, walks);
    } else {
        hipLaunchKernelGGL(gemm_shortk_kernel<true>, grid, dim3(SK_THREADS), SK_LDS, stream, a, tpb,
                           chunks, walks);
    }
}

}  // namespace gemm
}  // namespace es
