// N-D permute whose innermost mode changes (a true transposition), through LDS tiles.
//
// A permutation einsummable (one input, identity join, no aggregation, no broadcast;
// einsummable_t::is_permutation, src/einsummable/einsummable.cc:740-743) that keeps its
// innermost mode is a strided row copy and is handled by the generated elementwise kernel.
// When the innermost mode of the input is not the innermost mode of the output, a direct
// copy is uncoalesced on one side.  Here a tile over (input-inner mode, output-inner mode),
// 64 x 64 up to 256 x 64 elements, goes through LDS: rows are read along the input's contiguous mode and written along
// the output's contiguous mode, so both sides move whole 128..512-byte row segments.  All
// other modes form the batch.  Pure data movement: results are bit-identical to the CPU's
// permute_t (src/base/permute_.h) and to the interpreter.
#include "kernel_manager.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdlib>
#include <string>

namespace es
{
namespace
{

constexpr int TT = 64;      // tile edge
constexpr int MAXB = 6;     // batch modes

struct transpose_args_t {
    void const* in;
    void*       out;
    uint32_t    n_i, n_o;           // extents of the input-inner and output-inner modes
    int64_t     so_i;               // output stride of the input-inner mode
    int64_t     si_o;               // input stride of the output-inner mode
    uint32_t    tiles_i, tiles_o;
    uint64_t    n_blocks;
    uint32_t    nb;                 // number of batch modes
    uint32_t    plain_stores;       // results go through the L2 instead of streaming past it
    // 0: tiles in launch order, input-inner mode first (consecutive workgroups land on
    // different XCDs); 1: every XCD takes one contiguous run of that order, so that the
    // neighbours along a row share an L2; 2: the same with the output-inner mode first
    uint32_t    order;
    uint32_t    bsize[MAXB];        // innermost batch mode first
    int64_t     bsi[MAXB], bso[MAXB];
};

// Tile origin and batch offsets of a workgroup; false when the workgroup has no tile.
template <int EDGE, int EDGE_O = EDGE>
__device__ __forceinline__ bool locate(transpose_args_t const& a, uint32_t& i0, uint32_t& o0,
                                       int64_t& off_i, int64_t& off_o)
{
    uint64_t linear = uint64_t(blockIdx.y) * gridDim.x + blockIdx.x;
    if (linear >= a.n_blocks) return false;  // uniform over the workgroup
    if (a.order) {
        uint64_t const per = a.n_blocks / 8;
        if (linear < per * 8) linear = (linear % 8) * per + linear / 8;
    }
    uint32_t t = uint32_t(linear);
    uint32_t ti, to;
    if (a.order == 2) {
        to = t % a.tiles_o;
        t /= a.tiles_o;
        ti = t % a.tiles_i;
        t /= a.tiles_i;
    } else {
        ti = t % a.tiles_i;
        t /= a.tiles_i;
        to = t % a.tiles_o;
        t /= a.tiles_o;
    }
    uint32_t bidx = t;
    off_i = 0;
    off_o = 0;
#pragma unroll
    for (int d = 0; d != MAXB; ++d) {
        if (d < int(a.nb)) {
            uint32_t q = bidx / a.bsize[d];
            uint32_t r = bidx - q * a.bsize[d];
            off_i += int64_t(r) * a.bsi[d];
            off_o += int64_t(r) * a.bso[d];
            bidx = q;
        }
    }
    i0 = ti * EDGE;
    o0 = to * EDGE_O;
    return true;
}

// The same tile with 16-byte global accesses on both sides: a lane loads V = 16 / sizeof(T)
// consecutive elements of an input row and, after the turn through LDS, stores V consecutive
// elements of an output row.  Needs every row start on both sides 16-byte aligned (strides,
// batch offsets, extents and base pointers: checked on the host).
// The tile is TI elements of the input-inner mode by TO elements of the output-inner mode;
// vec_shape() picks it.
template <typename T, int TI, int TO>
__global__ __launch_bounds__(256) void transpose_vec_kernel(transpose_args_t a)
{
    constexpr int V = 16 / int(sizeof(T));
    constexpr int LPR = TI / V;      // lanes per tile row on the way in
    constexpr int RPP = 256 / LPR;   // tile rows per pass of the workgroup
    constexpr int LPR_O = TO / V;    // the same on the way out
    constexpr int RPP_O = 256 / LPR_O;
    // pitch: an odd number of 4-byte words, so that a column walks over all banks
    constexpr int PITCH = sizeof(T) == 2 ? TI + 2 : TI + 1;
    typedef T vecT __attribute__((ext_vector_type(V)));
    __shared__ T tile[TO * PITCH];

    uint32_t i0, o0;
    int64_t  off_i, off_o;
    if (!locate<TI, TO>(a, i0, o0, off_i, off_o)) return;
    T const* const in = static_cast<T const*>(a.in) + off_i;
    T* const       out = static_cast<T*>(a.out) + off_o;
    {
        uint32_t const col = (threadIdx.x % LPR) * V;
        uint32_t const row = threadIdx.x / LPR;
#pragma unroll
        for (int p = 0; p != TO / RPP; ++p) {
            uint32_t const ol = row + p * RPP;
            uint32_t const o = o0 + ol, i = i0 + col;
            if (o < a.n_o && i < a.n_i) {  // n_i is a multiple of V: a started vector is whole
                vecT v = __builtin_nontemporal_load(
                    reinterpret_cast<vecT const*>(in + int64_t(o) * a.si_o + i));
                if constexpr (sizeof(T) == 2) {
                    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
                    u32x4 w = __builtin_bit_cast(u32x4, v);
                    uint32_t* dst = reinterpret_cast<uint32_t*>(&tile[ol * PITCH + col]);
#pragma unroll
                    for (int j = 0; j != 4; ++j) dst[j] = w[j];
                } else {
#pragma unroll
                    for (int j = 0; j != V; ++j) tile[ol * PITCH + col + j] = v[j];
                }
            }
        }
    }
    __syncthreads();
    {
        uint32_t const col = (threadIdx.x % LPR_O) * V;
        uint32_t const row = threadIdx.x / LPR_O;
#pragma unroll
        for (int p = 0; p != TI / RPP_O; ++p) {
            uint32_t const il = row + p * RPP_O;
            uint32_t const i = i0 + il, o = o0 + col;
            if (i < a.n_i && o < a.n_o) {
                vecT v;
#pragma unroll
                for (int j = 0; j != V; ++j) v[j] = tile[(col + j) * PITCH + il];
                vecT* d = reinterpret_cast<vecT*>(out + int64_t(i) * a.so_i + o);
                // written in assembly: with a plain store in the other arm the compiler merges
                // the two and drops the streaming hint
                if (a.plain_stores) {
                    *d = v;
                } else {
                    asm volatile("global_store_dwordx4 %0, %1, off nt" : : "v"(d), "v"(v) : "memory");
                }
            }
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(transpose_args_t a)
{
    // pitch chosen odd in 4-byte words so that the column reads spread over all banks
    constexpr int PITCH = sizeof(T) == 2 ? TT + 2 : TT + 1;
    __shared__ T tile[TT][PITCH];

    uint32_t const lane = threadIdx.x & 63;
    uint32_t const wave = threadIdx.x >> 6;
    uint64_t const linear = uint64_t(blockIdx.y) * gridDim.x + blockIdx.x;
    if (linear >= a.n_blocks) return;  // uniform over the workgroup
    uint32_t t = uint32_t(linear);
    uint32_t const ti = t % a.tiles_i;
    t /= a.tiles_i;
    uint32_t const to = t % a.tiles_o;
    uint32_t bidx = t / a.tiles_o;

    int64_t off_i = 0, off_o = 0;
#pragma unroll
    for (int d = 0; d != MAXB; ++d) {
        if (d < int(a.nb)) {
            uint32_t q = bidx / a.bsize[d];
            uint32_t r = bidx - q * a.bsize[d];
            off_i += int64_t(r) * a.bsi[d];
            off_o += int64_t(r) * a.bso[d];
            bidx = q;
        }
    }
    T const* const in = static_cast<T const*>(a.in) + off_i;
    T* const       out = static_cast<T*>(a.out) + off_o;
    uint32_t const i0 = ti * TT, o0 = to * TT;

    // rows of the tile along the input's contiguous mode
#pragma unroll
    for (int rr = 0; rr != TT / 4; ++rr) {
        uint32_t o = o0 + wave * (TT / 4) + rr;
        uint32_t i = i0 + lane;
        if (o < a.n_o && i < a.n_i) tile[wave * (TT / 4) + rr][lane] = in[int64_t(o) * a.si_o + i];
    }
    __syncthreads();
#pragma unroll
    for (int rr = 0; rr != TT / 4; ++rr) {
        uint32_t i = i0 + wave * (TT / 4) + rr;
        uint32_t o = o0 + lane;
        if (i < a.n_i && o < a.n_o) out[int64_t(i) * a.so_i + o] = tile[lane][wave * (TT / 4) + rr];
    }
}

// Tile of the 16-byte kernel, measured on 4096..16384-square matrices with cold and with warm
// caches.  4-byte elements: 512-byte segments on the way in and 256-byte segments on the way
// out beat the square tile by 4..12 % once there are enough tiles to fill the device.
// 2-byte elements: the long tile pays once each XCD works on one contiguous run of tiles
// (8192 x 8192: 51.4 us square in launch order, 48.2 us long in runs; 16384 x 16384: 228 us
// against 213 us long, in runs, output-inner mode first); 4-byte elements gain nothing from
// the runs (91 us either way).
inline void vec_shape(int elem_size, uint32_t n_i, uint32_t n_o, uint64_t batch, uint32_t& edge_i,
                      uint32_t& edge_o, uint32_t& order)
{
    uint64_t const bytes = 2ull * n_i * n_o * batch * uint64_t(elem_size);
    const char*    env = std::getenv("ES_KM_TRANSPOSE_TILE");  // tuning and tests
    bool const     force_square = env && std::string(env) == "square";
    bool const     force_long = env && std::string(env) == "long";
    edge_i = edge_o = 64;
    order = 0;
    if (elem_size == 2) {
        edge_i = edge_o = 128;
        if (!force_square && (force_long || (bytes >= (128ull << 20) && n_i >= 256))) {
            edge_i = 256;
            edge_o = 64;
            order = bytes >= (1ull << 30) ? 2 : 1;
        }
    } else if (elem_size == 4) {
        uint64_t const tiles = uint64_t((n_i + 127) / 128) * ((n_o + 63) / 64) * batch;
        if (!force_square && (force_long || tiles >= 2048)) edge_i = 128;
    }
}

struct transpose_plan_t : plan_t {
    transpose_args_t args;
    int              elem_size;
    uint64_t         batch;
    bool             vec_ok;  // extents, strides and batch offsets keep rows 16-byte aligned
    bool             order_forced = false;

    void run(hipStream_t stream, void* out, void const* const* inns, void*, uint64_t) const override
    {
        transpose_args_t a = args;
        a.in = inns[0];
        a.out = out;
        bool const aligned = reinterpret_cast<uintptr_t>(a.in) % 16 == 0 &&
                             reinterpret_cast<uintptr_t>(a.out) % 16 == 0;
        bool const vec = vec_ok && aligned;
        uint32_t edge_i = 64, edge_o = 64;
        if (vec) {
            uint32_t order = 0;
            vec_shape(elem_size, a.n_i, a.n_o, batch, edge_i, edge_o, order);
            if (!order_forced) a.order = order;
        }
        a.tiles_i = (a.n_i + edge_i - 1) / edge_i;
        a.tiles_o = (a.n_o + edge_o - 1) / edge_o;
        uint64_t const blocks = uint64_t(a.tiles_i) * a.tiles_o * batch;
        a.n_blocks = blocks;
        // a grid dimension times the block size must stay below 2^32
        unsigned gx = unsigned(std::min<uint64_t>(blocks, 1ull << 22));
        unsigned gy = unsigned((blocks + gx - 1) / gx);
        dim3     grid(gx, gy), block(256);
        if (vec) {
            if (elem_size == 2 && edge_i == 256) {
                hipLaunchKernelGGL((transpose_vec_kernel<uint16_t, 256, 64>), grid, block, 0, stream, a);
            } else if (elem_size == 2) {
                hipLaunchKernelGGL((transpose_vec_kernel<uint16_t, 128, 128>), grid, block, 0, stream, a);
            } else if (elem_size == 4 && edge_i == 128) {
                hipLaunchKernelGGL((transpose_vec_kernel<uint32_t, 128, 64>), grid, block, 0, stream, a);
            } else if (elem_size == 4) {
                hipLaunchKernelGGL((transpose_vec_kernel<uint32_t, 64, 64>), grid, block, 0, stream, a);
            } else {
                hipLaunchKernelGGL((transpose_vec_kernel<uint64_t, 64, 64>), grid, block, 0, stream, a);
            }
        } else {
            switch (elem_size) {
                case 2:
                    hipLaunchKernelGGL((transpose_kernel<uint16_t>), grid, block, 0, stream, a);
                    break;
                case 4:
                    hipLaunchKernelGGL((transpose_kernel<uint32_t>), grid, block, 0, stream, a);
                    break;
                default:
                    hipLaunchKernelGGL((transpose_kernel<uint64_t>), grid, block, 0, stream, a);
                    break;
            }
        }
        hipError_t err = hipGetLastError();
        if (err != hipSuccess) {
            throw km_error(km_status::device,
                           std::string("transpose launch: ") + hipGetErrorString(err));
        }
    }
};

}  // namespace

std::shared_ptr<plan_t> plan_transpose(einsummable_t const& e, int)
{
    if (!e.is_permutation()) return nullptr;
    int const R = e.out_rank;
    if (R < 2) return nullptr;
    std::vector<int> const& inn = e.inns[0];
    int const mode_i = inn.back();  // contiguous in the input
    int const mode_o = R - 1;       // contiguous in the output
    if (mode_i == mode_o) return nullptr;  // inner mode preserved: a row copy, not a transpose
    if (R - 2 > MAXB) return nullptr;

    auto in_stride = [&](int m) {
        int64_t s = 1;
        for (int k = int(inn.size()) - 1; k >= 0; --k) {
            if (inn[k] == m) return s;
            s *= int64_t(e.join_shape[inn[k]]);
        }
        return int64_t(0);
    };
    auto out_stride = [&](int m) {
        int64_t s = 1;
        for (int k = R - 1; k > m; --k) s *= int64_t(e.join_shape[k]);
        return s;
    };
    if (e.out_nelem() >= (1ull << 40)) return nullptr;
    for (uint64_t d : e.join_shape) {
        if (d >= (1ull << 31)) return nullptr;
    }

    auto p = std::make_shared<transpose_plan_t>();
    transpose_args_t& a = p->args;
    a.in = nullptr;
    a.out = nullptr;
    a.n_i = uint32_t(e.join_shape[mode_i]);
    a.n_o = uint32_t(e.join_shape[mode_o]);
    a.so_i = out_stride(mode_i);
    a.si_o = in_stride(mode_o);
    a.tiles_i = (a.n_i + TT - 1) / TT;
    a.tiles_o = (a.n_o + TT - 1) / TT;
    a.nb = 0;
    uint64_t batch = 1;
    for (int d = 0; d != MAXB; ++d) {
        a.bsize[d] = 1;
        a.bsi[d] = a.bso[d] = 0;
    }
    for (int m = R - 1; m >= 0; --m) {
        if (m == mode_i || m == mode_o) continue;
        a.bsize[a.nb] = uint32_t(e.join_shape[m]);
        a.bsi[a.nb] = in_stride(m);
        a.bso[a.nb] = out_stride(m);
        batch *= e.join_shape[m];
        ++a.nb;
    }
    p->batch = batch;
    if (uint64_t(a.tiles_i) * a.tiles_o * batch >= (1ull << 31) || batch >= (1ull << 31)) {
        return nullptr;
    }
    p->elem_size = int(dtype_size(e.out_dtype()));
    {
        int64_t const V = 16 / p->elem_size;
        bool ok = a.n_i % V == 0 && a.n_o % V == 0 && a.si_o % V == 0 && a.so_i % V == 0;
        for (uint32_t d = 0; d != a.nb; ++d) ok = ok && a.bsi[d] % V == 0 && a.bso[d] % V == 0;
        p->vec_ok = ok;
    }
    // Streaming stores send each 128..256-byte segment to the memory by itself; through the
    // L2 the segments that neighbouring tiles write to the same rows leave together.  Kernel
    // durations, 8192 x 8192: 2-byte elements 61 -> 50 us, 4-byte elements 137 -> 95 us;
    // 16384 x 16384: 262 -> 230 us and 512 -> 474 us.  Small transposes, whose result stays
    // in the L2 anyway, are faster streaming (4096 x 4096 2-byte: 11.6 against 14.5 us).
    a.plain_stores = 2 * e.out_nelem() * uint64_t(p->elem_size) >= (128ull << 20);
    if (const char* env = std::getenv("ES_KM_TRANSPOSE_STORES")) {  // tuning and tests
        a.plain_stores = std::string(env) == "cached";
    }
    a.order = 0;
    p->workspace_bytes = 0;
    uint32_t edge_i = 64, edge_o = 64;
    if (p->vec_ok) vec_shape(p->elem_size, a.n_i, a.n_o, batch, edge_i, edge_o, a.order);
    if (const char* env = std::getenv("ES_KM_TRANSPOSE_ORDER")) {  // tuning and tests
        a.order = uint32_t(std::atoi(env)) % 3;
        p->order_forced = true;
    }
    p->description = "transpose_lds tile=" + std::to_string(edge_i) + "x" + std::to_string(edge_o) +
                     (p->vec_ok ? " vec16" : "") + (a.plain_stores ? " cached_stores" : "") +
                     (a.order == 1 ? " xcd_runs" : a.order == 2 ? " xcd_runs_out_first" : "") +
                     " batch=" + std::to_string(batch);
    return p;
}

}  // namespace es
