// touch_t kernels for gfx950: N-D copy-region / accumulate (rank <= 4 after simplify) and the
// constant / lower-triangular fills.  These replace touch1..touch4, fill_constant and
// fill_lowerTri of the reference (src/engine/gpu/cuda_kernels.cu:99-515, 579-647) and follow
// the value semantics of the CPU kernels (src/engine/touch.cc:119-135): `+=`, `*=`,
// std::min, std::max in the tensor's own dtype, so results are bit-identical to the CPU path.
//
// Layout: one thread moves one 16-byte vector (or one element when the windows are not
// 16-byte aligned) of the innermost dimension; consecutive lanes take consecutive vectors of
// a row, so every wavefront reads and writes whole 1 KiB row segments.  One vector per thread
// (four per thread, 256 lanes apart, was 2.7 times slower on a 16 MiB copy), its loads issued
// before its store.
#include "launch.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstddef>
#include <cstring>

namespace es
{
namespace
{

constexpr int TOUCH_BLOCK = 256;
constexpr int TOUCH_UNROLL = 1;

struct c64_t {
    float re, im;
};

template <typename T, int N>
struct alignas(sizeof(T) * N) vec_t {
    T v[N];
};

enum : int { OP_COPY = 0, OP_ADD = 1, OP_MUL = 2, OP_MIN = 3, OP_MAX = 4 };

template <int OP, typename T>
__device__ __forceinline__ T touch_op(T out, T inn)
{
#pragma clang fp contract(off)
    if constexpr (OP == OP_COPY) {
        return inn;
    } else if constexpr (OP == OP_ADD) {
        return out + inn;
    } else if constexpr (OP == OP_MUL) {
        return out * inn;
    } else if constexpr (OP == OP_MIN) {
        return (inn < out) ? inn : out;  // std::min(out, inn)
    } else {
        return (out < inn) ? inn : out;  // std::max(out, inn)
    }
}

template <int OP>
__device__ __forceinline__ c64_t touch_op_c64(c64_t out, c64_t inn)
{
#pragma clang fp contract(off)
    if constexpr (OP == OP_ADD) {
        return c64_t{out.re + inn.re, out.im + inn.im};
    } else if constexpr (OP == OP_MUL) {
        float ac = out.re * inn.re, bd = out.im * inn.im;
        float ad = out.re * inn.im, bc = out.im * inn.re;
        return c64_t{ac - bd, ad + bc};
    } else {
        return inn;
    }
}

template <int OP, typename T>
__device__ __forceinline__ T apply(T out, T inn)
{
    if constexpr (sizeof(T) == 8 && alignof(T) == 4) {
        return touch_op_c64<OP>(out, inn);
    } else {
        return touch_op<OP>(out, inn);
    }
}

// T: element type, V: elements per thread-vector
template <typename T, int V, int OP>
__global__ __launch_bounds__(TOUCH_BLOCK) void touch_kernel(touch_launch_t a, T* __restrict__ out,
                                                            T const* __restrict__ inn)
{
    using vt = vec_t<T, V>;
    uint64_t const first = (uint64_t(blockIdx.x) * TOUCH_UNROLL) * TOUCH_BLOCK + threadIdx.x;
    vt             x[TOUCH_UNROLL];
    vt             y[TOUCH_UNROLL];
    uint64_t       oo[TOUCH_UNROLL];
    bool           live[TOUCH_UNROLL];
#pragma unroll
    for (int u = 0; u != TOUCH_UNROLL; ++u) {
        uint64_t idx = first + uint64_t(u) * TOUCH_BLOCK;
        live[u] = idx < a.n_vec;
        if (live[u]) {
            uint64_t oi, ii;
            if (a.outer == 0) {
                // one contiguous row on both sides (what a whole-tensor copy simplifies to):
                // no index decomposition at all
                ii = a.base_inn + idx * V;
                oi = a.base_out + idx * V;
            } else if (a.outer == 1 && a.small) {
                uint32_t const r = uint32_t(idx) / uint32_t(a.vec_per_row);
                uint32_t const c = uint32_t(idx) - r * uint32_t(a.vec_per_row);
                ii = a.base_inn + r * a.str_inn[2] + uint64_t(c) * V;
                oi = a.base_out + r * a.str_out[2] + uint64_t(c) * V;
            } else if (a.small) {
                uint32_t r = uint32_t(idx);
                uint32_t c = r % uint32_t(a.vec_per_row);
                r /= uint32_t(a.vec_per_row);
                uint32_t i2 = r % uint32_t(a.size[2]);
                r /= uint32_t(a.size[2]);
                uint32_t i1 = r % uint32_t(a.size[1]);
                uint32_t i0 = r / uint32_t(a.size[1]);
                ii = a.base_inn + i0 * a.str_inn[0] + i1 * a.str_inn[1] + i2 * a.str_inn[2] +
                     uint64_t(c) * V;
                oi = a.base_out + i0 * a.str_out[0] + i1 * a.str_out[1] + i2 * a.str_out[2] +
                     uint64_t(c) * V;
            } else {
                uint64_t r = idx;
                uint64_t c = r % a.vec_per_row;
                r /= a.vec_per_row;
                uint64_t i2 = r % a.size[2];
                r /= a.size[2];
                uint64_t i1 = r % a.size[1];
                uint64_t i0 = r / a.size[1];
                ii = a.base_inn + i0 * a.str_inn[0] + i1 * a.str_inn[1] + i2 * a.str_inn[2] +
                     c * V;
                oi = a.base_out + i0 * a.str_out[0] + i1 * a.str_out[1] + i2 * a.str_out[2] +
                     c * V;
            }
            oo[u] = oi;
            x[u] = *reinterpret_cast<vt const*>(inn + ii);
            if constexpr (OP != OP_COPY) {
                y[u] = *reinterpret_cast<vt const*>(out + oi);
            }
        }
    }
#pragma unroll
    for (int u = 0; u != TOUCH_UNROLL; ++u) {
        if (live[u]) {
            vt r;
            if constexpr (OP == OP_COPY) {
                r = x[u];
            } else {
#pragma unroll
                for (int j = 0; j != V; ++j) r.v[j] = apply<OP, T>(y[u].v[j], x[u].v[j]);
            }
            *reinterpret_cast<vt*>(out + oo[u]) = r;
        }
    }
}

template <typename T, int V, int OP>
void launch_touch_v(touch_launch_t const& a, hipStream_t stream, void* out, void const* inn)
{
    uint64_t per_block = uint64_t(TOUCH_BLOCK) * TOUCH_UNROLL;
    uint64_t blocks = (a.n_vec + per_block - 1) / per_block;
    hipLaunchKernelGGL((touch_kernel<T, V, OP>), dim3((unsigned)blocks), dim3(TOUCH_BLOCK), 0,
                       stream, a, static_cast<T*>(out), static_cast<T const*>(inn));
}

template <typename T, int OP>
void launch_touch_t(touch_launch_t const& a, hipStream_t stream, void* out, void const* inn)
{
    constexpr int VMAX = 16 / sizeof(T);
    if (a.vec == VMAX) {
        launch_touch_v<T, VMAX, OP>(a, stream, out, inn);
    } else {
        launch_touch_v<T, 1, OP>(a, stream, out, inn);
    }
}

template <typename T>
void launch_touch_op(touch_launch_t const& a, int op, hipStream_t stream, void* out,
                     void const* inn)
{
    switch (op) {
        case OP_ADD:
            return launch_touch_t<T, OP_ADD>(a, stream, out, inn);
        case OP_MUL:
            return launch_touch_t<T, OP_MUL>(a, stream, out, inn);
        case OP_MIN:
            return launch_touch_t<T, OP_MIN>(a, stream, out, inn);
        case OP_MAX:
            return launch_touch_t<T, OP_MAX>(a, stream, out, inn);
    }
}

// ---- touches with pairwise disjoint windows, one per blockIdx.y

template <typename T>
__device__ __forceinline__ T apply_dyn(int op, T out, T inn)
{
    switch (op) {
        case OP_COPY:
            return inn;
        case OP_ADD:
            return apply<OP_ADD, T>(out, inn);
        case OP_MUL:
            return apply<OP_MUL, T>(out, inn);
        case OP_MIN:
            if constexpr (!(sizeof(T) == 8 && alignof(T) == 4)) return apply<OP_MIN, T>(out, inn);
            return inn;
        default:
            if constexpr (!(sizeof(T) == 8 && alignof(T) == 4)) return apply<OP_MAX, T>(out, inn);
            return inn;
    }
}

constexpr int TOUCH_LIST_BLOCK = TOUCH_LIST_BLOCK_HOST;
constexpr int TOUCH_LIST_WAVES = 4;  // wavefronts (row pieces) per workgroup

// ---- a list of touches folded by the owner of each output vector
//
// One wavefront = 64 consecutive output vectors of one row of the bounding box (a workgroup's
// wavefronts take consecutive rows).  Lane t tests whether item t reaches the wavefront (at most 64 items per launch), the
// ballot is the wavefront's list, and the items on it are folded in list order; everything
// about an item except the lane's own column is uniform and sits in one wide scalar load.
// What this replaces, on 64 accumulating windows of 512 x 512 at odd offsets of a 4096 x 4096
// f16 output: the same fold unrolled over 32 items per launch (the code outgrew the
// instruction cache: 2 x 77 us), a scalar walk over all items (several dependent scalar loads
// each: 189 us), workgroups of 256 (seven items each on average, one latency chain after the
// other: 48 us).  The wavefronts are short-lived and execute some six hundred instructions
// each, so the kernel is bound by instruction issue as much as by memory: folding two items
// per round instead of four (a wavefront meets one or two) took that case from 32 to 29 us,
// compiling the items' op and load path in (UOP) to 22 us; several rows per wavefront or
// more wavefronts per workgroup changed nothing.
//
// R4: items keep four dimensions (16 words); otherwise two (12 words; leading extents are 1).
// Words of an item, ND = 4 or 2: input pointer (2), base_inn (2), lo[ND], size[ND],
// str_inn[ND - 1], op | vec_rows << 8 | shift << 16.
//
// UOP: -1, or every item of the launch has this op and takes its input as shifted whole
// vectors (the usual case -- all of a tensor's partial blocks are added or copied, from
// buffers with aligned rows): the per-item choices are then made by the compiler.
template <typename T, int V, bool R4, int UOP>
__global__ __launch_bounds__(TOUCH_LIST_BLOCK* TOUCH_LIST_WAVES) void touch_list_kernel(
    touch_list_t b, T* __restrict__ out, uint32_t n_rows)
{
    static_assert(UOP < 0 || V * sizeof(T) == 16, "");
    using vt = vec_t<T, V>;
    constexpr int ND = R4 ? 4 : 2;
    constexpr int WI = R4 ? 16 : 12;
    uint32_t const lane = threadIdx.x % TOUCH_LIST_BLOCK;
    uint32_t       row = blockIdx.x / b.chunks_per_row;
    uint32_t const chunk = blockIdx.x - row * b.chunks_per_row;
    row = row * TOUCH_LIST_WAVES + threadIdx.x / TOUCH_LIST_BLOCK;
    if (row >= n_rows) return;
    uint32_t       u[3] = {0, 0, 0};  // the row's coordinates, right-aligned
    uint64_t       row_off = 0;
    if constexpr (R4) {
#pragma unroll
        for (int s = 2; s >= 0; --s) {
            uint32_t const q = row / b.box_size[s];
            u[s] = b.box_lo[s] + (row - q * b.box_size[s]);
            row = q;
            row_off += u[s] * b.out_str[s];
        }
    } else {
        u[2] = b.box_lo[2] + row;
        row_off = u[2] * b.out_str[2];
    }
    uint32_t const box_hi3 = b.box_lo[3] + b.box_size[3];
    uint32_t const col_lo = b.box_lo[3] + chunk * uint32_t(TOUCH_LIST_BLOCK) * V;
    uint32_t const col_hi =
        col_lo + uint32_t(TOUCH_LIST_BLOCK) * V < box_hi3 ? col_lo + uint32_t(TOUCH_LIST_BLOCK) * V : box_hi3;
    uint32_t const c3 = col_lo + lane * V;
    bool const     live = c3 < box_hi3;
    uint64_t const oo = row_off + c3;
    // The item table is read through the kernel-argument pointer (`b` is the first argument):
    // a run-time index into the by-value struct invites the compiler to copy the argument
    // block into private memory first.
    typedef uint32_t const __attribute__((address_space(4))) const_word_t;
    typedef char const __attribute__((address_space(4))) const_byte_t;
    const_word_t* const table = (const_word_t*)((const_byte_t*)__builtin_amdgcn_kernarg_segment_ptr() +
                                                offsetof(touch_list_t, w));
    // Where the windows cover most of the bounding box the old value is asked for before the
    // wavefront knows whether a window reaches it (the test is a round trip to the item table)
    vt val;
    if (b.eager && live) val = *reinterpret_cast<vt const*>(out + oo);
    uint64_t todo;
    {
        // every word is loaded before the first comparison (a test that stops at the first
        // miss waits for one load after the other)
        uint32_t const      t = lane;
        const_word_t* const it = table + (t < b.n ? t : 0u) * WI;
        uint32_t            lo[ND], sz[ND];
#pragma unroll
        for (int d = 0; d != ND; ++d) {
            lo[d] = it[4 + d];
            sz[d] = it[4 + ND + d];
        }
        bool hit = (t < b.n) & (col_lo < lo[ND - 1] + sz[ND - 1]) & (col_hi > lo[ND - 1]);
#pragma unroll
        for (int d = 0; d != ND - 1; ++d) hit = hit & (u[3 - (ND - 1) + d] - lo[d] < sz[d]);
        todo = __ballot(hit);
    }
    if (todo == 0) return;
    // otherwise the old value is on its way while the first item's words arrive; lanes that
    // no window reaches never store
    if (!b.eager && live) val = *reinterpret_cast<vt const*>(out + oo);
    bool have = false;
    // K items at a time: the words of all K, then the input vectors of all K, are under way
    // before the first one is folded in -- one item after the other, each a chain of a scalar
    // load, two vector loads and the update, a wavefront lived 14 k cycles for two items
    constexpr int K = 2;
    while (todo) {
        uint32_t w[K][WI];
        bool     valid[K];
#pragma unroll
        for (int k = 0; k != K; ++k) {
            valid[k] = todo != 0;
            uint32_t const t = valid[k] ? uint32_t(__builtin_ctzll(todo)) : 0u;
            if (valid[k]) todo &= todo - 1;
            const_word_t* const it = table + t * WI;
#pragma unroll
            for (int i = 0; i != WI; ++i) w[k][i] = it[i];
        }
        uint32_t d[K][8];
        uint32_t j_lo[K], j_hi[K];
        bool     covered[K];
        T const* elems[K];  // scalar path: the lane's first element
#pragma unroll
        for (int k = 0; k != K; ++k) {
            uint32_t const lo3 = w[k][4 + ND - 1], sz3 = w[k][4 + 2 * ND - 1];
            uint64_t       src_row = uint64_t(w[k][2]) | (uint64_t(w[k][3]) << 32);
#pragma unroll
            for (int dd = 0; dd != ND - 1; ++dd) {
                src_row += uint64_t(u[3 - (ND - 1) + dd] - w[k][4 + dd]) * w[k][4 + 2 * ND + dd];
            }
            covered[k] = valid[k] && live && c3 < lo3 + sz3 && c3 + V > lo3;
            // elements j_lo .. j_hi of this vector lie inside the window
            j_lo[k] = c3 >= lo3 ? 0u : lo3 - c3;
            j_hi[k] = c3 + V <= lo3 + sz3 ? uint32_t(V - 1) : lo3 + sz3 - 1 - c3;
            uint32_t const flags = w[k][4 + 3 * ND - 1];
            T const* const src =
                reinterpret_cast<T const*>(uint64_t(w[k][0]) | (uint64_t(w[k][1]) << 32)) + src_row;
            elems[k] = src + (int64_t(c3) - int64_t(lo3));
#pragma unroll
            for (int i = 0; i != 8; ++i) d[k][i] = 0;
            if constexpr (V * sizeof(T) == 16) {
                if (covered[k] && (UOP >= 0 || (flags & 0x100))) {
                    // The input's rows are 16-byte aligned but the window sits `sh` elements
                    // off the output's vector grid: the vector's elements come out of two
                    // aligned input vectors, shifted by a whole number of bytes that is the
                    // same for the whole item.  Neither vector is loaded unless one of its
                    // elements is needed: an aligned 16-byte load that holds a valid element
                    // cannot leave its page.
                    uint32_t const sh = (flags >> 16) & 0xf;
                    T const* const p0 = elems[k] - int64_t(sh);
                    if (j_lo[k] + sh < uint32_t(V)) {
                        vec_t<uint32_t, 4> const v0 = *reinterpret_cast<vec_t<uint32_t, 4> const*>(p0);
#pragma unroll
                        for (int i = 0; i != 4; ++i) d[k][i] = v0.v[i];
                    }
                    if (j_hi[k] + sh >= uint32_t(V)) {
                        vec_t<uint32_t, 4> const v1 =
                            *reinterpret_cast<vec_t<uint32_t, 4> const*>(p0 + V);
#pragma unroll
                        for (int i = 0; i != 4; ++i) d[k][4 + i] = v1.v[i];
                    }
                }
            }
        }
#pragma unroll
        for (int k = 0; k != K; ++k) {
            if (!covered[k]) continue;
            uint32_t const flags = w[k][4 + 3 * ND - 1];
            int const      op = UOP >= 0 ? UOP : int(flags & 0xff);
            bool const     full = j_lo[k] == 0 && j_hi[k] == uint32_t(V - 1);
            vt             x;
            bool           by_vector = false;
            if constexpr (V * sizeof(T) == 16) by_vector = UOP >= 0 || (flags & 0x100) != 0;
            if (by_vector) {
                uint32_t const bytes = ((flags >> 16) & 0xf) * uint32_t(sizeof(T));
                uint32_t const q = bytes >> 2, r = bytes & 3;
                uint32_t       o[4];
                switch (q) {  // uniform
                    case 0:
#pragma unroll
                        for (int i = 0; i != 4; ++i) o[i] = __builtin_amdgcn_alignbyte(d[k][i + 1], d[k][i], r);
                        break;
                    case 1:
#pragma unroll
                        for (int i = 0; i != 4; ++i) o[i] = __builtin_amdgcn_alignbyte(d[k][i + 2], d[k][i + 1], r);
                        break;
                    case 2:
#pragma unroll
                        for (int i = 0; i != 4; ++i) o[i] = __builtin_amdgcn_alignbyte(d[k][i + 3], d[k][i + 2], r);
                        break;
                    default:
#pragma unroll
                        for (int i = 0; i != 4; ++i) o[i] = __builtin_amdgcn_alignbyte(d[k][i + 4], d[k][i + 3], r);
                        break;
                }
                vec_t<uint32_t, 4> ov;
#pragma unroll
                for (int i = 0; i != 4; ++i) ov.v[i] = o[i];
                if constexpr (V * sizeof(T) == 16) x = __builtin_bit_cast(vt, ov);
            } else {
#pragma unroll
                for (int j = 0; j != V; ++j) {
                    if (uint32_t(j) >= j_lo[k] && uint32_t(j) <= j_hi[k]) x.v[j] = elems[k][j];
                }
            }
            have = true;
            if (full) {
                switch (op) {  // uniform
                    case OP_COPY:
                        val = x;
                        break;
                    case OP_ADD:
#pragma unroll
                        for (int j = 0; j != V; ++j) val.v[j] = apply_dyn<T>(OP_ADD, val.v[j], x.v[j]);
                        break;
                    default:
#pragma unroll
                        for (int j = 0; j != V; ++j) val.v[j] = apply_dyn<T>(op, val.v[j], x.v[j]);
                        break;
                }
            } else {
#pragma unroll
                for (int j = 0; j != V; ++j) {
                    if (uint32_t(j) >= j_lo[k] && uint32_t(j) <= j_hi[k]) {
                        val.v[j] = apply_dyn<T>(op, val.v[j], x.v[j]);
                    }
                }
            }
        }
    }
    if (have) *reinterpret_cast<vt*>(out + oo) = val;
}

template <typename T>
void launch_touch_list_t(touch_list_t const& b, hipStream_t stream, void* out)
{
    constexpr int VMAX = 16 / sizeof(T);
    dim3 const    block(TOUCH_LIST_BLOCK * TOUCH_LIST_WAVES);
    T* const      o = static_cast<T*>(out);
    bool const    r4 = b.rank > 2;
    // (the planner bounds rows x chunks of the bounding box)
    uint64_t const rows = uint64_t(b.box_size[0]) * b.box_size[1] * b.box_size[2];
    uint64_t const row_groups = (rows + TOUCH_LIST_WAVES - 1) / TOUCH_LIST_WAVES;
    dim3 const     grid(unsigned(row_groups * b.chunks_per_row));
    uint32_t const n_rows = uint32_t(rows);
    if (int(b.vec) == VMAX) {
        if (r4) {
            hipLaunchKernelGGL((touch_list_kernel<T, VMAX, true, -1>), grid, block, 0, stream, b, o,
                               n_rows);
        } else if (b.uniform_op == OP_ADD + 1) {
            hipLaunchKernelGGL((touch_list_kernel<T, VMAX, false, OP_ADD>), grid, block, 0, stream, b,
                               o, n_rows);
        } else if (b.uniform_op == OP_COPY + 1) {
            hipLaunchKernelGGL((touch_list_kernel<T, VMAX, false, OP_COPY>), grid, block, 0, stream,
                               b, o, n_rows);
        } else {
            hipLaunchKernelGGL((touch_list_kernel<T, VMAX, false, -1>), grid, block, 0, stream, b, o,
                               n_rows);
        }
    } else if (r4) {
        hipLaunchKernelGGL((touch_list_kernel<T, 1, true, -1>), grid, block, 0, stream, b, o, n_rows);
    } else {
        hipLaunchKernelGGL((touch_list_kernel<T, 1, false, -1>), grid, block, 0, stream, b, o, n_rows);
    }
}

template <typename T, int V>
__global__ __launch_bounds__(256) void touch_level_kernel(touch_level_t b, T* __restrict__ out)
{
    using vt = vec_t<T, V>;
    touch_item_t const& it = b.items[blockIdx.y];  // uniform index: scalar loads
    uint32_t const lo3 = it.lo[3], sz3 = it.size[3];
    // the output vectors that the window's rows overlap
    uint32_t const v_first = lo3 / V;
    uint32_t const vpr = (lo3 + sz3 - 1) / V - v_first + 1;
    uint64_t const n_vec = uint64_t(it.size[0]) * it.size[1] * it.size[2] * vpr;
    uint64_t const idx = uint64_t(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= n_vec) return;
    uint64_t       r = idx / vpr;
    uint32_t const c3 = (v_first + uint32_t(idx - r * vpr)) * V;
    uint32_t const d2 = uint32_t(r % it.size[2]);
    r /= it.size[2];
    uint32_t const d1 = uint32_t(r % it.size[1]);
    uint32_t const d0 = uint32_t(r / it.size[1]);
    uint64_t const oo = (it.lo[0] + d0) * b.out_str[0] + (it.lo[1] + d1) * b.out_str[1] +
                        (it.lo[2] + d2) * b.out_str[2] + c3;
    T const* const src = static_cast<T const*>(it.inn) + it.base_inn + d0 * it.str_inn[0] +
                         d1 * it.str_inn[1] + d2 * it.str_inn[2];
    int const  op = it.op;
    bool const full = c3 >= lo3 && c3 + V <= lo3 + sz3;
    if (full) {
        vt x;
        if (it.vec_inn) {
            x = *reinterpret_cast<vt const*>(src + (c3 - lo3));
        } else {
#pragma unroll
            for (int j = 0; j != V; ++j) x.v[j] = src[c3 - lo3 + uint32_t(j)];
        }
        if (op != OP_COPY) {
            vt const y = *reinterpret_cast<vt const*>(out + oo);
#pragma unroll
            for (int j = 0; j != V; ++j) x.v[j] = apply_dyn<T>(op, y.v[j], x.v[j]);
        }
        *reinterpret_cast<vt*>(out + oo) = x;
    } else {
#pragma unroll
        for (int j = 0; j != V; ++j) {
            uint32_t const d3 = c3 + uint32_t(j) - lo3;  // wraps below the window
            if (d3 < sz3) {
                T const x = src[d3];
                out[oo + j] = op == OP_COPY ? x : apply_dyn<T>(op, out[oo + j], x);
            }
        }
    }
}

template <typename T>
void launch_touch_level_t(touch_level_t const& b, hipStream_t stream, void* out)
{
    constexpr int VMAX = 16 / sizeof(T);
    dim3          grid(unsigned((b.max_vec + 255) / 256), unsigned(b.n));
    if (b.vec == VMAX) {
        hipLaunchKernelGGL((touch_level_kernel<T, VMAX>), grid, dim3(256), 0, stream, b,
                           static_cast<T*>(out));
    } else {
        hipLaunchKernelGGL((touch_level_kernel<T, 1>), grid, dim3(256), 0, stream, b,
                           static_cast<T*>(out));
    }
}

// ---- fills

template <int V>
__global__ __launch_bounds__(256) void fill_constant_kernel(uint64_t n_vec, vec_t<uint32_t, V> pat,
                                                            vec_t<uint32_t, V>* __restrict__ out)
{
    // one vector per thread; fills larger than the caches bypass them
    uint64_t const i = uint64_t(blockIdx.x) * 256 + threadIdx.x;
    if (i >= n_vec) return;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    static_assert(V == 4, "16-byte pattern");
    u32x4 const v = {pat.v[0], pat.v[1], pat.v[2], pat.v[3]};
    if (n_vec >= (4u << 20)) {
        // as an instruction: the optimiser merges a hinted and a plain store of the same
        // value in the two arms of a branch into one plain store
        asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 1"
                     :
                     : "v"(reinterpret_cast<u32x4*>(out) + i), "v"(v)
                     : "memory");
    } else {
        reinterpret_cast<u32x4*>(out)[i] = v;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void fill_tail_kernel(uint64_t begin, uint64_t end, T value,
                                                        T* __restrict__ out)
{
    uint64_t i = begin + uint64_t(blockIdx.x) * 256 + threadIdx.x;
    if (i < end) out[i] = value;
}

// out[r, c] = (r - start >= c) ? lower : upper, signed r - start
// (src/einsummable/fill.h:17-19); one thread writes V consecutive columns.
template <typename T, int V>
__global__ __launch_bounds__(256) void fill_lowertri_kernel(uint64_t nrow, uint64_t ncol,
                                                            int64_t start, T lower, T upper,
                                                            T* __restrict__ out)
{
    uint64_t vec_per_row = ncol / V;
    uint64_t n_vec = nrow * vec_per_row;
    uint64_t i = uint64_t(blockIdx.x) * 256 + threadIdx.x;
    uint64_t stride = uint64_t(gridDim.x) * 256;
    for (; i < n_vec; i += stride) {
        uint64_t  r = i / vec_per_row;
        uint64_t  c0 = (i % vec_per_row) * V;
        int64_t   edge = int64_t(r) - start;  // columns <= edge take `lower`
        vec_t<T, V> v;
#pragma unroll
        for (int j = 0; j != V; ++j) v.v[j] = (edge >= int64_t(c0 + j)) ? lower : upper;
        *reinterpret_cast<vec_t<T, V>*>(out + r * ncol + c0) = v;
    }
}

template <typename T>
void launch_lowertri(uint64_t nrow, uint64_t ncol, int64_t start, uint64_t lower_bits,
                     uint64_t upper_bits, hipStream_t stream, void* out)
{
    T lower, upper;
    std::memcpy(&lower, &lower_bits, sizeof(T));
    std::memcpy(&upper, &upper_bits, sizeof(T));
    constexpr int VMAX = 16 / sizeof(T);
    bool          wide = (ncol % VMAX == 0) && (reinterpret_cast<uintptr_t>(out) % 16 == 0);
    uint64_t      n_vec = wide ? nrow * (ncol / VMAX) : nrow * ncol;
    unsigned      blocks = (unsigned)std::min<uint64_t>((n_vec + 255) / 256, 65536);
    if (blocks == 0) return;
    if (wide) {
        hipLaunchKernelGGL((fill_lowertri_kernel<T, VMAX>), dim3(blocks), dim3(256), 0, stream,
                           nrow, ncol, start, lower, upper, static_cast<T*>(out));
    } else {
        hipLaunchKernelGGL((fill_lowertri_kernel<T, 1>), dim3(blocks), dim3(256), 0, stream, nrow,
                           ncol, start, lower, upper, static_cast<T*>(out));
    }
}

}  // namespace

void launch_touch(touch_launch_t const& a, int elem_size, int dtype_code, int op,
                  hipStream_t stream, void* out, void const* inn)
{
    if (a.n_vec == 0) return;
    if (op == OP_COPY) {
        // copies only depend on the element width
        switch (elem_size) {
            case 2:
                return launch_touch_t<uint16_t, OP_COPY>(a, stream, out, inn);
            case 4:
                return launch_touch_t<uint32_t, OP_COPY>(a, stream, out, inn);
            default:
                return launch_touch_t<uint64_t, OP_COPY>(a, stream, out, inn);
        }
    }
    switch (dtype_code) {
        case 0:
            return launch_touch_op<_Float16>(a, op, stream, out, inn);
        case 1:
            return launch_touch_op<float>(a, op, stream, out, inn);
        case 2:
            return launch_touch_op<double>(a, op, stream, out, inn);
        default:
            if (op == OP_ADD) return launch_touch_t<c64_t, OP_ADD>(a, stream, out, inn);
            return launch_touch_t<c64_t, OP_MUL>(a, stream, out, inn);
    }
}

void launch_touch_list(touch_list_t const& b, int elem_size, int dtype_code, bool any_castable,
                       hipStream_t stream, void* out)
{
    if (b.n == 0 || b.box_size[3] == 0) return;
    if (!any_castable) {
        switch (elem_size) {
            case 2:
                return launch_touch_list_t<uint16_t>(b, stream, out);
            case 4:
                return launch_touch_list_t<uint32_t>(b, stream, out);
            default:
                return launch_touch_list_t<uint64_t>(b, stream, out);
        }
    }
    switch (dtype_code) {
        case 0:
            return launch_touch_list_t<_Float16>(b, stream, out);
        case 1:
            return launch_touch_list_t<float>(b, stream, out);
        case 2:
            return launch_touch_list_t<double>(b, stream, out);
        default:
            return launch_touch_list_t<c64_t>(b, stream, out);
    }
}

void launch_touch_level(touch_level_t const& b, int elem_size, int dtype_code, bool any_castable,
                        hipStream_t stream, void* out)
{
    if (b.n == 0 || b.max_vec == 0) return;
    if (!any_castable) {
        switch (elem_size) {
            case 2:
                return launch_touch_level_t<uint16_t>(b, stream, out);
            case 4:
                return launch_touch_level_t<uint32_t>(b, stream, out);
            default:
                return launch_touch_level_t<uint64_t>(b, stream, out);
        }
    }
    switch (dtype_code) {
        case 0:
            return launch_touch_level_t<_Float16>(b, stream, out);
        case 1:
            return launch_touch_level_t<float>(b, stream, out);
        case 2:
            return launch_touch_level_t<double>(b, stream, out);
        default:
            return launch_touch_level_t<c64_t>(b, stream, out);
    }
}

void launch_fill_constant(int elem_size, uint64_t bits, uint64_t nelem, hipStream_t stream,
                          void* out)
{
    if (nelem == 0) return;
    // replicate the element into a 16-byte pattern
    vec_t<uint32_t, 4> pat;
    unsigned char      raw[16];
    for (int i = 0; i < 16; i += elem_size) std::memcpy(raw + i, &bits, size_t(elem_size));
    std::memcpy(&pat, raw, 16);
    uint64_t  bytes = nelem * uint64_t(elem_size);
    uintptr_t p = reinterpret_cast<uintptr_t>(out);
    uint64_t  head_bytes = (16 - (p % 16)) % 16;  // multiple of elem_size: out is element aligned
    if (head_bytes > bytes) head_bytes = bytes;
    uint64_t body_vec = (bytes - head_bytes) / 16;
    uint64_t tail_begin = (head_bytes + body_vec * 16) / uint64_t(elem_size);
    auto     edge = [&](uint64_t b, uint64_t e) {
        if (b == e) return;
        unsigned blocks = unsigned((e - b + 255) / 256);
        if (elem_size == 2) {
            hipLaunchKernelGGL((fill_tail_kernel<uint16_t>), dim3(blocks), dim3(256), 0, stream, b,
                               e, uint16_t(bits), static_cast<uint16_t*>(out));
        } else if (elem_size == 4) {
            hipLaunchKernelGGL((fill_tail_kernel<uint32_t>), dim3(blocks), dim3(256), 0, stream, b,
                               e, uint32_t(bits), static_cast<uint32_t*>(out));
        } else {
            hipLaunchKernelGGL((fill_tail_kernel<uint64_t>), dim3(blocks), dim3(256), 0, stream, b,
                               e, bits, static_cast<uint64_t*>(out));
        }
    };
    edge(0, head_bytes / uint64_t(elem_size));
    if (body_vec) {
        if (body_vec >= (1ull << 39)) return;  // beyond any device memory
        unsigned blocks = unsigned((body_vec + 255) / 256);
        hipLaunchKernelGGL((fill_constant_kernel<4>), dim3(blocks), dim3(256), 0, stream, body_vec,
                           pat,
                           reinterpret_cast<vec_t<uint32_t, 4>*>(static_cast<char*>(out) +
                                                                  head_bytes));
    }
    edge(tail_begin, nelem);
}

void launch_fill_lowertri(int elem_size, uint64_t lower_bits, uint64_t upper_bits, uint64_t nrow,
                          uint64_t ncol, int64_t start, hipStream_t stream, void* out)
{
    switch (elem_size) {
        case 2:
            return launch_lowertri<uint16_t>(nrow, ncol, start, lower_bits, upper_bits, stream,
                                             out);
        case 4:
            return launch_lowertri<uint32_t>(nrow, ncol, start, lower_bits, upper_bits, stream,
                                             out);
        default:
            return launch_lowertri<uint64_t>(nrow, ncol, start, lower_bits, upper_bits, stream,
                                             out);
    }
}

}  // namespace es
