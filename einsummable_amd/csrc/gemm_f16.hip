// fp16-in / fp32-accumulate instantiations of the MFMA GEMM kernel.
#include "gemm_dma_kernel.h"
#include "gemm_kernel.h"
#include "gemm_pc_kernel.h"
#include "gemm_shortk_kernel.h"

namespace es
{
namespace gemm
{

__global__ __launch_bounds__(256) void gemm_warm_kernel(chunk_t const* p, uint64_t n_chunks,
                                                        chunk_t const* q, uint64_t n_chunks_q,
                                                        uint32_t* sink)
{
    // 16 bytes per lane, four grid strides per thread, first over p, then over q; what is read
    // is folded into a word that is stored only to a sink nobody passes, which keeps the loads
    // alive
    uint64_t const stride = uint64_t(gridDim.x) * 256;
    uint64_t const total = n_chunks + n_chunks_q;
    uint64_t       i = uint64_t(blockIdx.x) * 256 + threadIdx.x;
    uint32_t       acc = 0;
#pragma unroll
    for (int r = 0; r != 4; ++r, i += stride) {
        if (i < total) {
            chunk_t const v = i < n_chunks ? p[i] : q[i - n_chunks];
            acc ^= v[0] ^ v[1] ^ v[2] ^ v[3];
        }
    }
    if (sink && acc == 0x9e3779b9u) *sink = acc;
}

// Reads both operands (either may be empty) into the memory-side cache with one launch.
void gemm_warm_operands(void const* p, uint64_t bytes_p, void const* q, uint64_t bytes_q,
                        hipStream_t stream)
{
    // the part before the first and after the last whole 16 bytes is left out: it shares its
    // lines with chunks that are read
    auto whole = [](void const* x, uint64_t bytes, chunk_t const*& first, uint64_t& n) {
        uint64_t const addr = reinterpret_cast<uint64_t>(x);
        uint64_t const lo = (addr + 15) & ~uint64_t(15);
        first = reinterpret_cast<chunk_t const*>(lo);
        n = (bytes < 64 || lo - addr >= bytes) ? 0 : (bytes - (lo - addr)) / 16;
    };
    chunk_t const *fp, *fq;
    uint64_t       np, nq;
    whole(p, bytes_p, fp, np);
    whole(q, bytes_q, fq, nq);
    if (np + nq == 0) return;
    uint64_t const blocks = (np + nq + 1023) / 1024;
    hipLaunchKernelGGL(gemm_warm_kernel, dim3(unsigned(blocks)), dim3(256), 0, stream, fp, np, fq, nq,
                       static_cast<uint32_t*>(nullptr));
}

// `a` arrives cut into bm x bn tiles.  A tile without a kernel for this problem's load paths
// (they can change at run time, with the alignment of the buffers) is replaced by 128 x 128.
void launch_gemm_f16(int bm, int bn, gemm_args_t const& a, hipStream_t stream)
{
    using T = _Float16;
    if (a.tiles_m == 0) return;
    if (a.warm_a_bytes || a.warm_b_bytes) {
        gemm_warm_operands(a.A, a.warm_a_bytes, a.B, a.warm_b_bytes, stream);
    }
    if (gemm_dma_eligible<T>(a)) {
        if (a.shortk && gemm_shortk_eligible(a)) return launch_gemm_shortk(a, stream);
        // Compute-bound products with both operands along k: slices of 128 bytes per row
        // (whole cache lines: half the requests to the L2 of 64-byte slices), loads spread
        // over the k-steps where three stages fit, and eight wavefronts, two per SIMD, so
        // that one covers the other's waits.  Measured against the four-wavefront kernel on
        // 64-byte slices: 8192^3 1.13 -> 1.21 PFLOP/s, 4096^3 1.04 -> 1.14, 2048 x 4096 x
        // 4096 0.80 -> 1.00, 2048 x 11008 x 4096 0.86 -> 1.01 (results bit-identical).
        // Both operands along k and the buffers as aligned as at build time: the persistent
        // kernels (four wavefronts with the accumulators in named registers on 256 x 256,
        // multiplying and loading wavefronts on the rectangular tiles)
        if (a.persistent == 1 && bm == 256 && bn == 256 && w4::gemm_w4_eligible<2>(a)) {
            return w4::launch_gemm_w4<256, 256, 2>(a, a.workgroups, stream);
        }
        if (a.persistent == 2 && pc::gemm_pc_eligible(a)) {
            if (bm == 128 && bn == 256) return pc::launch_gemm_pc<128, 256>(a, a.workgroups, stream);
            if (bm == 256 && bn == 128) return pc::launch_gemm_pc<256, 128>(a, a.workgroups, stream);
        }
        if (a.wave8 && a.a_mode <= 1 && a.b_mode <= 1) {
            // (each operand along k or along its own m / n mode)
            auto modes = [&](auto launch00, auto launch01, auto launch10, auto launch11) {
                if (a.a_mode == 0) {
                    a.b_mode == 0 ? launch00() : launch01();
                } else {
                    a.b_mode == 0 ? launch10() : launch11();
                }
                if (a.splits > 1) launch_gemm_fold<T>(a, stream);
            };
            if (bm == 256 && bn == 256 && gemm_dma_wide_eligible<T>(a, 2)) {
                modes([&] { launch_gemm_dma_kernel_mode<T, 256, 256, 2, 0, 0, 128, 2, 4>(a, stream); },
                      [&] { launch_gemm_dma_kernel_mode<T, 256, 256, 2, 0, 1, 128, 2, 4>(a, stream); },
                      [&] { launch_gemm_dma_kernel_mode<T, 256, 256, 2, 1, 0, 128, 2, 4>(a, stream); },
                      [&] { launch_gemm_dma_kernel_mode<T, 256, 256, 2, 1, 1, 128, 2, 4>(a, stream); });
                return;
            }
            if (bm == 256 && bn == 128 && gemm_dma_wide_eligible<T>(a, 3)) {
                modes([&] { launch_gemm_dma_kernel_mode<T, 256, 128, 3, 0, 0, 128, 4, 2>(a, stream); },
                      [&] { launch_gemm_dma_kernel_mode<T, 256, 128, 3, 0, 1, 128, 4, 2>(a, stream); },
                      [&] { launch_gemm_dma_kernel_mode<T, 256, 128, 3, 1, 0, 128, 4, 2>(a, stream); },
                      [&] { launch_gemm_dma_kernel_mode<T, 256, 128, 3, 1, 1, 128, 4, 2>(a, stream); });
                return;
            }
            if (bm == 128 && bn == 256 && gemm_dma_wide_eligible<T>(a, 3)) {
                modes([&] { launch_gemm_dma_kernel_mode<T, 128, 256, 3, 0, 0, 128, 2, 4>(a, stream); },
                      [&] { launch_gemm_dma_kernel_mode<T, 128, 256, 3, 0, 1, 128, 2, 4>(a, stream); },
                      [&] { launch_gemm_dma_kernel_mode<T, 128, 256, 3, 1, 0, 128, 2, 4>(a, stream); },
                      [&] { launch_gemm_dma_kernel_mode<T, 128, 256, 3, 1, 1, 128, 2, 4>(a, stream); });
                return;
            }
        }
        if (bm == 256 && bn == 256) return launch_gemm_dma_kernel<T, 256, 256, 4>(a, stream);
        if (bm == 256 && bn == 128) return launch_gemm_dma_kernel<T, 256, 128, 4>(a, stream);
        if (bm == 128 && bn == 256) return launch_gemm_dma_kernel<T, 128, 256, 4>(a, stream);
        // short reductions: three stages of a small tile keep three workgroups per compute
        // unit, whose loads, matrix work and stores overlap each other
        if (bm == 128 && bn == 128 && a.wide_slices && a.a_mode == 0 &&
            gemm_dma_wide_eligible<T>(a, uint32_t(a.wide_slices))) {
            // a large operand streamed once: whole cache lines per row and slice
            if (a.b_mode == 0) {
                if (a.wide_slices == 2) {
                    launch_gemm_dma_kernel_mode<T, 128, 128, 2, 0, 0, 128>(a, stream);
                } else {
                    launch_gemm_dma_kernel_mode<T, 128, 128, 3, 0, 0, 128>(a, stream);
                }
            } else if (a.wide_slices == 2) {
                launch_gemm_dma_kernel_mode<T, 128, 128, 2, 0, 1, 128>(a, stream);
            } else {
                launch_gemm_dma_kernel_mode<T, 128, 128, 3, 0, 1, 128>(a, stream);
            }
            if (a.splits > 1) launch_gemm_fold<T>(a, stream);
            return;
        }
        if (bm == 128 && bn == 128) {
            return a.K < 512 ? launch_gemm_dma_kernel<T, 128, 128, 3>(a, stream)
                             : launch_gemm_dma_kernel<T, 128, 128, 4>(a, stream);
        }
    }
    if (bm == 256 && bn == 256 && launch_gemm_fast<T, 256, 256>(a, stream)) return;
    gemm_args_t const b = with_tile(a, 128, 128);
    if (launch_gemm_fast<T, 128, 128>(b, stream)) return;
    launch_gemm_kernel<T, 128, 128, -1, -1>(b, stream);
}

// Measurement aid: matrix-core throughput with register-resident operands, i.e. the ceiling
// any fp16 GEMM on this device can approach.  With operands of random bits the cores draw more
// power than with zeros and the clock drops, so both are reported.
__global__ __launch_bounds__(256) void mfma_probe_kernel(chunk_t const* in, float* out, int iters)
{
    half8_t   x = __builtin_bit_cast(half8_t, in[threadIdx.x]);
    half8_t   y = __builtin_bit_cast(half8_t, in[threadIdx.x + 256]);
    float16_t acc[8];
#pragma unroll
    for (int i = 0; i != 8; ++i) {
#pragma unroll
        for (int e = 0; e != 16; ++e) acc[i][e] = 0;
    }
    for (int it = 0; it != iters; ++it) {
#pragma unroll
        for (int i = 0; i != 8; ++i) {
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(x, y, acc[i], 0, 0, 0);
        }
    }
    float s = 0;
#pragma unroll
    for (int i = 0; i != 8; ++i) {
#pragma unroll
        for (int e = 0; e != 16; ++e) s += acc[i][e];
    }
    out[blockIdx.x * 256 + threadIdx.x] = s;
}

// Returns TFLOP/s, or a negative value on a device error.  `operands`: 512 x 16 bytes on the
// device; `scratch`: blocks x 256 floats.
double probe_mfma_f16(void const* operands, void* scratch, int blocks, int iters,
                      hipStream_t stream)
{
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return -1.0;
    hipLaunchKernelGGL(mfma_probe_kernel, dim3(blocks), dim3(256), 0, stream,
                       static_cast<chunk_t const*>(operands), static_cast<float*>(scratch), 64);
    (void)hipEventRecord(e0, stream);
    hipLaunchKernelGGL(mfma_probe_kernel, dim3(blocks), dim3(256), 0, stream,
                       static_cast<chunk_t const*>(operands), static_cast<float*>(scratch), iters);
    (void)hipEventRecord(e1, stream);
    float ms = 0;
    bool  ok = hipEventSynchronize(e1) == hipSuccess &&
              hipEventElapsedTime(&ms, e0, e1) == hipSuccess && ms > 0;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (!ok) return -1.0;
    double flop = double(blocks) * 4.0 * double(iters) * 8.0 * 32768.0;
    return flop / (double(ms) * 1e-3) / 1e12;
}

}  // namespace gemm
}  // namespace es
