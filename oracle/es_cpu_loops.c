/*
 * es_cpu_loops.c -- TEST / BENCHMARK INFRASTRUCTURE, not part of the product.
 *
 * Optimised CPU loops for the reported CPU baseline: what the reference's CPU kernel executor
 * runs for the benchmark configurations, written as plain -O3 loops with OpenMP over rows
 * and timed by bench.py on one thread and on all host cores.  Only bench.py's cpu_baseline
 * leg and the tests that check these loops against the oracle may call them.
 *
 *   binary / broadcast elementwise loops     src/engine/cpu/kernel_executor.cc:786-914
 *   ab->a reductions, add accumulated in double, max native
 *                                             src/engine/cpu/kernel_executor.cc:1163-1253
 *   touch: rows of the window, out (op)= inn  src/engine/touch.cc:119-237
 *   permute with the inner mode kept: row copies
 *                                             src/base/permute_.h:1-234
 * fp16 values are converted with the F16C instructions and computed in fp32, one rounding per
 * stored value (the reference rounds after every operation in half-float software; the
 * products max(x,0)*y and the maxima are exact either way, exp(x-m) differs by the rounding
 * of x-m).  threads <= 0 means all cores OpenMP sees.
 */
#include <immintrin.h>
#include <math.h>
#include <omp.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

static inline __m256 load8(const uint16_t* p) { return _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)p)); }
static inline void   store8(uint16_t* p, __m256 v)
{
    _mm_storeu_si128((__m128i*)p, _mm256_cvtps_ph(v, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
}
static inline float    h2f(uint16_t h) { return _cvtsh_ss(h); }
static inline uint16_t f2h(float f) { return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC); }

static int nthreads(int threads) { return threads > 0 ? threads : omp_get_max_threads(); }

int es_cpu_max_threads(void) { return omp_get_max_threads(); }

/* ij,ij->ij  max(x,0)*y */
void es_cpu_relu_mul_f16(const uint16_t* x, const uint16_t* y, uint16_t* out, size_t n, int threads)
{
    const __m256 zero = _mm256_setzero_ps();
#pragma omp parallel for num_threads(nthreads(threads)) schedule(static)
    for (size_t i = 0; i < n / 8; ++i) {
        __m256 a = _mm256_max_ps(load8(x + 8 * i), zero);
        store8(out + 8 * i, _mm256_mul_ps(a, load8(y + 8 * i)));
    }
    for (size_t i = n / 8 * 8; i < n; ++i) out[i] = f2h(fmaxf(h2f(x[i]), 0.0f) * h2f(y[i]));
}

/* ij->i max */
void es_cpu_rowmax_f16(const uint16_t* x, uint16_t* out, size_t rows, size_t cols, int threads)
{
#pragma omp parallel for num_threads(nthreads(threads)) schedule(static)
    for (size_t r = 0; r < rows; ++r) {
        const uint16_t* p = x + r * cols;
        __m256          m = _mm256_set1_ps(-INFINITY);
        size_t          c = 0;
        for (; c + 8 <= cols; c += 8) m = _mm256_max_ps(m, load8(p + c));
        float t[8];
        _mm256_storeu_ps(t, m);
        float best = t[0];
        for (int j = 1; j < 8; ++j) best = fmaxf(best, t[j]);
        for (; c < cols; ++c) best = fmaxf(best, h2f(p[c]));
        out[r] = f2h(best);
    }
}

/* ij,i->ij exp(x - m) */
void es_cpu_exp_sub_f16(const uint16_t* x, const uint16_t* m, uint16_t* out, size_t rows,
                        size_t cols, int threads)
{
#pragma omp parallel for num_threads(nthreads(threads)) schedule(static)
    for (size_t r = 0; r < rows; ++r) {
        const uint16_t* p = x + r * cols;
        uint16_t*       q = out + r * cols;
        float const     mr = h2f(m[r]);
        float           buf[256];
        for (size_t c0 = 0; c0 < cols; c0 += 256) {
            size_t const w = cols - c0 < 256 ? cols - c0 : 256;
            for (size_t c = 0; c < w; ++c) buf[c] = h2f(p[c0 + c]) - mr;
#pragma omp simd
            for (size_t c = 0; c < w; ++c) buf[c] = expf(buf[c]);
            for (size_t c = 0; c < w; ++c) q[c0 + c] = f2h(buf[c]);
        }
    }
}

/* ij->i add, accumulated in double as the reference does for f16 and f32 */
void es_cpu_rowsum_f16(const uint16_t* x, uint16_t* out, size_t rows, size_t cols, int threads)
{
#pragma omp parallel for num_threads(nthreads(threads)) schedule(static)
    for (size_t r = 0; r < rows; ++r) {
        const uint16_t* p = x + r * cols;
        __m256d         s0 = _mm256_setzero_pd(), s1 = _mm256_setzero_pd();
        size_t          c = 0;
        for (; c + 8 <= cols; c += 8) {
            __m256 v = load8(p + c);
            s0 = _mm256_add_pd(s0, _mm256_cvtps_pd(_mm256_castps256_ps128(v)));
            s1 = _mm256_add_pd(s1, _mm256_cvtps_pd(_mm256_extractf128_ps(v, 1)));
        }
        double t[4];
        _mm256_storeu_pd(t, _mm256_add_pd(s0, s1));
        double s = (t[0] + t[1]) + (t[2] + t[3]);
        for (; c < cols; ++c) s += (double)h2f(p[c]);
        out[r] = f2h((float)s);
    }
}

/* abcd->acbd on 2-byte elements: rows of d elements move as a whole */
void es_cpu_permute_acbd_2byte(const uint16_t* in, uint16_t* out, size_t a, size_t b, size_t c,
                               size_t d, int threads)
{
#pragma omp parallel for num_threads(nthreads(threads)) collapse(2) schedule(static)
    for (size_t ia = 0; ia < a; ++ia) {
        for (size_t ic = 0; ic < c; ++ic) {
            for (size_t ib = 0; ib < b; ++ib) {
                memcpy(out + ((ia * c + ic) * b + ib) * d, in + ((ia * b + ib) * c + ic) * d, d * 2);
            }
        }
    }
}

/* one two-dimensional accumulate touch: out[ro + i, co + j] += inn[i, j], f16 */
void es_cpu_touch_add_f16(uint16_t* out, size_t out_cols, const uint16_t* inn, size_t rows,
                          size_t cols, size_t ro, size_t co, int threads)
{
#pragma omp parallel for num_threads(nthreads(threads)) schedule(static)
    for (size_t i = 0; i < rows; ++i) {
        uint16_t*       o = out + (ro + i) * out_cols + co;
        const uint16_t* x = inn + i * cols;
        size_t          j = 0;
        for (; j + 8 <= cols; j += 8) store8(o + j, _mm256_add_ps(load8(o + j), load8(x + j)));
        for (; j < cols; ++j) o[j] = f2h(h2f(o[j]) + h2f(x[j]));
    }
}
