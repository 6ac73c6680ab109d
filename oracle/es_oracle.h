/*
 * CPU oracle for the einsummable apply-node path.  TEST INFRASTRUCTURE ONLY:
 * this library is the checker that parity tests, the smoke test and the
 * benchmark's cpu_baseline leg compare against; no shipped code path may call it.
 *
 * Every function restates, in plain C, the semantics of a piece of
 * dcbdan/einsummable (paths relative to the reference tree):
 *   scalarop text grammar        src/einsummable/scalarop.cc:2678-3135
 *   per-op arithmetic            src/einsummable/scalarop.cc:554-780, 960-1010
 *   einsummable interpreter      src/einsummable/reference.cc:401-483
 *   agg_into (castable in dtype) src/einsummable/dbuffer.cc:343-347
 *   touch                        src/einsummable/reference.cc:522-607, src/engine/touch.cc
 *   touch simplify               src/einsummable/touch.cc:3-28
 *   fills                        src/einsummable/reference.cc:485-508
 *   merge_adjacent_dims / str    src/einsummable/einsummable.cc:32-218, 364-470
 *   accumulate-wide rule         src/engine/cpu/kernel_executor.cc:1163-1176
 */
#ifndef ES_ORACLE_H
#define ES_ORACLE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ES_O_F16 = 0, ES_O_F32 = 1, ES_O_F64 = 2, ES_O_C64 = 3 };

/* Evaluation modes.
 *  EXACT: every scalarop node is rounded to its own dtype and aggregation runs in the
 *         output dtype, in row-major order over the aggregated modes (reference.cc:456-482).
 *  WIDE : every real node is evaluated in double without intermediate rounding and
 *         add/mul aggregation runs in double, rounded once at the end (the "computed in
 *         higher precision" result that fp16/fp32 kernels are compared against).       */
enum { ES_O_EXACT = 0, ES_O_WIDE = 1 };

const char* es_oracle_last_error(void);

/* fp16 helpers (IEEE binary16, round-to-nearest-even, as half 2.2.0 half.hpp:373-374). */
uint16_t es_oracle_f64_to_f16(double v);
uint16_t es_oracle_f32_to_f16(float v);
float    es_oracle_f16_to_f32(uint16_t h);

/* Parse then print a scalarop (scalarop.cc:2881-3011). Returns 0 or -1. */
int es_oracle_scalarop_roundtrip(const char* text, char* out, size_t cap);

/* out_dtype, number of holes (max arg + 1) and each hole's dtype (-1 if unused). */
int es_oracle_scalarop_info(const char* text, int* out_dtype, int* n_inputs, int* inn_dtypes,
                            int cap);

/* Evaluate at one point. Inputs/outputs are raw little-endian bit patterns in a uint64_t
 * (f16 in the low 16 bits, f32 in the low 32, c64 = re | im<<32). */
int es_oracle_scalarop_eval(const char* text, int n_inputs, const uint64_t* input_bits, int mode,
                            uint64_t* out_bits, int* out_dtype);

/* Evaluate over n points: input k is a dense array of its dtype, out a dense array of
 * the scalarop's output dtype. */
int es_oracle_scalarop_map(const char* text, int n_inputs, const void* const* inputs, uint64_t n,
                           int mode, void* out);

/* The einsummable interpreter.  inns_flat/inns_offsets: input k uses modes
 * inns_flat[inns_offsets[k] .. inns_offsets[k+1]).  castable: '+','x','v','^' or 0.
 * The constructor's aggregation-mode renumbering (einsummable.cc:58-72) is applied. */
int es_oracle_einsummable(const uint64_t* join_shape, int join_rank, const int* inns_flat,
                          const int* inns_offsets, int n_inns, int out_rank, const char* join_text,
                          char castable, int mode, void* out, const void* const* inns);

/* merge_adjacent_dims (einsummable.cc:166-218).  Output arrays must hold join_rank /
 * the same number of mode ids as the input. Returns the new join rank (or -1). */
int es_oracle_merge_adjacent_dims(const uint64_t* join_shape, int join_rank, const int* inns_flat,
                                  const int* inns_offsets, int n_inns, int out_rank,
                                  uint64_t* new_join_shape, int* new_inns_flat,
                                  int* new_inns_offsets, int* new_out_rank);

/* einsummable_t::str() e.g. "ab,bc->ac" after aggregation renumbering. */
int es_oracle_einsummable_str(const int* inns_flat, const int* inns_offsets, int n_inns,
                              int out_rank, char* out, size_t cap);

/* parse_str (einsummable.cc:364-441): "ij,jk->ik" -> inns, out_rank. */
int es_oracle_einsummable_parse(const char* str, int* inns_flat, int* inns_offsets, int* n_inns,
                                int* out_rank, int cap);

/* touch: dims = rank x {d_inn, d_out, offset_inn, offset_out, size}. */
int es_oracle_touch(const uint64_t* dims, int rank, char castable, int dtype, void* out,
                    const void* inn);
int es_oracle_touch_simplify(const uint64_t* dims, int rank, uint64_t* out_dims, int* out_rank);

int es_oracle_fill_constant(int dtype, uint64_t bits, uint64_t nelem, void* out);
int es_oracle_fill_lowertri(int dtype, uint64_t lower_bits, uint64_t upper_bits, uint64_t nrow,
                            uint64_t ncol, int64_t start, void* out);

#ifdef __cplusplus
}
#endif
#endif
