/*
 * CPU oracle for the FP8 skinny-GEMM path.  TEST INFRASTRUCTURE ONLY.
 *
 * This library is the checker that the HIP kernels are compared against.  It is
 * linked or loaded only by the test-suite, the smoke check and the CPU-baseline
 * leg of the benchmark; no product code path may call into it.
 *
 * Reference restated (all paths under the reference tree):
 *   projects/skinny_gemm/test.cu:7-39     host_skinny_gemm  -> orc_gemm_ref / orc_gemm_omp
 *   projects/skinny_gemm/test.cu:94-107   delta metrics     -> orc_delta_metrics
 *   projects/common.cuh:97-105            fp8 host cast, SATFINITE -> orc_e4m3_encode
 *   projects/tiled_sum_reduce/test.cu:5-26 host_tiled_sum_reduce -> orc_tiled_sum_reduce
 *   projects/async_gemm_sparse/test.cu:7-38 host GEMM without scale, fp32 out -> orc_gemm_f32
 * The reference decodes E4M3 FNUZ through ROCm's hip_fp8.h and multiplies the two
 * operands as _Float16; this restatement decodes OCP E4M3 (the gfx950 MFMA
 * format) and multiplies in fp32, because 448*448 overflows fp16.
 * orc_gemm_f32 and orc_tiled_sum_reduce are checked bit for bit against those two
 * host loops themselves, compiled from the reference's sources (ref_host_loops.cpp ->
 * _ref/libref_host.so, tests/test_reference_host.py): outside the three codes the
 * formats read differently an FNUZ operand is exactly half the OCP one, so the
 * reference's fp32 result is this library's times 1/4.
 *
 * Functions with no counterpart in the reference ("parity unpinned" by the
 * reference; pinned by closed forms, brute force and library casts in
 * tests/test_oracle_*.py): OCP E4M3 numerics, bf16 output rounding, per-row
 * encode / decode / reduce, 2:4 prune / compress / decompress.
 */
#ifndef SG_ORACLE_H
#define SG_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- scalar formats ---------------------------------------------------- */
float    orc_e4m3_decode(uint8_t code);        /* OCP E4M3: 0x7f/0xff NaN, max 448 */
uint8_t  orc_e4m3_encode(float x);             /* RNE, saturate-to-finite (inf -> 448), NaN -> 0x7f|sign */
uint16_t orc_bf16_from_f32(float x);           /* RNE, NaN kept quiet */
float    orc_bf16_to_f32(uint16_t h);

void orc_e4m3_decode_n(const uint8_t* q, float* out, size_t n);
void orc_e4m3_encode_n(const float* x, uint8_t* out, size_t n);
void orc_bf16_from_f32_n(const float* x, uint16_t* out, size_t n);
void orc_bf16_to_f32_n(const uint16_t* h, float* out, size_t n);

/* ---- deterministic input generator (counter based) ---------------------- */
/* Element i of stream (seed, stream_id) depends on nothing but (seed, stream_id, i). */
uint64_t orc_rng_u64(uint64_t seed, uint64_t stream_id, uint64_t i);
void orc_fill_normal_f32(float* out, size_t n, uint64_t seed, uint64_t stream_id);
void orc_fill_uniform_f32(float* out, size_t n, uint64_t seed, uint64_t stream_id, float lo, float hi);
/* bf16(N(0,1)) with floor(frac * n) random positions overwritten by +/-mag */
void orc_fill_normal_bf16_outliers(uint16_t* out, size_t n, uint64_t seed, uint64_t stream_id,
                                   double frac, float mag);

/* ---- quantisation ------------------------------------------------------- */
float orc_absmax_f32(const float* x, size_t n);
/* scale = absmax/448 (absmax == 0 -> 1); q = e4m3_rne_sat(x / scale); returns scale */
float orc_quantize_tensor(const float* x, uint8_t* q, size_t n);

/* ---- dense GEMM: D[m,n] = scale * sum_k dec(A[i,k]) * dec(B[j*b_stride + k]) --- */
/* faithful single-thread loop, sequential fp32 accumulation over k, bf16 output */
void orc_gemm_ref(const uint8_t* A, const uint8_t* B, uint16_t* D, float scale,
                  int m, int n, int k, int b_stride);
/* same arithmetic and per-output summation order, decode LUT, OpenMP over n */
void orc_gemm_omp(const uint8_t* A, const uint8_t* B, uint16_t* D, float scale,
                  int m, int n, int k, int b_stride);
/* fp32 output of the same sum, scale applied (pass 1.0f for the async_gemm flavour) */
void orc_gemm_f32(const uint8_t* A, const uint8_t* B, float* D, float scale,
                  int m, int n, int k, int b_stride);
/* bf16( ((sum * scale) * row_scale[i]) * col_scale[j] ), each product rounded to fp32; either array may be NULL */
void orc_gemm_rowcol(const uint8_t* A, const uint8_t* B, uint16_t* D, float scale, const float* row_scale,
                     const float* col_scale, int m, int n, int k, int b_stride);
/* fp64 accumulated truth (no output rounding) */
void orc_gemm_f64(const uint8_t* A, const uint8_t* B, double* D, double scale,
                  int m, int n, int k, int b_stride);
/* The same sums taken the way gfx950's FP8 matrix instructions take them: inside every aligned run of
 * `group` consecutive k (8 for the dense instructions; 16 for 2:4 weights, whose 8 kept values per lane span
 * 16 k) products are aligned to the run's largest exponent sum and cut off 7 bits below their own last
 * mantissa bit; runs are added without further loss.  Measured on hardware, not taken from the reference. */
void orc_gemm_grouped_f32(const uint8_t* A, const uint8_t* B, float* D, float scale,
                          int m, int n, int k, int b_stride, int group);
void orc_gemm_grouped(const uint8_t* A, const uint8_t* B, uint16_t* D, float scale,
                      int m, int n, int k, int b_stride, int group);
int  orc_num_threads(void);

/* ---- 2:4 structured sparsity (weights N x K, groups of 4 along K) ------- */
/* keep the 2 largest |x| of each group, ties -> lower index; zeros the rest in place */
void orc_prune24_f32(float* B, int n, int k);
/* the same rule applied to E4M3 codes (magnitude = code & 0x7f); dropped positions become 0x00 */
void orc_prune24_e4m3(uint8_t* B, int n, int k);
/* dense E4M3 N x K (already 2:4) -> values N x K/2 + metadata N x K/8.
 * One nibble per group: low 2 bits = index of first kept value, high 2 bits =
 * index of the second (first < second); two groups per byte, lower group in the
 * low nibble.  A group with fewer than two non-zeros keeps the lowest free
 * indices so that first < second always holds.  Returns 0, or -1 if a group has
 * more than two non-zero codes. */
int  orc_compress24(const uint8_t* B, uint8_t* vals, uint8_t* meta, int n, int k);
void orc_decompress24(const uint8_t* vals, const uint8_t* meta, uint8_t* B, int n, int k);
void orc_gemm_sparse24_omp(const uint8_t* A, const uint8_t* vals, const uint8_t* meta,
                           uint16_t* D, float scale, int m, int n, int k);

/* ---- per-row FP8 codec (single-GPU half of an FP8 all-reduce) ----------- */
/* X bf16 rows x cols; scale[r] = absmax(row)/448 (0 -> 1; NaNs ignored); Q = e4m3_rne_sat(x/scale),
 * a NaN quotient (NaN input, inf/inf) -> 0x7f */
void orc_fp8_encode_rows(const uint16_t* X, uint8_t* Q, float* scales, int rows, int cols);
/* Y = bf16(dec(Q) * scale[r]) */
void orc_fp8_decode_rows(const uint8_t* Q, const float* scales, uint16_t* Y, int rows, int cols);
/* Y = bf16( sum_{i<nbuf} dec(Q_i) * scale_i[r] ), fp32, in buffer order.
 * Q: nbuf buffers each rows*cols apart; scales: nbuf arrays each rows apart. */
void orc_fp8_reduce_rows(const uint8_t* Q, const float* scales, uint16_t* Y,
                         int nbuf, int rows, int cols);

/* ---- fp32 batch sum: D = sum_b (A_b + B_b) ------------------------------ */
void orc_tiled_sum_reduce(const float* A, const float* B, float* D, int b, int m, int n);

/* ---- comparison metrics -------------------------------------------------- */
/* max and summed absolute difference of two bf16 arrays (the reference's test output) */
void orc_delta_metrics_bf16(const uint16_t* got, const uint16_t* ref, size_t n,
                            float* max_delta, float* total_delta);
/* max over elements of |d-ref| / max(|ref|, 1e-2 * rms(ref)) */
double orc_max_rel_err_bf16(const uint16_t* got, const uint16_t* ref, size_t n);

#ifdef __cplusplus
}
#endif
#endif
