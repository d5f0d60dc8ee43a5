/*
 * TEST INFRASTRUCTURE ONLY — CPU restatement of Arm Compute Library's quantized GEMM path.
 *
 * This file and everything else under oracle/ is the checker the parity tests compare the
 * HIP path against, and the CPU baseline bench.py times. Nothing the library ships may
 * include, link or call it.
 *
 * All citations are paths below the reference checkout (ACL 38.0.0).
 *
 * Conventions (identical to the reference):
 *  - matrices are row-major: A is M x K, B is K x N, dst is M x N; "ld*" are row strides in elements;
 *  - a_offset / b_offset are ADDED to every element of A / B before the product
 *    (arm_compute/runtime/NEON/functions/NEGEMMLowpMatrixMultiplyCore.h:95-97,
 *     tests/validation/reference/GEMMLowp.cpp:231-251);
 *  - shift > 0 is a rounding right shift after the multiply, shift < 0 a left shift before it
 *    (src/core/NEON/NEAsymm.h:97-121).
 *
 * Pinning status: every function here is checked against the reference's own portable
 * implementation (oracle/_ref, built from /root/reference by oracle/Makefile) and against
 * closed forms / brute force in tests/test_oracle_*.py.  orc_gemmlowp_f32 follows the NEON
 * source order of float operations (two roundings when offsets are non-zero); no aarch64 run
 * exists to confirm that no fused multiply-add is emitted there, so with non-zero offsets the
 * last-bit behaviour of that one function is "parity unpinned" (the reference's own test
 * oracle, one rounding, is also exported by oracle/_ref and both agree to 1e-6 relative).
 * orc_requant_fixedpoint_s16 follows the NEON source (rounding multiply); the reference's portable
 * test oracle uses the non-rounding multiply for every output type and no NEON test covers the
 * int16 kernel, so it is pinned by the architectural definition of SQRDMULH (big-integer model in
 * tests/test_oracle_gemm.py) and to within 1 of oracle/_ref: "parity unpinned" beyond that.
 * orc_f32_to_f16 / orc_gemmlowp_f16: the conversion is pinned against numpy's IEEE conversion (every half, every
 * midpoint, the thresholds) and the function against the reference's half dequantization + half addition in
 * oracle/_ref (identical bits without offsets; with offsets the float underneath is orc_gemmlowp_f32's).
 * Its act_twice clamp (an activation together with non-zero offsets on the F32 path) follows the
 * source order too; none of the reference's tests runs that combination: "parity unpinned".
 */
#ifndef ORACLE_GEMMLOWP_ORACLE_H
#define ORACLE_GEMMLOWP_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- requantization primitive ------------------------------------------------------------- */
int32_t orc_sqdmulh(int32_t a, int32_t b);
int32_t orc_rounding_shift_right(int32_t x, int32_t exponent);
/* full fixed-point stage on one accumulator; returns the int32 before narrowing */
int32_t orc_requant_s32(int32_t v, int32_t mult, int32_t shift, int32_t result_offset);
/* narrow + clamp: is_signed selects int8 / uint8 saturation, then [min_bound,max_bound] is applied */
int32_t orc_narrow_clamp(int32_t v, int is_signed, int32_t min_bound, int32_t max_bound);

/* float scale -> (Q31 multiplier, shift). returns 0 on success, non-zero where the reference errors */
int orc_calculate_quantized_multiplier(float multiplier, int32_t *quant_multiplier, int32_t *shift);

/* ---- GEMM ---------------------------------------------------------------------------------- */
/* a_signed / b_signed: 0 = uint8 storage, 1 = int8 storage */
void orc_gemmlowp_s32(const void *A, int a_signed, int64_t lda, const void *B, int b_signed, int64_t ldb,
                      int32_t *dst, int64_t ldd, int M, int N, int K, int32_t a_offset, int32_t b_offset);

/* stand-alone output stage on an int32 matrix; mult/shift have n_qparams entries (1 or N) */
void orc_output_stage_fixedpoint(const int32_t *src, int64_t lds, const int32_t *bias, void *dst, int64_t ldd,
                                 int dst_signed, int M, int N, const int32_t *mult, const int32_t *shift,
                                 int n_qparams, int32_t result_offset, int32_t min_bound, int32_t max_bound);

/* QUANTIZE_DOWN (integer multiplier): ((v + result_offset) * mult) >> shift, wrap-around, truncating shift, 0 <= shift < 32 */
int32_t orc_requant_scale_s32(int32_t v, int32_t mult, int32_t shift, int32_t result_offset);
void orc_output_stage_scale(const int32_t *src, int64_t lds, const int32_t *bias, void *dst, int64_t ldd, int dst_signed,
                            int M, int N, const int32_t *mult, const int32_t *shift, int n_qparams,
                            int32_t result_offset, int32_t min_bound, int32_t max_bound);
void orc_gemmlowp_scale(const void *A, int a_signed, int64_t lda, const void *B, int b_signed, int64_t ldb,
                        const int32_t *bias, void *dst, int64_t ldd, int dst_signed, int M, int N, int K,
                        int32_t a_offset, int32_t b_offset, const int32_t *mult, const int32_t *shift, int n_qparams,
                        int32_t result_offset, int32_t min_bound, int32_t max_bound);

/* int32 -> QSYMM16 stage (rounding doubling high multiply, no offset) */
int32_t orc_sqrdmulh_s32(int32_t a, int32_t b);
int16_t orc_requant_fixedpoint_s16(int32_t v, int32_t mult, int32_t shift, int32_t min_bound, int32_t max_bound);
void    orc_output_stage_fixedpoint_s16(const int32_t *src, int64_t ld_src, const int32_t *bias, int16_t *dst,
                                        int64_t ld_dst, int M, int N, int32_t mult, int32_t shift, int32_t min_bound,
                                        int32_t max_bound);

/* GEMM + offset contribution + bias + fixed-point stage in one call */
void orc_gemmlowp_fixedpoint(const void *A, int a_signed, int64_t lda, const void *B, int b_signed, int64_t ldb,
                             const int32_t *bias, void *dst, int64_t ldd, int dst_signed, int M, int N, int K,
                             int32_t a_offset, int32_t b_offset, const int32_t *mult, const int32_t *shift,
                             int n_qparams, int32_t result_offset, int32_t min_bound, int32_t max_bound);

/* GEMM with F32 dequantised output: float(acc)*scale (+bias) (+ previous dst when accumulate) (clamp when act_twice)
 * then + float(offset terms)*scale, then clamp */
void orc_gemmlowp_f32(const void *A, int a_signed, int64_t lda, const void *B, int b_signed, int64_t ldb,
                      const float *bias, float *dst, int64_t ldd, int M, int N, int K, int32_t a_offset,
                      int32_t b_offset, float scale, float act_min, float act_max, int accumulate, int act_twice);
uint16_t orc_f32_to_f16(float f);
float    orc_f16_to_f32(uint16_t h);
void     orc_gemmlowp_f16(const void *A, int a_signed, int64_t lda, const void *B, int b_signed, int64_t ldb,
                          const float *bias, uint16_t *dst, int64_t ldd, int M, int N, int K, int32_t a_offset,
                          int32_t b_offset, float scale, float act_min, float act_max, int accumulate, int act_twice);

/* ---- convolution lowering ------------------------------------------------------------------ */
/* NHWC src [batch][H][W][C] -> patch matrix [batch*OH*OW][KH*KW*C], K ordered (ky, kx, c) */
void orc_im2col_nhwc(const uint8_t *src, uint8_t *dst, int batch, int H, int W, int C, int KH, int KW,
                     int stride_x, int stride_y, int pad_left, int pad_top, int pad_right, int pad_bottom,
                     int dil_x, int dil_y, int pad_byte);
/* weights [OFM][KH][KW][C] -> B matrix [K = KH*KW*C][N = OFM] */
void orc_weights_reshape(const uint8_t *w, uint8_t *b_mat, int OFM, int KH, int KW, int C);
void orc_conv_out_dims(int H, int W, int KH, int KW, int stride_x, int stride_y, int pad_left, int pad_top,
                       int pad_right, int pad_bottom, int dil_x, int dil_y, int *OH, int *OW);
/* direct (no im2col) quantized NHWC convolution, used to check im2col+gemm against a second formulation */
void orc_conv_nhwc_direct(const void *src, int src_signed, const void *w, int w_signed, const int32_t *bias,
                          void *dst, int dst_signed, int batch, int H, int W, int C, int OFM, int KH, int KW,
                          int stride_x, int stride_y, int pad_left, int pad_top, int pad_right, int pad_bottom,
                          int dil_x, int dil_y, int32_t src_zero_point, int32_t w_zero_point,
                          const int32_t *mult, const int32_t *shift, int n_qparams, int32_t result_offset,
                          int32_t min_bound, int32_t max_bound);

/* ---- timed CPU baseline (same integers, OpenMP + SIMD when the host has it) ------------------ */
/* B is given as K x N row-major; packs it internally (not timed by callers that pass a prepacked handle) */
typedef struct orc_fast_gemm orc_fast_gemm;
orc_fast_gemm *orc_fast_prepare(const void *B, int b_signed, int64_t ldb, int N, int K);
void           orc_fast_destroy(orc_fast_gemm *g);
/* returns the SIMD level used: 0 scalar, 2 AVX2, 5 AVX-512 VNNI */
int orc_fast_gemmlowp_fixedpoint(const orc_fast_gemm *g, const void *A, int a_signed, int64_t lda,
                                 const int32_t *bias, void *dst, int64_t ldd, int dst_signed, int M,
                                 int32_t a_offset, int32_t b_offset, const int32_t *mult, const int32_t *shift,
                                 int n_qparams, int32_t result_offset, int32_t min_bound, int32_t max_bound);
int orc_fast_threads(void);

#ifdef __cplusplus
}
#endif
#endif
