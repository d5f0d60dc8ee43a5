/*
 * TEST INFRASTRUCTURE ONLY — scalar CPU restatement of the reference's quantized GEMM arithmetic.
 * See gemmlowp_oracle.h for conventions and pinning status. Plain C, no SIMD: clarity over speed.
 */
#include "gemmlowp_oracle.h"

#include <limits.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* int32 arithmetic with two's-complement wrap-around, as the NEON lanes (vaddq_s32 / vmulq_s32) do */
static inline int32_t wrap_add(int32_t a, int32_t b) { return (int32_t)((uint32_t)a + (uint32_t)b); }
static inline int32_t wrap_mul(int32_t a, int32_t b) { return (int32_t)((uint32_t)a * (uint32_t)b); }

/* SQDMULH: high half of the doubled 64-bit product, no rounding; saturates only INT32_MIN * INT32_MIN.
 * tests/validation/reference/UtilsQuantizedAsymm.h:60-67 ; vqdmulhq_s32 in src/core/NEON/NEAsymm.h:104-113 */
int32_t orc_sqdmulh(int32_t a, int32_t b)
{
    if (a == INT32_MIN && b == INT32_MIN)
        return INT32_MAX;
    const int64_t p = (int64_t)a * (int64_t)b; /* |p| <= 2^62, doubling done as a shift by 31 instead of 32 */
    return (int32_t)(p >> 31);
}

/* SRSHL by -exponent: (x + 2^(e-1)) >> e evaluated without intermediate overflow (round half up).
 * src/core/NEON/NEMath.inl:430-440 (vrshlq_s32) ; tests/validation/reference/UtilsQuantizedAsymm.h:53-56 */
int32_t orc_rounding_shift_right(int32_t x, int32_t exponent)
{
    if (exponent <= 0)
        return x;
    if (exponent > 62)
        return 0;
    return (int32_t)(((int64_t)x + ((int64_t)1 << (exponent - 1))) >> exponent);
}

/* src/core/NEON/NEAsymm.h:95-128 (per tensor), :233-296 (per channel: same per lane, branch on sign of shift)
 * tests/validation/reference/UtilsQuantizedAsymm.h:70-88 */
int32_t orc_requant_s32(int32_t v, int32_t mult, int32_t shift, int32_t result_offset)
{
    int32_t r;
    if (shift < 0)
    {
        const int32_t pre = (-shift >= 32) ? 0 : wrap_mul(v, (int32_t)((uint32_t)1 << (-shift)));
        r                 = orc_sqdmulh(pre, mult);
    }
    else
    {
        r = orc_rounding_shift_right(orc_sqdmulh(v, mult), shift);
    }
    return wrap_add(r, result_offset);
}

/* saturating narrow to the 8-bit type, then the bounded-relu clamp
 * src/core/NEON/NEAsymm.h:130-147 (u8), :205-216 (s8) */
int32_t orc_narrow_clamp(int32_t v, int is_signed, int32_t min_bound, int32_t max_bound)
{
    const int32_t lo = is_signed ? -128 : 0;
    const int32_t hi = is_signed ? 127 : 255;
    if (v < lo)
        v = lo;
    if (v > hi)
        v = hi;
    if (v < min_bound)
        v = min_bound;
    if (v > max_bound)
        v = max_bound;
    return v;
}

/* src/core/utils/quantization/AsymmHelpers.cpp:43-115 */
int orc_calculate_quantized_multiplier(float multiplier, int32_t *quant_multiplier, int32_t *shift)
{
    const float   epsilon = 0.00001f;
    const int64_t one_q31 = (int64_t)1 << 31;
    int           e       = 0;
    if (multiplier >= 1.f)
    {
        const double q       = frexp((double)multiplier, &e);
        int64_t      q_fixed = (int64_t)round(q * (double)one_q31);
        if (q_fixed > one_q31)
            return 1;
        if (q_fixed == one_q31)
        {
            q_fixed /= 2;
            ++e;
        }
        if (e < 0 || q_fixed > INT32_MAX)
            return 1;
        *quant_multiplier = (int32_t)q_fixed;
        *shift            = -e;
        return 0;
    }
    if (multiplier < -epsilon || multiplier > 1.0f + epsilon)
        return 1;
    const double q           = frexp((double)multiplier, &e);
    int32_t      right_shift = -e;
    int64_t      q_fixed     = (int64_t)round(q * (double)one_q31);
    if (q_fixed > one_q31)
        return 1;
    if (q_fixed == one_q31)
    {
        q_fixed /= 2;
        --right_shift;
    }
    if (right_shift < 0 || q_fixed > INT32_MAX)
        return 1;
    *quant_multiplier = (int32_t)q_fixed;
    *shift            = right_shift;
    return 0;
}

static inline int32_t load8(const void *p, int is_signed, int64_t idx)
{
    return is_signed ? (int32_t)((const int8_t *)p)[idx] : (int32_t)((const uint8_t *)p)[idx];
}

/* Raw accumulators and the sums the offset contribution needs.
 * acc: src/cpu/kernels/CpuGemmLowpMatrixMultiplyKernel.cpp (any int8 GEMM) ;
 * row/col sums: src/cpu/kernels/CpuGemmLowpMatrixReductionKernel.cpp:133-204, :273-446 */
static void gemm_acc_and_sums(const void *A, int a_signed, int64_t lda, const void *B, int b_signed, int64_t ldb,
                              int M, int N, int K, int32_t *acc, int32_t *rowsum, int32_t *colsum)
{
    for (int j = 0; j < N; ++j)
        colsum[j] = 0;
    for (int k = 0; k < K; ++k)
        for (int j = 0; j < N; ++j)
            colsum[j] = wrap_add(colsum[j], load8(B, b_signed, (int64_t)k * ldb + j));
    for (int i = 0; i < M; ++i)
    {
        int32_t *row = acc + (int64_t)i * N;
        int32_t  rs  = 0;
        for (int j = 0; j < N; ++j)
            row[j] = 0;
        for (int k = 0; k < K; ++k)
        {
            const int32_t a = load8(A, a_signed, (int64_t)i * lda + k);
            rs              = wrap_add(rs, a);
            if (b_signed)
            {
                const int8_t *b = (const int8_t *)B + (int64_t)k * ldb;
                for (int j = 0; j < N; ++j)
                    row[j] = wrap_add(row[j], a * (int32_t)b[j]);
            }
            else
            {
                const uint8_t *b = (const uint8_t *)B + (int64_t)k * ldb;
                for (int j = 0; j < N; ++j)
                    row[j] = wrap_add(row[j], a * (int32_t)b[j]);
            }
        }
        rowsum[i] = rs;
    }
}

/* acc + a_offset*colsum[j] + b_offset*rowsum[i] + a_offset*b_offset*K
 * src/cpu/kernels/gemmlowp/generic/neon/int32.cpp:56-283 ; src/cpu/operators/CpuGemmLowpMatrixMultiplyCore.cpp:281-321 */
static inline int32_t offset_term(int32_t a_offset, int32_t b_offset, int K, int32_t colsum, int32_t rowsum)
{
    int32_t t = wrap_mul(wrap_mul(a_offset, b_offset), K);
    t         = wrap_add(t, wrap_mul(a_offset, colsum));
    t         = wrap_add(t, wrap_mul(b_offset, rowsum));
    return t;
}

void orc_gemmlowp_s32(const void *A, int a_signed, int64_t lda, const void *B, int b_signed, int64_t ldb,
                      int32_t *dst, int64_t ldd, int M, int N, int K, int32_t a_offset, int32_t b_offset)
{
    int32_t *acc    = (int32_t *)malloc(sizeof(int32_t) * (size_t)(M > 0 ? M : 1) * (size_t)(N > 0 ? N : 1));
    int32_t *rowsum = (int32_t *)malloc(sizeof(int32_t) * (size_t)(M > 0 ? M : 1));
    int32_t *colsum = (int32_t *)malloc(sizeof(int32_t) * (size_t)(N > 0 ? N : 1));
    gemm_acc_and_sums(A, a_signed, lda, B, b_signed, ldb, M, N, K, acc, rowsum, colsum);
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j)
            dst[(int64_t)i * ldd + j] =
                wrap_add(acc[(int64_t)i * N + j], offset_term(a_offset, b_offset, K, colsum[j], rowsum[i]));
    free(acc);
    free(rowsum);
    free(colsum);
}

static inline void store8(void *dst, int dst_signed, int64_t idx, int32_t v)
{
    if (dst_signed)
        ((int8_t *)dst)[idx] = (int8_t)v;
    else
        ((uint8_t *)dst)[idx] = (uint8_t)v;
}

/* src/cpu/kernels/CpuGemmLowpQuantizeDownInt32ToInt8ScaleByFixedPointKernel.cpp:79-181 (and the Uint8 twin) */
void orc_output_stage_fixedpoint(const int32_t *src, int64_t lds, const int32_t *bias, void *dst, int64_t ldd,
                                 int dst_signed, int M, int N, const int32_t *mult, const int32_t *shift,
                                 int n_qparams, int32_t result_offset, int32_t min_bound, int32_t max_bound)
{
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j)
        {
            int32_t v = src[(int64_t)i * lds + j];
            if (bias)
                v = wrap_add(v, bias[j]);
            const int q = n_qparams > 1 ? j : 0;
            v           = orc_requant_s32(v, mult[q], shift[q], result_offset);
            store8(dst, dst_signed, (int64_t)i * ldd + j, orc_narrow_clamp(v, dst_signed, min_bound, max_bound));
        }
}

/* QUANTIZE_DOWN, the integer-multiplier stage: ((v + result_offset) * mult) >> shift with wrap-around arithmetic and a
 * truncating arithmetic shift (src/cpu/kernels/CpuGemmLowpQuantizeDownInt32ScaleKernel.cpp:92-180 and the scalar tail of
 * src/cpu/kernels/CpuGemmLowpOffsetContributionOutputStageKernel.cpp:348-362; reference test oracle
 * tests/validation/reference/GEMMLowp.cpp:66-104). shift is in [0, 31]. */
int32_t orc_requant_scale_s32(int32_t v, int32_t mult, int32_t shift, int32_t result_offset)
{
    const uint32_t u = ((uint32_t)v + (uint32_t)result_offset) * (uint32_t)mult;
    const int32_t  r = (int32_t)u;
    /* arithmetic shift right, written without relying on the sign behaviour of >> */
    return r >= 0 ? (r >> shift) : -(int32_t)(((uint32_t)(-(int64_t)r) + ((1u << shift) - 1u)) >> shift);
}

void orc_output_stage_scale(const int32_t *src, int64_t lds, const int32_t *bias, void *dst, int64_t ldd, int dst_signed,
                            int M, int N, const int32_t *mult, const int32_t *shift, int n_qparams,
                            int32_t result_offset, int32_t min_bound, int32_t max_bound)
{
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j)
        {
            int32_t v = src[(int64_t)i * lds + j];
            if (bias)
                v = wrap_add(v, bias[j]);
            const int q = n_qparams > 1 ? j : 0;
            v           = orc_requant_scale_s32(v, mult[q], shift[q], result_offset);
            store8(dst, dst_signed, (int64_t)i * ldd + j, orc_narrow_clamp(v, dst_signed, min_bound, max_bound));
        }
}

void orc_gemmlowp_scale(const void *A, int a_signed, int64_t lda, const void *B, int b_signed, int64_t ldb,
                        const int32_t *bias, void *dst, int64_t ldd, int dst_signed, int M, int N, int K,
                        int32_t a_offset, int32_t b_offset, const int32_t *mult, const int32_t *shift, int n_qparams,
                        int32_t result_offset, int32_t min_bound, int32_t max_bound)
{
    int32_t *t = (int32_t *)malloc(sizeof(int32_t) * (size_t)(M > 0 ? M : 1) * (size_t)(N > 0 ? N : 1));
    orc_gemmlowp_s32(A, a_signed, lda, B, b_signed, ldb, t, N, M, N, K, a_offset, b_offset);
    orc_output_stage_scale(t, N, bias, dst, ldd, dst_signed, M, N, mult, shift, n_qparams, result_offset, min_bound,
                           max_bound);
    free(t);
}

/* src/cpu/kernels/CpuGemmLowpOffsetContributionOutputStageKernel.cpp:248-364 (per tensor), :366-461 (per channel) */
void orc_gemmlowp_fixedpoint(const void *A, int a_signed, int64_t lda, const void *B, int b_signed, int64_t ldb,
                             const int32_t *bias, void *dst, int64_t ldd, int dst_signed, int M, int N, int K,
                             int32_t a_offset, int32_t b_offset, const int32_t *mult, const int32_t *shift,
                             int n_qparams, int32_t result_offset, int32_t min_bound, int32_t max_bound)
{
    int32_t *t = (int32_t *)malloc(sizeof(int32_t) * (size_t)(M > 0 ? M : 1) * (size_t)(N > 0 ? N : 1));
    orc_gemmlowp_s32(A, a_signed, lda, B, b_signed, ldb, t, N, M, N, K, a_offset, b_offset);
    orc_output_stage_fixedpoint(t, N, bias, dst, ldd, dst_signed, M, N, mult, shift, n_qparams, result_offset,
                                min_bound, max_bound);
    free(t);
}

/* SQRDMULH, the rounding doubling multiply returning the high half: sat((2*a*b + 2^31) >> 32) = sat((a*b + 2^30) >> 31).
 * Only a == b == INT32_MIN saturates. (Arm ARM, SQRDMULH; used as vqrdmulhq_n_s32 in src/core/NEON/NESymm.h:62-69 and
 * written out as (in_64 + (1 << 30)) >> 31 in its scalar twin, NESymm.h:105-114.) */
int32_t orc_sqrdmulh_s32(int32_t a, int32_t b)
{
    if (a == INT32_MIN && b == INT32_MIN)
        return INT32_MAX;
    return (int32_t)(((int64_t)a * (int64_t)b + ((int64_t)1 << 30)) >> 31);
}

/* src/core/NEON/NESymm.h:54-85 (the vector lanes: the left shift wraps in int32 as vmulq_n_s32 does, the right shift
 * is vrshlq_s32, i.e. round half up, exact): int32 -> int16, no offset; bounded == !(min <= -32768 && max >= 32767)
 * (src/cpu/kernels/CpuGemmLowpQuantizeDownInt32ToInt16ScaleByFixedPointKernel.cpp:205). */
int16_t orc_requant_fixedpoint_s16(int32_t v, int32_t mult, int32_t shift, int32_t min_bound, int32_t max_bound)
{
    int32_t r;
    if (shift < 0)
        r = orc_sqrdmulh_s32(-shift >= 32 ? 0 : wrap_mul(v, (int32_t)((uint32_t)1 << (-shift))), mult);
    else
        r = orc_rounding_shift_right(orc_sqrdmulh_s32(v, mult), shift);
    if (r < -32768)
        r = -32768;
    if (r > 32767)
        r = 32767;
    if (!(min_bound <= -32768 && max_bound >= 32767))
    {
        if (r < min_bound)
            r = min_bound;
        if (r > max_bound)
            r = max_bound;
    }
    return (int16_t)r;
}

/* CpuGemmLowpQuantizeDownInt32ToInt16ScaleByFixedPointKernel::run_internal (.cpp:76-200): bias add wraps */
void orc_output_stage_fixedpoint_s16(const int32_t *src, int64_t ld_src, const int32_t *bias, int16_t *dst,
                                     int64_t ld_dst, int M, int N, int32_t mult, int32_t shift, int32_t min_bound,
                                     int32_t max_bound)
{
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j)
        {
            const int32_t v = (int32_t)((uint32_t)src[(int64_t)i * ld_src + j] + (uint32_t)(bias ? bias[j] : 0));
            dst[(int64_t)i * ld_dst + j] = orc_requant_fixedpoint_s16(v, mult, shift, min_bound, max_bound);
        }
}

/* src/core/NEON/kernels/arm_gemm/quantized.cpp:977-1030 (float(acc)*scale, + bias, + previous destination value when
 * accumulating, clamp) followed by src/cpu/kernels/gemmlowp/generic/neon/impl.h:95-155 + fp32.cpp:31-54
 * (+= float(offset terms)*scale) and the CpuActivation post-op
 * (src/cpu/operators/CpuGemmLowpMatrixMultiplyCore.cpp:326-332,806-810). The first clamp only exists for the
 * activations the assembly GEMM takes (src/core/utils/AssemblyUtils.cpp:32-62: RELU, BOUNDED_RELU and LU_BOUNDED_RELU
 * with lower bound 0): act_twice says whether it does. It only matters when an offset term follows it.
 * accumulate: dst holds the previous values on entry (GEMMInfo::accumulate). */
void orc_gemmlowp_f32(const void *A, int a_signed, int64_t lda, const void *B, int b_signed, int64_t ldb,
                      const float *bias, float *dst, int64_t ldd, int M, int N, int K, int32_t a_offset,
                      int32_t b_offset, float scale, float act_min, float act_max, int accumulate, int act_twice)
{
    int32_t *acc    = (int32_t *)malloc(sizeof(int32_t) * (size_t)(M > 0 ? M : 1) * (size_t)(N > 0 ? N : 1));
    int32_t *rowsum = (int32_t *)malloc(sizeof(int32_t) * (size_t)(M > 0 ? M : 1));
    int32_t *colsum = (int32_t *)malloc(sizeof(int32_t) * (size_t)(N > 0 ? N : 1));
    gemm_acc_and_sums(A, a_signed, lda, B, b_signed, ldb, M, N, K, acc, rowsum, colsum);
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j)
        {
            volatile float r = (float)acc[(int64_t)i * N + j] * scale; /* volatile: forbid FMA contraction */
            if (bias)
                r = r + bias[j];
            if (accumulate)
                r = r + dst[(int64_t)i * ldd + j];
            if (a_offset != 0 || b_offset != 0)
            {
                if (act_twice)
                {
                    if (r < act_min)
                        r = act_min;
                    if (r > act_max)
                        r = act_max;
                }
                /* each term is only formed when its offset is non-zero, exactly like the four branches of
                 * neon_run_offset_contribution_float; the integer sum is identical either way */
                const int32_t  off    = offset_term(a_offset, b_offset, K, colsum[j], rowsum[i]);
                volatile float scaled = (float)off * scale;
                r                     = r + scaled;
            }
            float o = r;
            if (o < act_min)
                o = act_min;
            if (o > act_max)
                o = act_max;
            dst[(int64_t)i * ldd + j] = o;
        }
    free(acc);
    free(rowsum);
    free(colsum);
}

/* float -> IEEE half, round to nearest, ties to even: how the reference's host-side half type converts
 * (support/Half.h:33-34 sets HALF_ROUND_STYLE 1 and HALF_ROUND_TIES_TO_EVEN 1 for include/half/half.hpp) and what
 * vcvt_f16_f32 does in src/cpu/kernels/gemmlowp/generic/neon/fp16.cpp:52-55. Returns the 16 bits. */
uint16_t orc_f32_to_f16(float f)
{
    uint32_t x;
    memcpy(&x, &f, sizeof(x));
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t mag  = x & 0x7FFFFFFFu;
    if (mag >= 0x7F800000u) /* infinity / NaN */
        return (uint16_t)(sign | 0x7C00u | (mag > 0x7F800000u ? 0x0200u | ((mag >> 13) & 0x03FFu) : 0u));
    if (mag >= 0x477FF000u) /* rounds to a magnitude >= 65520: overflows to infinity */
        return (uint16_t)(sign | 0x7C00u);
    if (mag < 0x33000001u) /* at most half of the smallest subnormal (2^-25): rounds to zero */
        return (uint16_t)sign;
    const int      e    = (int)(mag >> 23) - 127;       /* unbiased exponent, -25 .. 15 */
    const uint32_t man  = (mag & 0x007FFFFFu) | 0x00800000u; /* 24-bit significand with the leading one */
    /* shift so that the result keeps 11 significant bits (normal) or fewer (subnormal, e < -14) */
    const int      sh   = e < -14 ? 13 + (-14 - e) : 13;
    uint32_t       q    = man >> sh;
    const uint32_t rem  = man & ((1u << sh) - 1u), half = 1u << (sh - 1);
    if (rem > half || (rem == half && (q & 1u)))
        ++q;
    /* q carries the leading one for normals: (e+15) << 10 added to q - 0x400; a carry out of the significand bumps
     * the exponent by itself. Subnormals: exponent field 0, q is the fraction (a carry makes the smallest normal). */
    const uint32_t h = e < -14 ? q : (((uint32_t)(e + 15) << 10) + (q - 0x400u));
    return (uint16_t)(sign | h);
}

float orc_f16_to_f32(uint16_t h)
{
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t ex   = (h >> 10) & 0x1Fu, fr = h & 0x3FFu;
    uint32_t       x;
    if (ex == 0x1Fu)
        x = sign | 0x7F800000u | (fr << 13);
    else if (ex != 0)
        x = sign | ((ex + 112u) << 23) | (fr << 13);
    else if (fr == 0)
        x = sign;
    else
    {
        int      e = -1;
        uint32_t m = fr;
        do
        {
            ++e;
            m <<= 1;
        } while ((m & 0x400u) == 0);
        x = sign | ((uint32_t)(112 - e) << 23) | ((m & 0x3FFu) << 13);
    }
    float f;
    memcpy(&f, &x, sizeof(f));
    return f;
}

/* GEMMLowp with an F16 destination (src/cpu/operators/CpuGemmLowpMatrixMultiplyCore.cpp:305-309,374-375; test
 * tests/validation/NEON/GEMMLowp.cpp:598-621; reference values tests/validation/fixtures/GEMMLowpFixture.h:908-920 =
 * half(float(s32) * scale), to which the previous half values are added IN HALF when accumulating: both operands
 * widened, one float addition, rounded again). Here: the float result of orc_gemmlowp_f32 rounded to half; when
 * accumulating, that half is added to the previous half the fixture's way and the activation clamp, which must follow
 * the addition, is applied to the sum (the clamp ahead of the offset term that act_twice stands for is then skipped).
 * Without offsets this is the fixture's value bit for bit; with offsets the float value underneath differs by the
 * rounding order of orc_gemmlowp_f32 (<= 1e-5 relative), which rarely crosses a half rounding boundary (the NEON kernels
 * themselves add in half precision and are only held to a 0.2 relative tolerance by that test). */
void orc_gemmlowp_f16(const void *A, int a_signed, int64_t lda, const void *B, int b_signed, int64_t ldb,
                      const float *bias, uint16_t *dst, int64_t ldd, int M, int N, int K, int32_t a_offset,
                      int32_t b_offset, float scale, float act_min, float act_max, int accumulate, int act_twice)
{
    float *tmp = (float *)malloc(sizeof(float) * (size_t)(M > 0 ? M : 1) * (size_t)(N > 0 ? N : 1));
    orc_gemmlowp_f32(A, a_signed, lda, B, b_signed, ldb, bias, tmp, N, M, N, K, a_offset, b_offset, scale,
                     accumulate ? -INFINITY : act_min, accumulate ? INFINITY : act_max, 0, accumulate ? 0 : act_twice);
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j)
        {
            uint16_t h = orc_f32_to_f16(tmp[(int64_t)i * N + j]);
            if (accumulate)
            {
                volatile float sum = orc_f16_to_f32(dst[(int64_t)i * ldd + j]) + orc_f16_to_f32(h);
                if (sum < act_min)
                    sum = act_min;
                if (sum > act_max)
                    sum = act_max;
                h = orc_f32_to_f16(sum);
            }
            dst[(int64_t)i * ldd + j] = h;
        }
    free(tmp);
}

/* src/core/Utils.cpp:288-332 (FLOOR rounding, the default of PadStrideInfo) */
void orc_conv_out_dims(int H, int W, int KH, int KW, int stride_x, int stride_y, int pad_left, int pad_top,
                       int pad_right, int pad_bottom, int dil_x, int dil_y, int *OH, int *OW)
{
    int w = (int)floorf((float)(W + pad_left + pad_right - (dil_x * (KW - 1) + 1)) / (float)stride_x + 1.f);
    int h = (int)floorf((float)(H + pad_top + pad_bottom - (dil_y * (KH - 1) + 1)) / (float)stride_y + 1.f);
    *OW   = w < 1 ? 1 : w;
    *OH   = h < 1 ? 1 : h;
}

/* src/cpu/kernels/directconv2d/impl.h:148-220 (linearize_volume_nhwc), :307-389 (run_im2col, start = o*stride - pad,
 * pad value = src zero point :333-334) ; tests/validation/reference/Im2Col.cpp:108-170 */
void orc_im2col_nhwc(const uint8_t *src, uint8_t *dst, int batch, int H, int W, int C, int KH, int KW,
                     int stride_x, int stride_y, int pad_left, int pad_top, int pad_right, int pad_bottom,
                     int dil_x, int dil_y, int pad_byte)
{
    int OH, OW;
    orc_conv_out_dims(H, W, KH, KW, stride_x, stride_y, pad_left, pad_top, pad_right, pad_bottom, dil_x, dil_y, &OH,
                      &OW);
    const int64_t K = (int64_t)KH * KW * C;
    for (int n = 0; n < batch; ++n)
        for (int oy = 0; oy < OH; ++oy)
            for (int ox = 0; ox < OW; ++ox)
            {
                uint8_t *row = dst + (((int64_t)n * OH + oy) * OW + ox) * K;
                for (int ky = 0; ky < KH; ++ky)
                    for (int kx = 0; kx < KW; ++kx)
                    {
                        const int iy  = oy * stride_y - pad_top + ky * dil_y;
                        const int ix  = ox * stride_x - pad_left + kx * dil_x;
                        uint8_t  *out = row + ((int64_t)ky * KW + kx) * C;
                        if (iy < 0 || iy >= H || ix < 0 || ix >= W)
                            memset(out, pad_byte, (size_t)C);
                        else
                            memcpy(out, src + (((int64_t)n * H + iy) * W + ix) * C, (size_t)C);
                    }
            }
}

/* src/cpu/kernels/CpuWeightsReshapeKernel.cpp:150-166: k = c + kx*C + ky*C*KW, one column of B per filter */
void orc_weights_reshape(const uint8_t *w, uint8_t *b_mat, int OFM, int KH, int KW, int C)
{
    const int64_t K = (int64_t)KH * KW * C;
    for (int o = 0; o < OFM; ++o)
        for (int64_t k = 0; k < K; ++k)
            b_mat[k * OFM + o] = w[(int64_t)o * K + k];
}

/* tests/validation/reference/Convolution3d.h:120-245 restated for NHWC storage: out-of-image taps are skipped,
 * which equals padding with the zero point because (zero_point + input_offset) == 0 */
void orc_conv_nhwc_direct(const void *src, int src_signed, const void *w, int w_signed, const int32_t *bias,
                          void *dst, int dst_signed, int batch, int H, int W, int C, int OFM, int KH, int KW,
                          int stride_x, int stride_y, int pad_left, int pad_top, int pad_right, int pad_bottom,
                          int dil_x, int dil_y, int32_t src_zero_point, int32_t w_zero_point,
                          const int32_t *mult, const int32_t *shift, int n_qparams, int32_t result_offset,
                          int32_t min_bound, int32_t max_bound)
{
    int OH, OW;
    orc_conv_out_dims(H, W, KH, KW, stride_x, stride_y, pad_left, pad_top, pad_right, pad_bottom, dil_x, dil_y, &OH,
                      &OW);
    for (int n = 0; n < batch; ++n)
        for (int oy = 0; oy < OH; ++oy)
            for (int ox = 0; ox < OW; ++ox)
                for (int o = 0; o < OFM; ++o)
                {
                    int32_t acc = 0;
                    for (int ky = 0; ky < KH; ++ky)
                        for (int kx = 0; kx < KW; ++kx)
                        {
                            const int iy = oy * stride_y - pad_top + ky * dil_y;
                            const int ix = ox * stride_x - pad_left + kx * dil_x;
                            if (iy < 0 || iy >= H || ix < 0 || ix >= W)
                                continue;
                            for (int c = 0; c < C; ++c)
                            {
                                const int32_t iv = load8(src, src_signed, (((int64_t)n * H + iy) * W + ix) * C + c);
                                const int32_t wv =
                                    load8(w, w_signed, (((int64_t)o * KH + ky) * KW + kx) * C + c);
                                acc = wrap_add(acc, wrap_mul(iv - src_zero_point, wv - w_zero_point));
                            }
                        }
                    if (bias)
                        acc = wrap_add(acc, bias[o]);
                    const int q = n_qparams > 1 ? o : 0;
                    acc         = orc_requant_s32(acc, mult[q], shift[q], result_offset);
                    store8(dst, dst_signed, (((int64_t)n * OH + oy) * OW + ox) * OFM + o,
                           orc_narrow_clamp(acc, dst_signed, min_bound, max_bound));
                }
}
