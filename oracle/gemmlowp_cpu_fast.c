/*
 * TEST INFRASTRUCTURE ONLY — the timed CPU baseline: the same integers as gemmlowp_oracle.c
 * (checked bit-for-bit against it in tests/test_oracle_fast.py), computed with OpenMP over output
 * blocks and AVX-512 VNNI / AVX2 inner products when the host CPU has them (run-time dispatch, so
 * one binary built in the container runs on any x86-64 host).
 *
 * Structure mirrors the reference's fused path: B re-laid out once (pretranspose_B_array,
 * src/cpu/operators/internal/CpuGemmAssemblyDispatch.cpp:594-617) with its column sums
 * (src/core/NEON/kernels/arm_gemm/quantized.cpp:915-971), row sums of A per run (:802-838), and the
 * requantisation applied to each finished output block (requantize_block_32, :54-261).
 *
 * Operand normalisation: A is brought to uint8 and B to int8 by flipping the top bit where needed
 * (x ^ 0x80), compensated by -128 / +128 on that operand's offset — the reference's own
 * _flip_signedness trick (src/cpu/operators/CpuGemmLowpMatrixMultiplyCore.cpp:153-190); the sum
 * of (a + a_off)(b + b_off) is the same polynomial, so the int32 result is unchanged.
 */
#include "gemmlowp_oracle.h"

#include <immintrin.h>
#include <limits.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

struct orc_fast_gemm
{
    int      N, K, Kp, Np;
    int      b_flipped;
    int8_t  *bt;     /* [Np][Kp] int8, K contiguous, zero padded */
    int32_t *colsum; /* [Np] sums of the int8 (possibly flipped) values */
};

int orc_fast_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

orc_fast_gemm *orc_fast_prepare(const void *B, int b_signed, int64_t ldb, int N, int K)
{
    orc_fast_gemm *g = (orc_fast_gemm *)calloc(1, sizeof(*g));
    g->N             = N;
    g->K             = K;
    g->Kp            = (K + 63) & ~63;
    g->Np            = (N + 3) & ~3;
    g->b_flipped     = !b_signed;
    g->bt            = (int8_t *)aligned_alloc(64, (size_t)g->Np * (size_t)g->Kp);
    g->colsum        = (int32_t *)calloc((size_t)g->Np, sizeof(int32_t));
    memset(g->bt, 0, (size_t)g->Np * (size_t)g->Kp);
    const uint8_t flip = b_signed ? 0 : 0x80;
#pragma omp parallel for schedule(static)
    for (int j = 0; j < N; ++j)
    {
        int8_t *row = g->bt + (size_t)j * g->Kp;
        int32_t s   = 0;
        for (int k = 0; k < K; ++k)
        {
            const int8_t v = (int8_t)(((const uint8_t *)B)[(int64_t)k * ldb + j] ^ flip);
            row[k]         = v;
            s += v;
        }
        g->colsum[j] = s;
    }
    return g;
}

void orc_fast_destroy(orc_fast_gemm *g)
{
    if (!g)
        return;
    free(g->bt);
    free(g->colsum);
    free(g);
}

/* 4 x 4 block of dot products over Kp bytes; a rows are uint8, b rows int8 */
typedef void (*block_fn)(const uint8_t *a0, const uint8_t *a1, const uint8_t *a2, const uint8_t *a3, const int8_t *b,
                         int Kp, int32_t out[16]);

static void block_scalar(const uint8_t *a0, const uint8_t *a1, const uint8_t *a2, const uint8_t *a3, const int8_t *b,
                         int Kp, int32_t out[16])
{
    const uint8_t *a[4] = {a0, a1, a2, a3};
    for (int r = 0; r < 4; ++r)
        for (int c = 0; c < 4; ++c)
        {
            int32_t       s  = 0;
            const int8_t *bc = b + (size_t)c * Kp;
            for (int k = 0; k < Kp; ++k)
                s += (int32_t)a[r][k] * (int32_t)bc[k];
            out[r * 4 + c] = s;
        }
}

__attribute__((target("avx2"))) static inline int32_t hsum256(__m256i v)
{
    __m128i s = _mm_add_epi32(_mm256_castsi256_si128(v), _mm256_extracti128_si256(v, 1));
    s         = _mm_add_epi32(s, _mm_shuffle_epi32(s, 0x4e));
    s         = _mm_add_epi32(s, _mm_shuffle_epi32(s, 0xb1));
    return _mm_cvtsi128_si32(s);
}

__attribute__((target("avx2"))) static void block_avx2(const uint8_t *a0, const uint8_t *a1, const uint8_t *a2,
                                                       const uint8_t *a3, const int8_t *b, int Kp, int32_t out[16])
{
    __m256i        acc[16];
    const uint8_t *a[4] = {a0, a1, a2, a3};
    for (int i = 0; i < 16; ++i)
        acc[i] = _mm256_setzero_si256();
    for (int k = 0; k < Kp; k += 16)
    {
        __m256i av[4], bv[4];
        for (int r = 0; r < 4; ++r)
            av[r] = _mm256_cvtepu8_epi16(_mm_loadu_si128((const __m128i *)(a[r] + k)));
        for (int c = 0; c < 4; ++c)
            bv[c] = _mm256_cvtepi8_epi16(_mm_loadu_si128((const __m128i *)(b + (size_t)c * Kp + k)));
        for (int r = 0; r < 4; ++r)
            for (int c = 0; c < 4; ++c)
                acc[r * 4 + c] = _mm256_add_epi32(acc[r * 4 + c], _mm256_madd_epi16(av[r], bv[c]));
    }
    for (int i = 0; i < 16; ++i)
        out[i] = hsum256(acc[i]);
}

__attribute__((target("avx512f,avx512bw,avx512vl,avx512vnni"))) static void
block_vnni(const uint8_t *a0, const uint8_t *a1, const uint8_t *a2, const uint8_t *a3, const int8_t *b, int Kp,
           int32_t out[16])
{
    __m512i        acc[16];
    const uint8_t *a[4] = {a0, a1, a2, a3};
    for (int i = 0; i < 16; ++i)
        acc[i] = _mm512_setzero_si512();
    for (int k = 0; k < Kp; k += 64)
    {
        __m512i av[4], bv[4];
        for (int r = 0; r < 4; ++r)
            av[r] = _mm512_loadu_si512((const void *)(a[r] + k));
        for (int c = 0; c < 4; ++c)
            bv[c] = _mm512_loadu_si512((const void *)(b + (size_t)c * Kp + k));
        for (int r = 0; r < 4; ++r)
            for (int c = 0; c < 4; ++c)
                acc[r * 4 + c] = _mm512_dpbusd_epi32(acc[r * 4 + c], av[r], bv[c]);
    }
    for (int i = 0; i < 16; ++i)
        out[i] = _mm512_reduce_add_epi32(acc[i]);
}

static int pick_level(void)
{
    const char *force = getenv("ORC_FAST_LEVEL");
    int         lvl   = 0;
    __builtin_cpu_init();
    if (__builtin_cpu_supports("avx2"))
        lvl = 2;
    if (__builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw") &&
        __builtin_cpu_supports("avx512vl") && __builtin_cpu_supports("avx512vnni"))
        lvl = 5;
    if (force)
    {
        const int f = atoi(force);
        if (f < lvl)
            lvl = f >= 2 ? 2 : 0;
    }
    return lvl;
}

int orc_fast_gemmlowp_fixedpoint(const orc_fast_gemm *g, const void *A, int a_signed, int64_t lda,
                                 const int32_t *bias, void *dst, int64_t ldd, int dst_signed, int M,
                                 int32_t a_offset, int32_t b_offset, const int32_t *mult, const int32_t *shift,
                                 int n_qparams, int32_t result_offset, int32_t min_bound, int32_t max_bound)
{
    const int      lvl = pick_level();
    const block_fn fn  = lvl == 5 ? block_vnni : lvl == 2 ? block_avx2 : block_scalar;
    const int      N = g->N, K = g->K, Kp = g->Kp;
    const int      Mp = (M + 3) & ~3;
    /* A -> uint8 [Mp][Kp], zero padded (zero bytes meet zero bytes of B in the K padding) */
    uint8_t       *au     = (uint8_t *)aligned_alloc(64, (size_t)Mp * (size_t)Kp);
    int32_t       *rowsum = (int32_t *)malloc(sizeof(int32_t) * (size_t)Mp);
    const uint8_t  flip   = a_signed ? 0x80 : 0;
    const uint32_t ao     = (uint32_t)a_offset - (a_signed ? 128u : 0u);
    const uint32_t bo     = (uint32_t)b_offset + (g->b_flipped ? 128u : 0u);
#pragma omp parallel for schedule(static)
    for (int i = 0; i < Mp; ++i)
    {
        uint8_t *row = au + (size_t)i * Kp;
        int32_t  s   = 0;
        if (i < M)
        {
            const uint8_t *src = (const uint8_t *)A + (int64_t)i * lda;
            for (int k = 0; k < K; ++k)
            {
                row[k] = src[k] ^ flip;
                s += row[k];
            }
            memset(row + K, 0, (size_t)(Kp - K));
        }
        else
            memset(row, 0, (size_t)Kp);
        rowsum[i] = s;
    }
    const int NC = 64, MC = 128;
    const int n_panels = (N + NC - 1) / NC, m_panels = (M + MC - 1) / MC;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (int jp = 0; jp < n_panels; ++jp)
        for (int ip = 0; ip < m_panels; ++ip)
        {
            const int j_end = (jp + 1) * NC < g->Np ? (jp + 1) * NC : g->Np;
            const int i_end = (ip + 1) * MC < Mp ? (ip + 1) * MC : Mp;
            for (int i = ip * MC; i < i_end; i += 4)
                for (int j = jp * NC; j < j_end; j += 4)
                {
                    int32_t blk[16];
                    fn(au + (size_t)i * Kp, au + (size_t)(i + 1) * Kp, au + (size_t)(i + 2) * Kp,
                       au + (size_t)(i + 3) * Kp, g->bt + (size_t)j * Kp, Kp, blk);
                    for (int r = 0; r < 4 && i + r < M; ++r)
                        for (int c = 0; c < 4 && j + c < N; ++c)
                        {
                            uint32_t t = (uint32_t)blk[r * 4 + c];
                            t += ao * bo * (uint32_t)K + ao * (uint32_t)g->colsum[j + c] +
                                 bo * (uint32_t)rowsum[i + r];
                            if (bias)
                                t += (uint32_t)bias[j + c];
                            const int q = n_qparams > 1 ? j + c : 0;
                            int32_t   v = orc_requant_s32((int32_t)t, mult[q], shift[q], result_offset);
                            v           = orc_narrow_clamp(v, dst_signed, min_bound, max_bound);
                            if (dst_signed)
                                ((int8_t *)dst)[(int64_t)(i + r) * ldd + j + c] = (int8_t)v;
                            else
                                ((uint8_t *)dst)[(int64_t)(i + r) * ldd + j + c] = (uint8_t)v;
                        }
                }
        }
    free(au);
    free(rowsum);
    return lvl;
}
