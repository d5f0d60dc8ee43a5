// K3: bandwidth-bound GEMM for M <= 16 (decode-shaped: one token batch against a large weight matrix).
//
// The reference has no dedicated kernel above M == 1 (GemvPretransposed, src/core/NEON/kernels/arm_gemm/gemm_qint8.cpp:75-79)
// and otherwise runs its hybrid kernels; here the whole run is one streaming pass over B at HBM speed.
//
// B is packed at prepare time into 1 KiB blocks of 16 columns x 64 k in matrix-core operand order
// (Bs[Np/16][Kp/64][64 lanes][16 bytes]), so every wave-wide load is one contiguous, fully coalesced 1 KiB read and a
// column group's K range is one contiguous stream. A block owns one group of 16 output columns; its waves split the
// k blocks, each keeping UNROLL loads in flight, multiply with v_mfma_i32_16x16x64_i8 (A rows padded to 16 with
// zeros; A itself is tiny and stays in L2), reduce the partial 16 x 16 accumulators through LDS, and wave 0 applies the
// fused offset / requantisation epilogue.
#include "internal.hpp"

namespace mi355
{
typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int SK_WAVES  = 8;
constexpr int SK_UNROLL = 8;

template <int EPI, bool FLIP_A>
__global__ __launch_bounds__(SK_WAVES * 64) void gemm_skinny_kernel(GemmArgs g)
{
    __shared__ __attribute__((aligned(16))) int32_t red[SK_WAVES][64][4];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int ng   = blockIdx.x;
    const int KB   = (int)(g.Kp / 64);

    // this wave's contiguous range of k blocks
    const int per  = (KB + SK_WAVES - 1) / SK_WAVES;
    const int kb0  = wave * per;
    const int kb1  = min(KB, kb0 + per);

    const int   arow   = lane & 15;
    const int   akc    = (lane >> 4) * 16;
    const bool  a_live = arow < g.M;
    const int8_t *__restrict__ a_ptr = g.A + (int64_t)min(arow, g.M - 1) * g.lda + akc;
    const int8_t *__restrict__ b_ptr = g.Bp + ((int64_t)ng * KB * 64 + lane) * 16;

    v4i acc = {0, 0, 0, 0};
    for (int kb = kb0; kb < kb1; kb += SK_UNROLL)
    {
        v4i fa[SK_UNROLL], fb[SK_UNROLL];
#pragma unroll
        for (int u = 0; u < SK_UNROLL; ++u)
        {
            const int kk = kb + u;
            fb[u]        = (v4i){0, 0, 0, 0};
            fa[u]        = (v4i){0, 0, 0, 0};
            if (kk < kb1)
            {
                fb[u] = *(const v4i *)(b_ptr + (int64_t)kk * 1024);
                const int rem = g.K - (kk * 64 + akc);
                if (a_live && rem > 0)
                {
                    fa[u] = rem >= 16 ? *(const v4i *)(a_ptr + (int64_t)kk * 64)
                                      : load16_partial(a_ptr + (int64_t)kk * 64, rem);
                    if (FLIP_A)
                        fa[u] ^= (int)0x80808080;
                }
            }
        }
#pragma unroll
        for (int u = 0; u < SK_UNROLL; ++u)
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[u], fb[u], acc, 0, 0, 0);
    }

    *(v4i *)&red[wave][lane][0] = acc;
    __syncthreads();
    if (wave != 0)
        return;
#pragma unroll
    for (int w = 1; w < SK_WAVES; ++w)
    {
        const v4i o = *(const v4i *)&red[w][lane][0];
        acc += o;
    }

    // accumulator r of lane l is row 4*(l/16) + r, column l%16
    const EpiParams &p = g.epi;
    const int        j = ng * 16 + (lane & 15);
    if (j >= g.N)
        return;
    const int32_t cv = p.colvec[j];
    int32_t       mu = p.mult_s, sh = p.shift_s;
    if (EPI == EPI_FIXEDPOINT && p.mult)
    {
        mu = p.mult[j];
        sh = p.shift[j];
    }
    const float bf = (EPI == EPI_F32 && p.bias_f32) ? p.bias_f32[j] : 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r)
    {
        const int i = 4 * (lane >> 4) + r;
        if (i < g.M)
        {
            const int32_t rv  = p.rowvec ? p.rowvec[i] : 0;
            const int64_t idx = (int64_t)i * g.ldd + j;
            if (EPI == EPI_S32)
                ((int32_t *)g.D)[idx] = (int32_t)((uint32_t)acc[r] + (uint32_t)cv + (uint32_t)rv);
            else if (EPI == EPI_FIXEDPOINT)
                ((int8_t *)g.D)[idx] = (int8_t)epi_fixedpoint(acc[r], cv, rv, mu, sh, p);
            else
                ((float *)g.D)[idx] =
                    epi_f32(acc[r], (int32_t)((uint32_t)cv + (uint32_t)rv), bf, p.bias_f32 != nullptr, p);
        }
    }
}

int skinny_launch(int epi, bool flip_a, const GemmArgs &args, hipStream_t s)
{
    if (args.M < 1 || args.M > SKINNY_MAX_M || args.Kp % 64 != 0 || args.K > args.Kp)
        return (int)hipErrorInvalidValue;
    const dim3 grid((args.N + 15) / 16), block(SK_WAVES * 64);
    GemmArgs   a = args;
#define MI355_SK(E, F) gemm_skinny_kernel<E, F><<<grid, block, 0, s>>>(a)
    if (epi == EPI_S32)
        flip_a ? MI355_SK(EPI_S32, true) : MI355_SK(EPI_S32, false);
    else if (epi == EPI_FIXEDPOINT)
        flip_a ? MI355_SK(EPI_FIXEDPOINT, true) : MI355_SK(EPI_FIXEDPOINT, false);
    else if (epi == EPI_F32)
        flip_a ? MI355_SK(EPI_F32, true) : MI355_SK(EPI_F32, false);
    else
        return (int)hipErrorInvalidValue;
#undef MI355_SK
    return (int)hipGetLastError();
}
} // namespace mi355
