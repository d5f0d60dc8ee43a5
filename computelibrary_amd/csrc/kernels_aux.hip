// Bandwidth-bound helper kernels of the quantized-GEMM path: B packing + column sums (prepare time), the A pre-pass
// (row sums / padded copy), the stand-alone output stage, explicit im2col, and a one-thread-per-output GEMM used only
// for cross-checking the matrix-core kernels.
#include "internal.hpp"

namespace mi355
{
typedef int v4i __attribute__((ext_vector_type(4)));

static inline int launch_status()
{
    return (int)hipGetLastError();
}

// sum of the four int8 lanes of a dword
__device__ __forceinline__ int32_t sum4_i8(int32_t w)
{
    return __builtin_amdgcn_sdot4(w, 0x01010101, 0, false);
}

__global__ void fill_i32_kernel(int32_t *p, int32_t v, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n)
        p[i] = v;
}
int fill_i32_launch(int32_t *p, int32_t v, int64_t n, hipStream_t s)
{
    if (n <= 0)
        return 0;
    fill_i32_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s>>>(p, v, n);
    return launch_status();
}

// ---- split K: the partial products of `splits` K slices (S32 planes of M rows of ldp words, `plane` words apart) summed
// and put through the epilogue the fused kernel would have applied. One thread per 4 consecutive columns of a row.
// Same arithmetic as epilogue_store_t: the sum of the slices is the accumulator of the whole K
// (what CpuGemmLowpOffsetContributionOutputStageKernel, src/cpu/kernels/CpuGemmLowpOffsetContributionOutputStageKernel.cpp:
// 830-940, is handed by the matrix multiply before it).
template <int EPI>
__global__ __launch_bounds__(256) void splitk_finish_kernel(const int32_t *__restrict__ parts, int64_t plane, int ldp, int splits,
                                                            GemmArgs g)
{
    typedef int   v4i __attribute__((ext_vector_type(4)));
    const EpiParams &p  = g.epi;
    const int        n4 = (g.N + 3) / 4;
    const int64_t    t  = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= (int64_t)g.M * n4)
        return;
    const int i = (int)(t / n4), j0 = (int)(t % n4) * 4;
    v4i       acc = {0, 0, 0, 0};
    for (int sl = 0; sl < splits; ++sl) // (columns from N on hold whatever the allocation held: never used below)
        acc += *(const v4i *)(parts + (int64_t)sl * plane + (int64_t)i * ldp + j0);
    const int32_t rv  = p.rowvec ? p.rowvec[i] : 0;
    const int64_t idx = (int64_t)i * g.ldd + j0;
    const bool    vec = p.vec_store && j0 + 3 < g.N;
    char         *D   = (char *)g.D;
    v4i           o   = {0, 0, 0, 0};
#pragma unroll
    for (int c = 0; c < 4; ++c)
    {
        const int j = j0 + c;
        if (j >= g.N)
            continue;
        const int32_t cv = p.colvec[j];
        if (EPI == EPI_FIXEDPOINT)
            o[c] = epi_fixedpoint(acc[c], cv, rv, p.mult ? p.mult[j] : p.mult_s, p.shift ? p.shift[j] : p.shift_s, p);
        else if (EPI == EPI_S32)
            o[c] = (int32_t)((uint32_t)acc[c] + (uint32_t)cv + (uint32_t)rv + (p.accumulate ? (uint32_t)((int32_t *)D)[idx + c] : 0u));
        else
            o[c] = __float_as_int(epi_f32(acc[c], (int32_t)((uint32_t)cv + (uint32_t)rv), p.bias_f32 ? p.bias_f32[j] : 0.f,
                                          p.bias_f32 != nullptr, p, p.accumulate ? ((float *)D)[idx + c] : 0.f));
    }
    if (EPI == EPI_FIXEDPOINT)
    {
        if (vec)
            *(uint32_t *)(D + idx) = ((uint32_t)o[0] & 0xFFu) | (((uint32_t)o[1] & 0xFFu) << 8) | (((uint32_t)o[2] & 0xFFu) << 16) |
                                     (((uint32_t)o[3] & 0xFFu) << 24);
        else
            for (int c = 0; c < 4 && j0 + c < g.N; ++c)
                D[idx + c] = (char)o[c];
    }
    else
    {
        if (vec)
            *(v4i *)((int32_t *)D + idx) = o;
        else
            for (int c = 0; c < 4 && j0 + c < g.N; ++c)
                ((int32_t *)D)[idx + c] = o[c];
    }
}
int splitk_finish_launch(int epi, const GemmArgs &g, const int32_t *parts, int64_t plane, int ldp, int splits, hipStream_t s)
{
    if (g.M < 1 || g.N < 1 || splits < 1 || ldp % 4 != 0 || plane % 4 != 0 || ((uintptr_t)parts & 15) != 0 || g.epi.colvec == nullptr)
        return (int)hipErrorInvalidValue;
    const int64_t  n = (int64_t)g.M * ((g.N + 3) / 4);
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (epi == EPI_FIXEDPOINT)
        splitk_finish_kernel<EPI_FIXEDPOINT><<<dim3(blocks), dim3(256), 0, s>>>(parts, plane, ldp, splits, g);
    else if (epi == EPI_S32)
        splitk_finish_kernel<EPI_S32><<<dim3(blocks), dim3(256), 0, s>>>(parts, plane, ldp, splits, g);
    else if (epi == EPI_F32)
        splitk_finish_kernel<EPI_F32><<<dim3(blocks), dim3(256), 0, s>>>(parts, plane, ldp, splits, g);
    else
        return (int)hipErrorInvalidValue;
    return launch_status();
}

// ---- P1: B[K][ldb] -> Bp[Np][Kp] (transpose to K-contiguous, optional sign flip, zero padding) + column sums ----------
// Replaces pretranspose_B_array (src/cpu/operators/internal/CpuGemmAssemblyDispatch.cpp:594-617) / CpuGemmTranspose1xWKernel and
// CpuGemmLowpMatrixBReductionKernel (src/cpu/kernels/CpuGemmLowpMatrixReductionKernel.cpp:273-446) in one pass over B.
// kf > 1 re-orders K on the way: packed row k = a*kf + b (b < kf) is source row b*(K/kf) + a, which is what
// CpuConvertFullyConnectedWeightsKernel does to weights trained in the other data layout
// (src/cpu/kernels/CpuConvertFullyConnectedWeightsKernel.cpp:60-66,118-121 with kf = its _factor2).
__device__ __forceinline__ int k_source(int k, int K, int kf)
{
    return kf > 1 ? (k % kf) * (K / kf) + k / kf : k;
}

__global__ __launch_bounds__(256) void pack_b_kernel(const uint8_t *__restrict__ B, int64_t ldb, int K, int N, int Kp,
                                                     uint8_t flip, int kf, int8_t *__restrict__ Bp,
                                                     int32_t *__restrict__ colsum)
{
    __shared__ __attribute__((aligned(16))) uint8_t tile[64][64 + 16]; // [n][k]
    const int          n0 = blockIdx.x * 64, k0 = blockIdx.y * 64;
    const int          tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
    for (int kk = 0; kk < 16; ++kk)
    {
        const int k = k0 + ty * 16 + kk, n = n0 + tx;
        uint8_t   v = 0;
        if (k < K && n < N)
            v = B[(int64_t)k_source(k, K, kf) * ldb + n] ^ flip;
        tile[tx][ty * 16 + kk] = v;
    }
    __syncthreads();
    const int n = threadIdx.x >> 2, kc = (threadIdx.x & 3) * 16;
    const v4i v = *(const v4i *)&tile[n][kc];
    *(v4i *)(Bp + (int64_t)(n0 + n) * Kp + k0 + kc) = v;
    int32_t s = sum4_i8(v.x) + sum4_i8(v.y) + sum4_i8(v.z) + sum4_i8(v.w);
    s += __shfl_xor(s, 1);
    s += __shfl_xor(s, 2);
    if ((threadIdx.x & 3) == 0 && s != 0)
        atomicAdd(colsum + n0 + n, s);
}

int pack_b_launch(const void *B, int64_t ldb, int K, int N, int Kp, int Np, bool flip, int kf, int8_t *Bp,
                  int32_t *colsum, hipStream_t s)
{
    if (Np % 64 || Kp % 64 || Np < N || Kp < K || (kf > 1 && K % kf != 0))
        return (int)hipErrorInvalidValue;
    int e = fill_i32_launch(colsum, 0, Np, s);
    if (e)
        return e;
    pack_b_kernel<<<dim3(Np / 64, Kp / 64), dim3(256), 0, s>>>((const uint8_t *)B, ldb, K, N, Kp, flip ? 0x80 : 0, kf,
                                                               Bp, colsum);
    return launch_status();
}

// B already K-contiguous: Bt[N][ldk] (convolution weights [OFM][KH*KW*C], the layout CpuWeightsReshapeKernel
// produces transposed: src/cpu/kernels/CpuWeightsReshapeKernel.cpp:150-166)
__global__ __launch_bounds__(256) void pack_bt_kernel(const uint8_t *__restrict__ Bt, int64_t ldk, int K, int N, int Kp,
                                                      int Np, uint8_t flip, int kf, int8_t *__restrict__ Bp,
                                                      int32_t *__restrict__ colsum)
{
    const int     cpr = Kp / 16;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)Np * cpr)
        return;
    const int n = (int)(idx / cpr), kc = (int)(idx % cpr) * 16;
    union
    {
        v4i     v;
        uint8_t b[16];
    } u;
    int32_t        s   = 0;
    const uint8_t *row = Bt + (int64_t)n * ldk + kc;
    if (n < N && kc + 16 <= K && (((uintptr_t)row) & 15) == 0 && kf <= 1)
    {
        // whole aligned 16-byte piece of a row
        u.v = *(const v4i *)row;
        const int f4 = (int)(flip * 0x01010101u);
#pragma unroll
        for (int t = 0; t < 4; ++t)
            u.v[t] ^= f4;
#pragma unroll
        for (int t = 0; t < 16; ++t)
            s += (int8_t)u.b[t];
    }
    else
    {
#pragma unroll
        for (int t = 0; t < 16; ++t)
        {
            uint8_t x = 0;
            if (n < N && kc + t < K)
                x = Bt[(int64_t)n * ldk + k_source(kc + t, K, kf)] ^ flip;
            u.b[t] = x;
            s += (int8_t)x;
        }
    }
    *(v4i *)(Bp + (int64_t)n * Kp + kc) = u.v;
    if (s != 0)
        atomicAdd(colsum + n, s);
}

int pack_bt_launch(const void *Bt, int64_t ldk, int K, int N, int Kp, int Np, bool flip, int kf, int8_t *Bp,
                   int32_t *colsum, hipStream_t s)
{
    if (Kp % 16 || Np < N || Kp < K || (kf > 1 && K % kf != 0))
        return (int)hipErrorInvalidValue;
    int e = fill_i32_launch(colsum, 0, Np, s);
    if (e)
        return e;
    const int64_t total = (int64_t)Np * (Kp / 16);
    pack_bt_kernel<<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s>>>((const uint8_t *)Bt, ldk, K, N, Kp, Np,
                                                                               flip ? 0x80 : 0, kf, Bp, colsum);
    return launch_status();
}

// Bp[Np][Kp] -> Bs[Np/16][Kp/64][64][16]: 1 KiB blocks holding 16 columns x 64 k in the lane order the 16x16x64 matrix
// instruction reads its B operand (lane l: column l%16, bytes 16*(l/16) .. +16 of the k block)
__global__ __launch_bounds__(256) void pack_b_skinny_kernel(const int8_t *__restrict__ Bp, int Kp, int Np,
                                                            int8_t *__restrict__ Bs)
{
    const int64_t idx   = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t total = (int64_t)Np * Kp / 16;
    if (idx >= total)
        return;
    const int     lane = (int)(idx & 63);
    const int64_t blk  = idx >> 6;
    const int     KB   = Kp / 64;
    const int     kb = (int)(blk % KB), ng = (int)(blk / KB);
    const int     col = lane & 15, kc = lane >> 4;
    *(v4i *)(Bs + idx * 16) = *(const v4i *)(Bp + (int64_t)(ng * 16 + col) * Kp + kb * 64 + kc * 16);
}

int pack_b_skinny_launch(const int8_t *Bp, int Kp, int Np, int8_t *Bs, hipStream_t s)
{
    if (Kp % 64 || Np % 16)
        return (int)hipErrorInvalidValue;
    const int64_t total = (int64_t)Np * Kp / 16;
    pack_b_skinny_kernel<<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s>>>(Bp, Kp, Np, Bs);
    return launch_status();
}

// Row sums of the patch matrix without the patch matrix: rowvec[m] = b_off * sum over the taps and channels of output
// pixel m of the (sign-normalised) source byte, the padding value where a tap lies outside the image - what
// CpuGemmLowpMatrixAReductionKernel computes from the im2col buffer
// (src/cpu/kernels/CpuGemmLowpMatrixReductionKernel.cpp:133-204). One thread per output pixel.
__global__ __launch_bounds__(256) void conv_rowsum_kernel(const uint8_t *__restrict__ src, ConvGeom g, int M, uint8_t flip,
                                                          uint32_t b_off, int32_t *__restrict__ rowvec)
{
    const int m = blockIdx.x * blockDim.x + threadIdx.x;
    if (m >= M)
        return;
    const int     ox = m % g.OW, t = m / g.OW, oy = t % g.OH, n = t / g.OH;
    const int     pad = (int8_t)((g.pad_word & 0xFFu) ^ flip);
    const int64_t img = (int64_t)n * g.H * g.W * g.C;
    int32_t       sum = 0;
    for (int ky = 0; ky < g.KH; ++ky)
        for (int kx = 0; kx < g.KW; ++kx)
        {
            const int iy = oy * g.stride_y - g.pad_top + ky * g.dil_y, ix = ox * g.stride_x - g.pad_left + kx * g.dil_x;
            if (iy < 0 || iy >= g.H || ix < 0 || ix >= g.W)
            {
                sum += pad * g.C;
                continue;
            }
            const uint8_t *p = src + img + ((int64_t)iy * g.W + ix) * g.C;
            int            c = 0;
            if ((((uintptr_t)p) & 3) == 0)
                for (; c + 4 <= g.C; c += 4)
                {
                    const uint32_t w = *(const uint32_t *)(p + c) ^ (flip * 0x01010101u);
                    sum += (int8_t)(w & 0xFF) + (int8_t)((w >> 8) & 0xFF) + (int8_t)((w >> 16) & 0xFF) + (int8_t)(w >> 24);
                }
            for (; c < g.C; ++c)
                sum += (int8_t)(p[c] ^ flip);
        }
    rowvec[m] = (int32_t)(b_off * (uint32_t)sum);
}

// g.pad_word: the raw padding byte replicated
int conv_rowsum_launch(const void *src, const ConvGeom &g, int M, bool flip, int32_t b_off, int32_t *rowvec, hipStream_t s)
{
    conv_rowsum_kernel<<<dim3((M + 255) / 256), dim3(256), 0, s>>>((const uint8_t *)src, g, M, flip ? 0x80 : 0, (uint32_t)b_off,
                                                                  rowvec);
    return launch_status();
}

// The first `rows` (a multiple of 64) rows of Bp as the narrow kernel keeps them in LDS: rows of `chunks` 16-byte pieces of data plus
// NARROW_PAD_PIECES of padding, zero beyond Kp - the workgroups copy this image into LDS with plain linear transfers
__global__ __launch_bounds__(256) void pack_b_narrow_kernel(const int8_t *__restrict__ Bp, int Kp, int chunks, int rows,
                                                            int8_t *__restrict__ Bn)
{
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    constexpr int PAD = NARROW_PAD_PIECES;
    if (idx >= rows * (chunks + PAD))
        return;
    const int r = idx / (chunks + PAD), c = idx - r * (chunks + PAD);
    v4i       v = {0, 0, 0, 0};
    if (c < chunks && c * 16 < Kp)
        v = *(const v4i *)(Bp + (int64_t)r * Kp + c * 16);
    *(v4i *)(Bn + (int64_t)idx * 16) = v;
}

int pack_b_narrow_launch(const int8_t *Bp, int Kp, int Np, int chunks, int rows, int8_t *Bn, hipStream_t s)
{
    if (Kp % 16 || rows < 64 || rows % 64 != 0 || Np < rows || chunks < 1)
        return (int)hipErrorInvalidValue;
    pack_b_narrow_kernel<<<dim3((rows * (chunks + NARROW_PAD_PIECES) + 255) / 256), dim3(256), 0, s>>>(Bp, Kp, chunks, rows, Bn);
    return launch_status();
}

// colvec[j] = a_off*colsum[j] + a_off*b_off*K (+ bias[j]); the per-column part of the offset contribution, folded with the
// bias like arm_gemm's col_bias (src/core/NEON/kernels/arm_gemm/quantized.cpp:963-968)
__global__ void colvec_kernel(const int32_t *__restrict__ colsum, const int32_t *__restrict__ bias, uint32_t a_off,
                              uint32_t b_off, uint32_t K, int N, int32_t *__restrict__ colvec)
{
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= N)
        return;
    uint32_t v = a_off * (uint32_t)colsum[j] + a_off * b_off * K;
    if (bias)
        v += (uint32_t)bias[j];
    colvec[j] = (int32_t)v;
}

int colvec_launch(const int32_t *colsum, const int32_t *bias, int32_t a_off, int32_t b_off, int K, int N,
                  int32_t *colvec, hipStream_t s)
{
    colvec_kernel<<<dim3((N + 255) / 256), dim3(256), 0, s>>>(colsum, bias, (uint32_t)a_off, (uint32_t)b_off,
                                                              (uint32_t)K, N, colvec);
    return launch_status();
}

// Digest (multiplier, shift) per column into the QP_* vectors of epilogue.hpp; *neg is set when a multiplier is negative
// (then the branch-free form does not apply). mult / shift may be nullptr: per-tensor values mult_s / shift_s.
__global__ void qparams_kernel(const int32_t *__restrict__ mult, const int32_t *__restrict__ shift, int32_t mult_s,
                               int32_t shift_s, int N, int Np, int32_t *__restrict__ qp, int32_t *__restrict__ neg)
{
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= Np)
        return;
    int32_t m = 0, s = 0;
    if (j < N)
    {
        m = mult ? mult[j] : mult_s;
        s = shift ? shift[j] : shift_s;
    }
    if (m < 0)
        atomicOr(neg, 1);
    if (j < N && !(m >= 0x40000000 && s >= 2 && s < 32))
        atomicOr(neg, 2); // not the common case (normalised multiplier, right shift by 2 or more)
    if (s >= 32 || s <= -32)
        m = 0, s = 0; // the reference arithmetic yields 0 for these
    const uint32_t m2          = (uint32_t)m << 1;
    qp[QP_S2 * (int64_t)Np + j]    = (int32_t)m2;
    qp[QP_CMASK * (int64_t)Np + j] = ((uint32_t)m >= 0x40000000u) ? -1 : 0;
    qp[QP_LS * (int64_t)Np + j]    = s < 0 ? -s : 0;
    qp[QP_RSM1 * (int64_t)Np + j]  = s > 1 ? s - 1 : 0;
    qp[QP_RMASK * (int64_t)Np + j] = s > 0 ? 1 : 0;
}

int qparams_launch(const int32_t *mult, const int32_t *shift, int32_t mult_s, int32_t shift_s, int N, int Np,
                   int32_t *qp, int32_t *neg, hipStream_t s)
{
    int e = fill_i32_launch(neg, 0, 1, s);
    if (e)
        return e;
    qparams_kernel<<<dim3((Np + 255) / 256), dim3(256), 0, s>>>(mult, shift, mult_s, shift_s, N, Np, qp, neg);
    return launch_status();
}

// ---- A pre-pass -----------------------------------------------------------------------------------------------------
// One block per row. Optionally writes the row sign-flipped and zero-padded to Kp (for A whose rows are not 16-byte
// aligned), optionally reduces it: rowvec[i] = b_off * sum_k flip(A[i][k])
// (CpuGemmLowpMatrixAReductionKernel, src/cpu/kernels/CpuGemmLowpMatrixReductionKernel.cpp:133-204).
template <int VEC>
__global__ __launch_bounds__(256) void a_prepass_kernel(const uint8_t *__restrict__ A, int64_t lda, int64_t a_bs, int K, uint8_t flip,
                                                        int8_t *__restrict__ Ap, int Kp, int32_t *__restrict__ rowvec,
                                                        uint32_t b_off)
{
    // (grid: rows x batch entries; the copies and the sums of the entries lie one after the other)
    const int      row  = blockIdx.y * gridDim.x + blockIdx.x;
    const uint8_t *src  = A + (int64_t)blockIdx.y * a_bs + (int64_t)blockIdx.x * lda;
    const int      kmax = Ap ? Kp : K;
    int32_t        s    = 0;
    for (int k = threadIdx.x * VEC; k < kmax; k += 256 * VEC)
    {
        union
        {
            uint8_t  b[VEC];
            uint32_t w[VEC >= 4 ? VEC / 4 : 1];
        } u;
        if (k < K)
        {
            if (VEC == 1)
                u.b[0] = src[k] ^ flip;
            else
            {
#pragma unroll
                for (int t = 0; t < VEC / 4; ++t)
                    u.w[t] = *(const uint32_t *)(src + k + 4 * t) ^ (flip * 0x01010101u);
            }
        }
        else
        {
#pragma unroll
            for (int t = 0; t < (VEC >= 4 ? VEC / 4 : 1); ++t)
                u.w[t] = 0;
            if (VEC == 1)
                u.b[0] = 0;
        }
        if (VEC == 1)
            s += (int8_t)u.b[0];
        else
        {
#pragma unroll
            for (int t = 0; t < VEC / 4; ++t)
                s += sum4_i8((int32_t)u.w[t]);
        }
        if (Ap)
        {
            if (VEC == 1)
                Ap[(int64_t)row * Kp + k] = (int8_t)u.b[0];
            else
            {
#pragma unroll
                for (int t = 0; t < VEC / 4; ++t)
                    *(uint32_t *)(Ap + (int64_t)row * Kp + k + 4 * t) = u.w[t];
            }
        }
    }
    if (rowvec)
    {
        __shared__ int32_t part[4];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1)
            s += __shfl_xor(s, o);
        if ((threadIdx.x & 63) == 0)
            part[threadIdx.x >> 6] = s;
        __syncthreads();
        if (threadIdx.x == 0)
            rowvec[row] = (int32_t)(b_off * (uint32_t)(part[0] + part[1] + part[2] + part[3]));
    }
}

int a_prepass_launch(const void *A, int64_t lda, int64_t a_bs, int batch, int M, int K, bool flip, int8_t *Ap, int Kp,
                     int32_t *rowvec, int32_t b_off, hipStream_t s)
{
    if (M <= 0 || batch <= 0)
        return 0;
    if (batch > 65535)
        return (int)hipErrorInvalidValue;
    const uintptr_t mix  = (uintptr_t)A | (uintptr_t)lda | (uintptr_t)K | (batch > 1 ? (uintptr_t)a_bs : 0);
    const uint8_t   f    = flip ? 0x80 : 0;
    const dim3      grid(M, batch), block(256);
    if ((mix & 15) == 0)
        a_prepass_kernel<16><<<grid, block, 0, s>>>((const uint8_t *)A, lda, a_bs, K, f, Ap, Kp, rowvec, (uint32_t)b_off);
    else if ((mix & 7) == 0)
        a_prepass_kernel<8><<<grid, block, 0, s>>>((const uint8_t *)A, lda, a_bs, K, f, Ap, Kp, rowvec, (uint32_t)b_off);
    else if ((mix & 3) == 0)
        a_prepass_kernel<4><<<grid, block, 0, s>>>((const uint8_t *)A, lda, a_bs, K, f, Ap, Kp, rowvec, (uint32_t)b_off);
    else
        a_prepass_kernel<1><<<grid, block, 0, s>>>((const uint8_t *)A, lda, a_bs, K, f, Ap, Kp, rowvec, (uint32_t)b_off);
    return launch_status();
}

// ---- K2: stand-alone output stage --------------------------------------------------------------------------------------
// CpuGemmLowpQuantizeDownInt32To{Int8,Uint8}ScaleByFixedPointKernel
// (src/cpu/kernels/CpuGemmLowpQuantizeDownInt32ToInt8ScaleByFixedPointKernel.cpp:79-181): 4 B read + 1 B written per element
template <bool VEC4>
__global__ __launch_bounds__(256) void output_stage_kernel(const int32_t *__restrict__ src, int64_t ld_src,
                                                           const int32_t *__restrict__ bias, int8_t *__restrict__ dst,
                                                           int64_t ld_dst, int M, int N, EpiParams p)
{
    const int     per_row = VEC4 ? N / 4 : N;
    const int64_t idx     = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)M * per_row)
        return;
    const int i = (int)(idx / per_row), q = (int)(idx % per_row);
    if (VEC4)
    {
        const int j = q * 4;
        v4i       v = *(const v4i *)(src + (int64_t)i * ld_src + j);
        v4i       b = {0, 0, 0, 0};
        if (bias)
            b = *(const v4i *)(bias + j);
        uint32_t out = 0;
#pragma unroll
        for (int t = 0; t < 4; ++t)
        {
            const int32_t mu = p.mult ? p.mult[j + t] : p.mult_s;
            const int32_t sh = p.shift ? p.shift[j + t] : p.shift_s;
            out |= ((uint32_t)epi_fixedpoint(v[t], b[t], 0, mu, sh, p) & 0xFFu) << (8 * t);
        }
        *(uint32_t *)(dst + (int64_t)i * ld_dst + j) = out;
    }
    else
    {
        const int32_t mu = p.mult ? p.mult[q] : p.mult_s;
        const int32_t sh = p.shift ? p.shift[q] : p.shift_s;
        dst[(int64_t)i * ld_dst + q] =
            (int8_t)epi_fixedpoint(src[(int64_t)i * ld_src + q], bias ? bias[q] : 0, 0, mu, sh, p);
    }
}

// CpuGemmLowpQuantizeDownInt32ToInt16ScaleByFixedPointKernel
// (src/cpu/kernels/CpuGemmLowpQuantizeDownInt32ToInt16ScaleByFixedPointKernel.cpp:76-200): 4 B read + 2 B written per element
template <bool VEC4>
__global__ __launch_bounds__(256) void output_stage_s16_kernel(const int32_t *__restrict__ src, int64_t ld_src,
                                                               const int32_t *__restrict__ bias, int16_t *__restrict__ dst,
                                                               int64_t ld_dst, int M, int N, EpiParams p)
{
    const int     per_row = VEC4 ? N / 4 : N;
    const int64_t idx     = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)M * per_row)
        return;
    const int i = (int)(idx / per_row), q = (int)(idx % per_row);
    if (VEC4)
    {
        typedef short v4s __attribute__((ext_vector_type(4)));
        const int j = q * 4;
        v4i       v = *(const v4i *)(src + (int64_t)i * ld_src + j);
        v4i       b = {0, 0, 0, 0};
        if (bias)
            b = *(const v4i *)(bias + j);
        v4s o;
#pragma unroll
        for (int t = 0; t < 4; ++t)
            o[t] = (short)requant_fixedpoint_s16((int32_t)((uint32_t)v[t] + (uint32_t)b[t]), p.mult_s, p.shift_s, p.lo, p.hi);
        *(v4s *)(dst + (int64_t)i * ld_dst + j) = o;
    }
    else
        dst[(int64_t)i * ld_dst + q] = (int16_t)requant_fixedpoint_s16(
            (int32_t)((uint32_t)src[(int64_t)i * ld_src + q] + (uint32_t)(bias ? bias[q] : 0)), p.mult_s, p.shift_s, p.lo, p.hi);
}

int output_stage_s16_launch(const int32_t *src, int64_t ld_src, const int32_t *bias, void *dst, int64_t ld_dst, int M,
                            int N, const EpiParams &epi, hipStream_t s)
{
    if (M <= 0 || N <= 0)
        return 0;
    const bool vec = (N % 4 == 0) && (ld_src % 4 == 0) && (ld_dst % 4 == 0) && (((uintptr_t)src & 15) == 0) &&
                     (((uintptr_t)dst & 7) == 0) && (bias == nullptr || ((uintptr_t)bias & 15) == 0);
    const int64_t total = (int64_t)M * (vec ? N / 4 : N);
    const dim3    grid((unsigned)((total + 255) / 256)), block(256);
    if (vec)
        output_stage_s16_kernel<true><<<grid, block, 0, s>>>(src, ld_src, bias, (int16_t *)dst, ld_dst, M, N, epi);
    else
        output_stage_s16_kernel<false><<<grid, block, 0, s>>>(src, ld_src, bias, (int16_t *)dst, ld_dst, M, N, epi);
    return launch_status();
}

int output_stage_launch(const int32_t *src, int64_t ld_src, const int32_t *bias, void *dst, int64_t ld_dst, int M,
                        int N, const EpiParams &epi, hipStream_t s)
{
    if (M <= 0 || N <= 0)
        return 0;
    const bool vec = (N % 4 == 0) && (ld_src % 4 == 0) && (ld_dst % 4 == 0) && (((uintptr_t)src & 15) == 0) &&
                     (((uintptr_t)dst & 3) == 0) && (bias == nullptr || ((uintptr_t)bias & 15) == 0);
    const int64_t total = (int64_t)M * (vec ? N / 4 : N);
    const dim3    grid((unsigned)((total + 255) / 256)), block(256);
    if (vec)
        output_stage_kernel<true><<<grid, block, 0, s>>>(src, ld_src, bias, (int8_t *)dst, ld_dst, M, N, epi);
    else
        output_stage_kernel<false><<<grid, block, 0, s>>>(src, ld_src, bias, (int8_t *)dst, ld_dst, M, N, epi);
    return launch_status();
}

// ---- explicit im2col (NHWC) ----------------------------------------------------------------------------------------------
// CpuIm2ColKernel / linearize_volume_nhwc (src/cpu/kernels/directconv2d/impl.h:148-220,307-389). Used when the implicit
// loader does not apply (channel count not a multiple of 16, asymmetric weights) and exported on its own.
template <int VEC>
__global__ __launch_bounds__(256) void im2col_nhwc_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                          int64_t rows, ConvGeom g, int64_t ld_dst)
{
    const int     K    = g.KH * g.KW * g.C;
    const int     upr  = K / VEC; // units per row
    const int64_t idx  = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows * upr)
        return;
    const int64_t m = idx / upr;
    const int     k = (int)(idx % upr) * VEC;
    const int     tap = k / g.C, c0 = k - tap * g.C;
    const int     ky = tap / g.KW, kx = tap - ky * g.KW;
    const int     ox = (int)(m % g.OW);
    const int64_t t  = m / g.OW;
    const int     oy = (int)(t % g.OH);
    const int64_t n  = t / g.OH;
    const int     iy = oy * g.stride_y - g.pad_top + ky * g.dil_y;
    const int     ix = ox * g.stride_x - g.pad_left + kx * g.dil_x;
    const bool    in = iy >= 0 && iy < g.H && ix >= 0 && ix < g.W;
    const uint8_t *s = src + ((n * g.H + iy) * g.W + ix) * g.C + c0;
    uint8_t       *d = dst + m * ld_dst + k;
    if (VEC == 16)
    {
        const int pw = (int)g.pad_word;
        v4i       v  = {pw, pw, pw, pw};
        if (in)
            v = *(const v4i *)s;
        *(v4i *)d = v;
    }
    else
        *d = in ? *s : (uint8_t)(g.pad_word & 0xFF);
}

int im2col_nhwc_launch(const void *src, void *dst, int batch, const ConvGeom &g, int64_t ld_dst, hipStream_t s)
{
    const int64_t rows = (int64_t)batch * g.OH * g.OW;
    const int     K    = g.KH * g.KW * g.C;
    if (rows <= 0 || K <= 0)
        return 0;
    const bool vec = (g.C % 16 == 0) && (((uintptr_t)src & 15) == 0) && (((uintptr_t)dst & 15) == 0) &&
                     (ld_dst % 16 == 0);
    const int64_t total = rows * (vec ? K / 16 : K);
    const dim3    grid((unsigned)((total + 255) / 256)), block(256);
    if (vec)
        im2col_nhwc_kernel<16><<<grid, block, 0, s>>>((const uint8_t *)src, (uint8_t *)dst, rows, g, ld_dst);
    else
        im2col_nhwc_kernel<1><<<grid, block, 0, s>>>((const uint8_t *)src, (uint8_t *)dst, rows, g, ld_dst);
    return launch_status();
}

// ---- matrix transpose of bytes or 32-bit words: [batch][R][C] -> [batch][C][R] --------------------------------------
// The NCHW <-> NHWC conversions around the NHWC convolution kernel (one image is a C x HW matrix of bytes, or of floats
// for the dequantised destination) and of NCHW weights ([OFM][C][KH*KW] -> [OFM][KH*KW][C]). 64 x 64 tiles through LDS
// so that reads and writes both run along rows.
template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(const T *__restrict__ src, T *__restrict__ dst, int R, int C)
{
    __shared__ T tile[64][65];
    const int64_t      base = (int64_t)blockIdx.z * R * C;
    const int          r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const int          tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll 4
    for (int y = ty; y < 64; y += 4)
        if (r0 + y < R && c0 + tx < C)
            tile[y][tx] = src[base + (int64_t)(r0 + y) * C + c0 + tx];
    __syncthreads();
#pragma unroll 4
    for (int y = ty; y < 64; y += 4)
        if (c0 + y < C && r0 + tx < R)
            dst[base + (int64_t)(c0 + y) * R + r0 + tx] = tile[tx][y];
}

int transpose_bytes_launch(const void *src, void *dst, int batch, int R, int C, hipStream_t s)
{
    if (batch <= 0 || R <= 0 || C <= 0)
        return 0;
    if (batch > 65535 || (R + 63) / 64 > 65535)
        return (int)hipErrorInvalidValue;
    const dim3 grid((unsigned)((C + 63) / 64), (unsigned)((R + 63) / 64), (unsigned)batch), block(256);
    transpose_kernel<uint8_t><<<grid, block, 0, s>>>((const uint8_t *)src, (uint8_t *)dst, R, C);
    return launch_status();
}

int transpose_words_launch(const void *src, void *dst, int batch, int R, int C, hipStream_t s)
{
    if (batch <= 0 || R <= 0 || C <= 0)
        return 0;
    if (batch > 65535 || (R + 63) / 64 > 65535)
        return (int)hipErrorInvalidValue;
    const dim3 grid((unsigned)((C + 63) / 64), (unsigned)((R + 63) / 64), (unsigned)batch), block(256);
    transpose_kernel<uint32_t><<<grid, block, 0, s>>>((const uint32_t *)src, (uint32_t *)dst, R, C);
    return launch_status();
}

// ---- segment gather / scatter between two stride sets ------------------------------------------------------------------
// Segment (i1, i2, i3) of seg bytes lives at i1*st[0] + i2*st[1] + i3*st[2] on either side: tensors that carry padding
// (along the channel dimension, between rows, between planes or images; ITensorInfo::strides_in_bytes()) to dense and back.
__global__ __launch_bounds__(256) void restride_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                       int64_t total, int seg, int64_t n1, int64_t n2, RestrideSteps ss,
                                                       RestrideSteps ds)
{
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total)
        return;
    const int64_t sgm = idx / seg;
    const int     c   = (int)(idx - sgm * seg);
    const int64_t q1  = sgm / n1, i1 = sgm - q1 * n1;
    const int64_t i3 = q1 / n2, i2 = q1 - i3 * n2;
    dst[i1 * ds.st[0] + i2 * ds.st[1] + i3 * ds.st[2] + c] = src[i1 * ss.st[0] + i2 * ss.st[1] + i3 * ss.st[2] + c];
}

int restride_nd_launch(const void *src, void *dst, int seg, int64_t n1, int64_t n2, int64_t n3, const RestrideSteps &ss,
                       const RestrideSteps &ds, hipStream_t s)
{
    if (seg <= 0 || n1 <= 0 || n2 <= 0 || n3 <= 0)
        return 0;
    const int64_t total = n1 * n2 * n3 * seg;
    if ((total + 255) / 256 > 0x7FFFFFFF)
        return (int)hipErrorInvalidValue;
    restride_kernel<<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s>>>((const uint8_t *)src, (uint8_t *)dst, total,
                                                                                 seg, n1, n2, ss, ds);
    return launch_status();
}

int restride_launch(const void *src, void *dst, int64_t segments, int seg, int64_t src_stride, int64_t dst_stride,
                    hipStream_t s)
{
    return restride_nd_launch(src, dst, seg, segments, 1, 1, RestrideSteps{{src_stride, 0, 0}}, RestrideSteps{{dst_stride, 0, 0}}, s);
}

// ---- F16 destinations: [batch][M][N] halfs with row / batch strides <- the dense F32 matrix the GEMM kernels write --------
// Conversion to half rounds to nearest even (the reference's host-side half type is configured the same way,
// support/Half.h:33-34). Accumulating: the rounded half is added to the previous half as the reference's test oracle
// adds halfs (both widened, one float addition, rounded again; tests/validation/fixtures/GEMMLowpFixture.h:912-918),
// and the activation clamp follows the addition.
__global__ __launch_bounds__(256) void f32_to_f16_kernel(const float *__restrict__ f, _Float16 *__restrict__ h,
                                                         int64_t total, int M, int N, int64_t ldh, int64_t h_batch_stride,
                                                         int accumulate, float act_min, float act_max)
{
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total)
        return;
    const int64_t row = idx / N;
    const int     j   = (int)(idx - row * N);
    const int64_t bz  = row / M;
    const int     i   = (int)(row - bz * M);
    const int64_t hi  = bz * h_batch_stride + (int64_t)i * ldh + j;
    _Float16      v   = (_Float16)f[idx];
    if (accumulate)
    {
        const float sum = (float)h[hi] + (float)v;
        v               = (_Float16)fminf(fmaxf(sum, act_min), act_max);
    }
    h[hi] = v;
}

int f32_to_f16_launch(const float *dense_f32, void *half_matrix, int batch, int M, int N, int64_t ldh,
                      int64_t h_batch_stride, bool accumulate, float act_min, float act_max, hipStream_t s)
{
    const int64_t total = (int64_t)batch * M * N;
    if (total <= 0)
        return 0;
    if ((total + 255) / 256 > 0x7FFFFFFF)
        return (int)hipErrorInvalidValue;
    f32_to_f16_kernel<<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s>>>(
        dense_f32, (_Float16 *)half_matrix, total, M, N, ldh, h_batch_stride, accumulate ? 1 : 0, act_min, act_max);
    return launch_status();
}

// ---- one thread per output: the plainest possible statement of the path, for cross-checking only ----------------------
template <int EPI>
__global__ __launch_bounds__(256) void simple_gemm_kernel(GemmArgs g, uint8_t flip)
{
    const int j = blockIdx.x * 16 + (threadIdx.x & 15);
    const int i = blockIdx.y * 16 + (threadIdx.x >> 4);
    const int bz = blockIdx.z;
    if (i >= g.M || j >= g.N)
        return;
    const uint8_t *a = (const uint8_t *)g.A + (int64_t)bz * g.a_batch_stride + (int64_t)i * g.lda;
    const int8_t  *b = g.Bp + (int64_t)bz * g.bp_batch_stride + (int64_t)j * g.Kp;
    int32_t        acc = 0;
    for (int k = 0; k < g.K; ++k)
        acc += (int32_t)(int8_t)(a[k] ^ flip) * (int32_t)b[k];
    const EpiParams &p   = g.epi;
    const int32_t    cv  = p.colvec[(int64_t)bz * p.colvec_batch_stride + j];
    const int32_t    rv  = p.rowvec ? p.rowvec[(int64_t)bz * p.rowvec_batch_stride + i] : 0;
    const int64_t    idx = (int64_t)bz * g.d_batch_stride + (int64_t)i * g.ldd + j;
    if (EPI == EPI_S32)
        ((int32_t *)g.D)[idx] = (int32_t)((uint32_t)acc + (uint32_t)cv + (uint32_t)rv +
                                          (p.accumulate ? (uint32_t)((int32_t *)g.D)[idx] : 0u));
    else if (EPI == EPI_FIXEDPOINT)
        ((int8_t *)g.D)[idx] =
            (int8_t)epi_fixedpoint(acc, cv, rv, p.mult ? p.mult[j] : p.mult_s, p.shift ? p.shift[j] : p.shift_s, p);
    else
        ((float *)g.D)[idx] = epi_f32(acc, (int32_t)((uint32_t)cv + (uint32_t)rv), p.bias_f32 ? p.bias_f32[j] : 0.f,
                                      p.bias_f32 != nullptr, p, p.accumulate ? ((float *)g.D)[idx] : 0.f);
}

int simple_gemm_launch(int epi, bool flip_a, const GemmArgs &args, int batch, hipStream_t s)
{
    const dim3    grid((args.N + 15) / 16, (args.M + 15) / 16, batch), block(256);
    const uint8_t f = flip_a ? 0x80 : 0;
    if (epi == EPI_S32)
        simple_gemm_kernel<EPI_S32><<<grid, block, 0, s>>>(args, f);
    else if (epi == EPI_FIXEDPOINT)
        simple_gemm_kernel<EPI_FIXEDPOINT><<<grid, block, 0, s>>>(args, f);
    else
        simple_gemm_kernel<EPI_F32><<<grid, block, 0, s>>>(args, f);
    return launch_status();
}
// ---- runs of C bytes -> runs of Cp >= C bytes (the first C copied, the rest set to `fill`): pixels of an NHWC image or
// taps of OHWI weights whose channel count the 16-byte loaders cannot take, padded to the next multiple of 16. The
// channels added meet weights that are zero in the kernels' signed form, so they change no sum. One thread per
// 16 bytes of output.
__global__ __launch_bounds__(256) void channel_pad_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, int64_t runs, int C,
                                                          int Cp, uint32_t fill)
{
    typedef int v4i __attribute__((ext_vector_type(4)));
    const int     per = Cp / 16;
    const int64_t t   = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= runs * per)
        return;
    const int64_t  r  = t / per;
    const int      c0 = (int)(t - r * per) * 16;
    const uint8_t *in = src + r * C + c0;
    uint32_t       w[4];
#pragma unroll
    for (int q = 0; q < 4; ++q)
    {
        w[q] = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b)
        {
            const int c = c0 + q * 4 + b;
            w[q] |= (uint32_t)(c < C ? in[q * 4 + b] : (uint8_t)fill) << (8 * b);
        }
    }
    *(v4i *)(dst + r * Cp + c0) = (v4i){(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
}
int channel_pad_launch(const void *src, void *dst, int64_t runs, int C, int Cp, uint8_t fill, hipStream_t s)
{
    if (runs <= 0)
        return 0;
    if (C < 1 || Cp < C || Cp % 16 != 0 || ((uintptr_t)dst & 15) != 0)
        return (int)hipErrorInvalidValue;
    const int64_t n = runs * (Cp / 16);
    if ((n + 255) / 256 > 0x7fffffff)
        return (int)hipErrorInvalidValue;
    channel_pad_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s>>>((const uint8_t *)src, (uint8_t *)dst, runs, C, Cp, fill);
    return launch_status();
}

} // namespace mi355
