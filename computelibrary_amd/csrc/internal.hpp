// Declarations shared between the C-ABI layer (capi.hip) and the kernel translation units.
#pragma once
#include "epilogue.hpp"

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi355
{
// Padding of the packed B matrix Bp[Np][Kp] (int8, K contiguous, zero filled beyond N and K)
constexpr int PACK_N_ALIGN = 256;
constexpr int PACK_K_ALIGN = 128;

inline int round_up(int v, int a)
{
    return (v + a - 1) / a * a;
}

// Geometry of the on-the-fly im2col A loader (implicit GEMM). row m = (n, oy, ox), k = (ky, kx, c).
struct ConvGeom
{
    int32_t H, W, C, KH, KW, OH, OW;
    int32_t stride_x, stride_y, pad_left, pad_top, dil_x, dil_y;
    uint32_t pad_word; // the padding byte (already sign-flipped if the loader flips) replicated into 4 bytes
    // floor(2^32 / d) + 1 for d = C, KW, OW, OH (0 when d == 1): x / d == mulhi(x, magic) exactly while x * d < 2^32
    uint32_t magic_C, magic_KW, magic_OW, magic_OH;
};

// x / d for the divisors above (see ConvGeom::magic_*); the caller guarantees x * d < 2^32
__device__ __forceinline__ int fast_div(int x, uint32_t magic)
{
    return magic ? (int)__umulhi((uint32_t)x, magic) : x;
}

struct GemmArgs
{
    const int8_t *A;  // dense: [batch][M][lda] ; conv: NHWC source
    const int8_t *Bp; // [batch?][Np][Kp]
    void         *D;
    int64_t       lda, a_batch_stride;
    int64_t       Kp, bp_batch_stride;
    int64_t       ldd, d_batch_stride;
    int32_t       M, N, K; // K: valid depth of A (bytes readable per row)
    int32_t       tiles_m, tiles_n;
    EpiParams     epi;
    ConvGeom      conv;
    const int8_t *fill16; // 16 readable bytes: what a staged 16-byte column reads where A has no data (zeros / pad value)
    const int8_t *a_end;  // dense A: one past the last byte of the last row of the last batch (no 16-byte read may cross it)
    // floor(2^32 / d) + 1 for d = tiles_m * tiles_n and d = 4 * tiles_n (see fast_div), valid for every tile id of the
    // launch; tile_magic_ok == 0: divide
    uint32_t magic_tiles, magic_group;
    int32_t  tile_magic_ok;
    int32_t  nblocks; // workgroups of the launch (gridDim.x is a hidden argument behind this block: one more fetch)
    // implicit convolution whose K range runs as slices (the batch entries of one launch): K values per slice, a whole
    // number of K steps; entry z covers k in [z * k_slice, (z + 1) * k_slice) of the patch and K holds k_slice. 0: no slices
    int32_t  k_slice;
    // dense A whose K ends inside the last K step, set by dma_launch: the batch entry in whose last row tile a 16-byte
    // column of that step could reach beyond a_end. Every other tile may fetch the step whole - the columns at and
    // beyond K then hold whatever follows in memory and meet the zero rows of the packed B. -1: no tile may.
    int32_t  lean_tail_bz;
};

struct MfmaConfig
{
    const char *name;
    int         BM, BN, BK;
    int         waves = 0, lds_bytes = 0; // per workgroup (filled in for the pipelined kernel's configurations)
};

typedef int v4i_t __attribute__((ext_vector_type(4)));

// 16 bytes of an A row of which only the first `rem` (0 < rem < 16) exist; p is 4-byte aligned. Bytes past the
// row's end read as zero (they meet the zero padding of the packed B, so their value is irrelevant, but the
// access itself must stay inside the tensor).
__device__ __forceinline__ v4i_t load16_partial(const int8_t *p, int rem)
{
    v4i_t v = {0, 0, 0, 0};
#pragma unroll
    for (int t = 0; t < 4; ++t)
    {
        const int r = rem - 4 * t;
        if (r >= 4)
            v[t] = *(const int *)(p + 4 * t);
        else if (r > 0)
        {
            uint32_t w = 0;
            for (int b = 0; b < r; ++b)
                w |= (uint32_t)(uint8_t)p[4 * t + b] << (8 * b);
            v[t] = (int)w;
        }
    }
    return v;
}

// gemm_mfma.hip
int         mfma_num_configs();
MfmaConfig  mfma_config(int idx);
// epi: EPI_*, flip_a: xor 0x80 on A bytes in the loader, conv: implicit-GEMM loader. Returns hipError_t as int.
int         mfma_launch(int cfg_idx, int epi, bool flip_a, bool conv, const GemmArgs &args, int batch, hipStream_t s);

// gemm_dma.hip — same contract as mfma_launch; additionally needs 16-byte aligned A rows, K % 16 == 0 and args.fill16
int         dma_num_configs();
MfmaConfig  dma_config(int idx);
int         dma_launch(int cfg_idx, int epi, bool flip_a, bool conv, const GemmArgs &args, int batch, hipStream_t s);

// gemm_narrow.hip — N <= 64, K <= 1152, 16-byte aligned operands: A straight from global memory into the matrix cores'
// operand layout, B resident in LDS; dense or implicit convolution (C % 16 == 0). needs args.fill16
// (args.Bp: the image written by pack_b_narrow_launch with narrow_panel_chunks(K) + NARROW_PAD_PIECES pieces per row)
int  narrow_panel_chunks(int K); // 0: K outside the kernel's range
// Pieces of padding after each row of that image. A ds_read_b128 goes through LDS in four batches of 16 lanes - lanes
// {0-3, 12-15, 20-23, 24-27}, {4-11, 16-19, 28-31} and the same of the upper half - and a batch is free of bank
// conflicts when its 16 addresses differ modulo 256 bytes: with lane l at row l % 16, piece l / 16 that holds for a row
// pitch of 32 modulo 64 bytes (measured: 2.8 clocks per instruction and compute unit against 4.6 with 16 modulo 64).
constexpr int NARROW_PAD_PIECES = 2;
bool narrow_applies(const GemmArgs &args, bool conv);
// *band (when given): whether the launch took the form that stages a band of input rows in LDS (large images)
int  narrow_launch(int epi, bool flip_a, bool conv, const GemmArgs &args, hipStream_t s, bool *band = nullptr);

// gemm_skinny.hip — M <= 64, B packed in matrix-core operand order (see pack_b_skinny)
constexpr int SKINNY_MAX_M = 64;
// *variant (when given): a static string naming the form of the kernel that ran
int skinny_launch(int epi, bool flip_a, const GemmArgs &args, int batch, hipStream_t s, const char **variant = nullptr);

// kernels_aux.hip
// B [K][ldb] (row-major, N contiguous) -> Bp [Np][Kp] int8 (flip: xor 0x80), colsum[Np] (sums of the packed int8 values)
int pack_b_launch(const void *B, int64_t ldb, int K, int N, int Kp, int Np, bool flip, int kf, int8_t *Bp, int32_t *colsum,
                  hipStream_t s);
// B given as [N][ldk] with K contiguous (conv weights [OFM][KH*KW*C])
int pack_bt_launch(const void *Bt, int64_t ldk, int K, int N, int Kp, int Np, bool flip, int kf, int8_t *Bp, int32_t *colsum,
                   hipStream_t s);
// Bp [Np][Kp] -> operand order for the skinny kernel: [Np/16][Kp/64][64 lanes][16 bytes]
int pack_b_skinny_launch(const int8_t *Bp, int Kp, int Np, int8_t *Bs, hipStream_t s);
// rows 0..63 of Bp -> [64][chunks + 1] pieces of 16 bytes (the last one padding), zero beyond Kp
int pack_b_narrow_launch(const int8_t *Bp, int Kp, int Np, int chunks, int rows, int8_t *Bn, hipStream_t s);
// colvec[j] = a_off*colsum[j] + a_off*b_off*K (+ bias[j])
int colvec_launch(const int32_t *colsum, const int32_t *bias, int32_t a_off, int32_t b_off, int K, int N,
                  int32_t *colvec, hipStream_t s);
// (multiplier, shift) per column -> qp[QP_COUNT][Np]; *neg != 0 afterwards if any multiplier is negative
int qparams_launch(const int32_t *mult, const int32_t *shift, int32_t mult_s, int32_t shift_s, int N, int Np,
                   int32_t *qp, int32_t *neg, hipStream_t s);
// A pre-pass over `batch` matrices a_bs bytes apart, one launch: optional padded + flipped copies Ap[batch][M][Kp]
// and/or rowvec[batch][M], rowvec[b][i] = b_off * sum_k(flip(A_b[i][k]))
int a_prepass_launch(const void *A, int64_t lda, int64_t a_bs, int batch, int M, int K, bool flip, int8_t *Ap, int Kp,
                     int32_t *rowvec, int32_t b_off, hipStream_t s);
// rowvec[m] = b_off * (sum of the sign-normalised patch of output pixel m); g.pad_word = the raw padding byte, replicated
int conv_rowsum_launch(const void *src, const ConvGeom &g, int M, bool flip, int32_t b_off, int32_t *rowvec, hipStream_t s);
int output_stage_launch(const int32_t *src, int64_t ld_src, const int32_t *bias, void *dst, int64_t ld_dst, int M,
                        int N, const EpiParams &epi, hipStream_t s);
// sum of `splits` S32 planes (M rows of ldp words, `plane` words apart) through epilogue `epi` of g into g.D
int splitk_finish_launch(int epi, const GemmArgs &g, const int32_t *parts, int64_t plane, int ldp, int splits, hipStream_t s);
int output_stage_s16_launch(const int32_t *src, int64_t ld_src, const int32_t *bias, void *dst, int64_t ld_dst, int M,
                            int N, const EpiParams &epi, hipStream_t s);
// [batch][R][C] bytes -> [batch][C][R]
int transpose_bytes_launch(const void *src, void *dst, int batch, int R, int C, hipStream_t s);
int transpose_words_launch(const void *src, void *dst, int batch, int R, int C, hipStream_t s);
// `runs` runs of C bytes -> runs of Cp bytes (Cp a multiple of 16): the first C copied, the rest set to `fill`
int channel_pad_launch(const void *src, void *dst, int64_t runs, int C, int Cp, uint8_t fill, hipStream_t s);
// dst[s * dst_stride + c] = src[s * src_stride + c] for s < segments, c < seg (bytes)
// dense F32 [batch][M][N] -> F16 destination (row stride ldh, batch stride, in elements), optionally added to its
// previous contents in half arithmetic and clamped
int f32_to_f16_launch(const float *dense_f32, void *half_matrix, int batch, int M, int N, int64_t ldh,
                      int64_t h_batch_stride, bool accumulate, float act_min, float act_max, hipStream_t s);
// compute units of the current device (0 when it cannot be asked)
int device_cus();
// byte steps of dimensions 1, 2 and 3 of a tensor whose dimension 0 is a run of contiguous bytes
struct RestrideSteps
{
    int64_t st[3];
};
int restride_nd_launch(const void *src, void *dst, int seg, int64_t n1, int64_t n2, int64_t n3, const RestrideSteps &ss,
                       const RestrideSteps &ds, hipStream_t s);
int restride_launch(const void *src, void *dst, int64_t segments, int seg, int64_t src_stride, int64_t dst_stride,
                    hipStream_t s);
int im2col_nhwc_launch(const void *src, void *dst, int batch, const ConvGeom &g, int64_t ld_dst, hipStream_t s);
// one thread per output; A dense [M][lda] (unflipped or flipped per flip_a), Bp packed
int simple_gemm_launch(int epi, bool flip_a, const GemmArgs &args, int batch, hipStream_t s);
int fill_i32_launch(int32_t *p, int32_t v, int64_t n, hipStream_t s);
} // namespace mi355
