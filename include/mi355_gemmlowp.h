/*
 * mi355_gemmlowp.h — C ABI of the MI355X (gfx950) quantized-GEMM path.
 *
 * This is the only boundary below which HIP is used. The C++ host layer that mirrors the
 * arm_compute function classes (NEGEMMLowpMatrixMultiplyCore, NEGEMMLowpOutputStage,
 * NEGEMMConvolutionLayer) calls these entry points; so can any other language through its FFI.
 *
 * The lifecycle follows the object the reference's operators drive for this path,
 * arm_gemm::GemmCommon (src/cpu/kernels/assembly/arm_gemm/gemm_common.hpp:56-302):
 *   configure -> pretranspose_B_array / set_quantized_bias -> set_arrays -> execute
 * becomes
 *   mi355_gemmlowp_create -> mi355_gemmlowp_prepare -> mi355_gemmlowp_run.
 *
 * Conventions
 *  - Matrices are row-major. A is M x K, B is K x N (or N x K with b_transposed), D is M x N ("ld*" = row stride in elements,
 *    "*_batch_stride" = distance between consecutive matrices in elements; b_batch_stride 0
 *    shares one B between all batches).
 *  - a_offset / b_offset are ADDED to every element before the product, exactly as
 *    NEGEMMLowpMatrixMultiplyCore treats QuantizationInfo::offset
 *    (arm_compute/runtime/NEON/functions/NEGEMMLowpMatrixMultiplyCore.h:95-97).
 *  - Every data pointer may be a host pointer or a device pointer; the library finds out with
 *    hipPointerGetAttributes. Host buffers are staged through device memory owned by the
 *    handle (synchronous, like the reference's run()); device buffers are used in place and
 *    the call only enqueues work on `stream` (a hipStream_t passed as void*, NULL = default
 *    stream). A handle asks once per pointer value and argument: it remembers which kind the
 *    value last given for A, D and the float bias was, until the handle is destroyed. If memory
 *    of one kind is freed and the SAME address comes back from an allocation of the other kind
 *    between two runs of one handle, pass a different address first or use a new handle.
 *  - All functions return 0 on success, non-zero on failure; mi355_last_error() then returns
 *    a thread-local message. No exception crosses this boundary.
 *  - A handle is single-caller: one call at a time per handle. Distinct handles may be used
 *    from distinct threads / streams.
 */
#ifndef MI355_GEMMLOWP_H
#define MI355_GEMMLOWP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum mi355_dtype
{
    MI355_U8  = 0, /* QASYMM8 */
    MI355_S8  = 1, /* QASYMM8_SIGNED, QSYMM8, QSYMM8_PER_CHANNEL */
    MI355_S32 = 2,
    MI355_F32 = 3,
    MI355_S16 = 4, /* QSYMM16: only as the destination of mi355_output_stage_run */
    MI355_F16 = 5  /* IEEE half: only as the destination of mi355_gemmlowp_run with MI355_EPI_F32 */
} mi355_dtype;

/* What happens to the int32 accumulators. Replaces the choice the reference makes between
 * CpuGemmLowpOffsetContributionKernel (S32 / F32) and
 * CpuGemmLowpOffsetContributionOutputStageKernel (src/cpu/operators/CpuGemmLowpMatrixMultiplyCore.cpp:281-321). */
typedef enum mi355_epilogue
{
    MI355_EPI_S32        = 0, /* dst = acc + offset contribution                       (int32) */
    MI355_EPI_FIXEDPOINT = 1, /* + bias, QUANTIZE_DOWN_FIXEDPOINT, clamp               (uint8 / int8) */
    MI355_EPI_F32        = 2  /* float(acc)*scale (+ f32 bias) + float(offsets)*scale, activation clamp (float).
                               * With an MI355_F16 destination the same float result is rounded to half, nearest even
                               * (the F16 leg of the dequantising GEMMLowp: src/cpu/operators/
                               * CpuGemmLowpMatrixMultiplyCore.cpp:305-309,374-375 and
                               * src/cpu/kernels/gemmlowp/generic/neon/fp16.cpp:32-70; with MI355_GEMM_ACCUMULATE the
                               * previous half values are widened, added in float, and the sum rounded once). */
} mi355_epilogue;

/* Which kernel family runs the product. The reference chooses among its kernels the same way: a method table that the
 * caller may narrow with arm_gemm::GemmConfig (method / filter, src/cpu/kernels/assembly/arm_gemm/arm_gemm.hpp:94-130;
 * table in src/core/NEON/kernels/arm_gemm/gemm_qint8.cpp:75-250), with CpuGemmLowpMatrixMultiplyKernel as the plain
 * fallback (src/cpu/operators/CpuGemmLowpMatrixMultiplyCore.cpp:216-263). */
typedef enum mi355_path
{
    MI355_PATH_AUTO   = 0, /* pipelined matrix-core kernel, or the streaming kernel for small M (<= 32; <= 64 with
                            * N < 8192 or with K <= 4096 a multiple of 64) */
    MI355_PATH_SIMPLE = 1, /* one thread per output, no matrix cores: the plain fallback (any alignment, any shape) */
    MI355_PATH_MFMA   = 2, /* a tiled matrix-core kernel whatever M is */
    MI355_PATH_SKINNY = 3, /* the streaming kernel (M <= 64) */
    MI355_PATH_TILE   = 16 /* MI355_PATH_TILE + n: the pipelined kernel with its n-th tile configuration (n counts the
                            * rows of its table, 256x128x128 first) wherever that configuration can take the shape */
} mi355_path;

typedef enum mi355_stage
{
    /* QUANTIZE_DOWN_FIXEDPOINT: rounding_shift(sqdmulh(v, multiplier), shift) + result_offset
     * (src/core/NEON/NEAsymm.h:87-148) */
    MI355_STAGE_FIXEDPOINT = 0,
    /* QUANTIZE_DOWN: ((v + result_offset) * multiplier) >> shift, wrap-around multiply, truncating shift, shift in
     * [0, 31] (src/cpu/kernels/CpuGemmLowpQuantizeDownInt32ScaleKernel.cpp:92-180; scalar form in
     * src/cpu/kernels/CpuGemmLowpOffsetContributionOutputStageKernel.cpp:348-362). The reference's vector lanes for a
     * signed destination additionally clamp negative results to 0 before narrowing
     * (CpuGemmLowpOffsetContributionOutputStageKernel.cpp:137-160) while its scalar tail and its test oracle do not:
     * this library follows the scalar form and the test oracle. */
    MI355_STAGE_SCALE = 1
} mi355_stage;

/* Mirrors the fields of GEMMLowpOutputStageInfo the integer output stages read
 * (arm_compute/function_info/GEMMInfo.h:49-82). With per_channel != 0 the per-column
 * multiplier / shift arrays are passed to mi355_gemmlowp_prepare instead. */
typedef struct mi355_requant
{
    int32_t per_channel;
    int32_t multiplier;
    int32_t shift; /* > 0: rounding right shift after the multiply; < 0: left shift before it */
    int32_t result_offset;
    int32_t min_bound;
    int32_t max_bound;
    int32_t stage; /* mi355_stage: which of the two integer output stages of GEMMLowpOutputStageType */
} mi355_requant;

/* mi355_gemm_desc::flags */
enum mi355_gemm_flags
{
    /* S32 / F32 destinations only: the result is added to what the destination holds (GEMMInfo::accumulate,
     * src/cpu/operators/CpuGemmLowpMatrixMultiplyCore.cpp:393-401; int32 adds wrap as they do in the GEMM's own
     * accumulators, the float add sits between the bias and the offset term, src/core/NEON/kernels/arm_gemm/
     * quantized.cpp:1007-1014). */
    MI355_GEMM_ACCUMULATE = 1,
    /* F32 destination: the activation clamp [act_min, act_max] is applied to float(acc)*scale (+bias) (+previous)
     * AND again after the offset term, as the reference does when the activation is one its assembly GEMM fuses
     * (quantized.cpp:1015 inside the merge, then the CpuActivation post-op,
     * src/cpu/operators/CpuGemmLowpMatrixMultiplyCore.cpp:326-332). Without the bit: once, at the end. */
    MI355_GEMM_ACT_TWICE = 2
};

typedef struct mi355_gemm_desc
{
    int32_t       M, N, K, batch;
    int32_t       a_dtype, b_dtype, dst_dtype; /* mi355_dtype */
    int32_t       epilogue;                    /* mi355_epilogue */
    int64_t       lda, ldb, ldd;
    int64_t       a_batch_stride, b_batch_stride, d_batch_stride;
    int32_t       a_offset, b_offset;
    mi355_requant requant;          /* MI355_EPI_FIXEDPOINT only */
    float         scale;            /* MI355_EPI_F32 only: a.scale * b.scale */
    float         act_min, act_max; /* MI355_EPI_F32 only: activation clamp, +-INFINITY for none */
    int32_t       path;             /* mi355_path */
    int32_t       b_transposed;     /* != 0: B is handed over as its transpose, N rows of K elements (ldb = row stride
                                       >= K, b_batch_stride between such matrices) - how fully connected weights arrive
                                       before CpuTransposeKernel (src/cpu/operators/CpuFullyConnected.cpp:283-292) */
    int32_t       b_k_interleave;   /* f > 1: the rows of B (its K index) are re-ordered while packing: row a*f + b
                                       (b < f) of the matrix that is multiplied is row b*(K/f) + a of the matrix handed
                                       over. Replaces CpuConvertFullyConnectedWeights
                                       (src/cpu/kernels/CpuConvertFullyConnectedWeightsKernel.cpp:60-66,118-121; f is its
                                       _factor2). 0 or 1: none. Must divide K. */
    int32_t       flags;            /* MI355_GEMM_* bits (enum mi355_gemm_flags) */
    /* Matrices whose M rows are the rows of several planes with a gap between the planes: GEMMInfo::
     * reinterpret_input_as_3d (A is [K, W, H, batch] read as W*H rows) and depth_output_gemm3d (D is [N, W, H, batch])
     * on tensors padded along y (src/cpu/operators/CpuGemmLowpMatrixMultiplyCore.cpp:520-534; strides per
     * arm_compute/core/ITensorInfo.h:81-334). Row r of a matrix is row r % plane_rows of plane r / plane_rows; planes
     * are a_plane_stride bytes (d_plane_stride destination elements) apart. plane_rows = 0: no planes (rows lda / ldd
     * apart throughout). plane_rows must divide M. Such a matrix is gathered into (scattered from) a dense device
     * buffer by one extra pass. */
    int32_t       a_plane_rows, d_plane_rows;
    int64_t       a_plane_stride, d_plane_stride;
} mi355_gemm_desc;

typedef struct mi355_gemm_handle mi355_gemm_handle;

/* Replaces CpuGemmLowpMatrixMultiplyCore::configure (src/cpu/operators/CpuGemmLowpMatrixMultiplyCore.cpp:116-360):
 * checks the descriptor, picks the kernel, sizes the device workspace. Allocates nothing on the device yet. */
int mi355_gemmlowp_create(const mi355_gemm_desc *desc, mi355_gemm_handle **out);

/* Replaces CpuGemmLowpMatrixMultiplyCore::prepare (:813-846) = pretranspose_B_array + column sums of B
 * (src/cpu/operators/internal/CpuGemmAssemblyDispatch.cpp:594-617, src/cpu/kernels/CpuGemmLowpMatrixReductionKernel.cpp:273-446)
 * + set_quantized_bias (:963-968 of src/core/NEON/kernels/arm_gemm/quantized.cpp): re-lays B out for the
 * matrix cores, reduces its columns, and folds a_offset*colsum + a_offset*b_offset*K + bias into one per-column
 * int32 vector. bias (N int32) may be NULL; mult / shift (N int32 each) are read only when requant.per_channel.
 * Call again whenever B, bias or the per-channel vectors change (a non-constant B: before every run). */
int mi355_gemmlowp_prepare(mi355_gemm_handle *h, const void *B, const int32_t *bias, const int32_t *mult,
                           const int32_t *shift, void *stream);

/* Replaces CpuGemmLowpMatrixMultiplyCore::update_quantization_parameters (:852-876): new offsets, per-tensor
 * requantisation and dequantisation scale without re-packing B. */
int mi355_gemmlowp_update_quant(mi355_gemm_handle *h, int32_t a_offset, int32_t b_offset,
                                const mi355_requant *requant, float scale, void *stream);

/* New row and batch strides (same units as in mi355_gemm_desc) for the calls that follow: ldb / b_batch_stride are read
 * by the next mi355_gemmlowp_prepare, the others by the next mi355_gemmlowp_run; nothing already packed is touched.
 * The reference reads every stride from the tensors when it runs, not when it is configured
 * (src/cpu/operators/internal/CpuGemmAssemblyDispatch.cpp:658-672,696-697), and its fixtures add padding in between
 * (tests/validation/fixtures/CpuGEMMLowpFixture.h:117). A shared B cannot become a batched one or the reverse. */
int mi355_gemmlowp_set_strides(mi355_gemm_handle *h, int64_t lda, int64_t ldb, int64_t ldd, int64_t a_batch_stride,
                               int64_t b_batch_stride, int64_t d_batch_stride);
/* The same with the plane strides of mi355_gemm_desc (a_plane_stride in bytes, d_plane_stride in destination
 * elements; ignored for a matrix created without planes). mi355_gemmlowp_set_strides leaves planes without a gap. */
int mi355_gemmlowp_set_strides_3d(mi355_gemm_handle *h, int64_t lda, int64_t ldb, int64_t ldd, int64_t a_batch_stride,
                                  int64_t b_batch_stride, int64_t d_batch_stride, int64_t a_plane_stride,
                                  int64_t d_plane_stride);

/* Replaces CpuGemmLowpMatrixMultiplyCore::run (:647-811). bias_f32 (N floats, MI355_EPI_F32 only) may be NULL. */
int mi355_gemmlowp_run(mi355_gemm_handle *h, const void *A, const float *bias_f32, void *D, void *stream);

/* mi355_gemmlowp_run for callers that cannot allocate device memory while they run (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc). It has no counterpart in the reference. Same arguments and
 * result as mi355_gemmlowp_run, with these differences: A, D and bias_f32 must be device memory; the run's workspace -
 * the row sums of A (4 bytes per row and batch entry, rounded up to 256; needed when b_offset != 0 or B is unsigned)
 * followed by the padded copy of A (batch * M * round_up(K, 128) bytes; needed when a row of A does not start on a
 * 4-byte boundary) - lives in one fixed array of mi355_gemmlowp_noalloc_workspace_bytes() (8 MiB) that each GPU holds
 * for the life of the process; a run that needs more is refused with an error, as is an F16 destination. The call
 * allocates and frees nothing and only enqueues kernels (and one event) on `stream`. Every call on a GPU uses that
 * GPU's one array (nothing in it has to start at zero: the kernels overwrite what they read), so calls that overlap in
 * time on one GPU - different streams, different handles - would race: calls on one stream are ordered by the stream;
 * a call that needs the workspace while the kernels of a call on ANOTHER stream are still pending is refused with an
 * error (synchronise, or keep to one stream). Under HIP graph capture nothing is recorded or checked: the order of the
 * graphs that share the array is the caller's business. The array's address and the event are set up by the first call
 * on each GPU. The handle must be prepared. */
int    mi355_gemmlowp_run_noalloc(mi355_gemm_handle *h, const void *A, const float *bias_f32, void *D, void *stream);
size_t mi355_gemmlowp_noalloc_workspace_bytes(void);

void mi355_gemmlowp_destroy(mi355_gemm_handle *h);

/* Name of the kernel variant the handle dispatches to, e.g. "mfma_256x128x64" (static string). */
const char *mi355_gemmlowp_kernel_name(const mi355_gemm_handle *h);

/* Stand-alone output stage on an int32 matrix. Replaces CpuGemmLowpOutputStage::run ->
 * CpuGemmLowpQuantizeDownInt32To{Int8,Uint8}ScaleByFixedPointKernel
 * (src/cpu/operators/CpuGemmLowpOutputStage.cpp:163-167,
 *  src/cpu/kernels/CpuGemmLowpQuantizeDownInt32ToInt8ScaleByFixedPointKernel.cpp:79-181). Stateless.
 * With dst_dtype MI355_S16 it replaces CpuGemmLowpQuantizeDownInt32ToInt16ScaleByFixedPointKernel
 * (src/cpu/kernels/CpuGemmLowpQuantizeDownInt32ToInt16ScaleByFixedPointKernel.cpp:76-200, arithmetic in
 *  src/core/NEON/NESymm.h:54-85): the multiply is the ROUNDING doubling high multiply there, there is no result offset
 *  (it must be 0), ld_dst counts int16 elements, and the bounds are either the whole int16 range or inside it. */
typedef struct mi355_output_stage_desc
{
    int32_t       M, N;
    int64_t       ld_src, ld_dst;
    int32_t       dst_dtype; /* MI355_U8, MI355_S8, or MI355_S16 (FIXEDPOINT only) */
    mi355_requant requant;   /* per-tensor */
} mi355_output_stage_desc;

int mi355_output_stage_run(const mi355_output_stage_desc *desc, const int32_t *src, const int32_t *bias, void *dst,
                           void *stream);

typedef enum mi355_conv_layout
{
    MI355_NHWC = 0, /* src [batch][H][W][C], weights [OFM][KH][KW][C], dst [batch][OH][OW][OFM] */
    /* src [batch][C][H][W], weights [OFM][C][KH][KW], dst [batch][OFM][OH][OW]: the reference's other layout
     * (im2col over channel planes + CpuCol2ImKernel, src/cpu/operators/CpuGemmConv2d.cpp:556-621; same integers).
     * Converted to and from NHWC on the device around the same kernels: one extra pass over src and dst. */
    MI355_NCHW = 1
} mi355_conv_layout;

typedef enum mi355_conv_path
{
    MI355_CONV_AUTO     = 0, /* implicit GEMM where the shape allows; channel counts that are not a multiple of 16 are
                              * padded to one (one pass over the source) so that the 16-byte loaders apply */
    MI355_CONV_EXPLICIT = 1, /* CpuIm2ColKernel's way: the patch matrix is written out, then a dense GEMM */
    MI355_CONV_IN_PLACE = 2  /* implicit GEMM on the caller's channel count: no padded copy of the source; channel counts
                              * that are not a multiple of 16 take the loader that gathers single bytes */
} mi355_conv_path;

/* Quantized NHWC convolution lowered to GEMM. Replaces CpuGemmConv2d::{configure,prepare,run}
 * (src/cpu/operators/CpuGemmConv2d.cpp:461-651, :1011-1101, :923-1008): CpuIm2ColKernel + CpuWeightsReshapeKernel
 * + CpuGemmLowpMatrixMultiplyCore. src is [batch][H][W][C], weights [OFM][KH][KW][C], dst [batch][OH][OW][OFM].
 * src_offset / weights_offset are the ADDED offsets (the negated zero points, as configure_mm passes them,
 * :266-280); pad_value is the byte im2col writes for out-of-image taps (the src zero point,
 * src/cpu/kernels/directconv2d/impl.h:333-334). */
typedef struct mi355_conv_desc
{
    int32_t       batch, H, W, C, OFM, KH, KW;
    int32_t       stride_x, stride_y, pad_left, pad_top, pad_right, pad_bottom, dilation_x, dilation_y;
    int32_t       src_dtype, weights_dtype, dst_dtype; /* mi355_dtype (8-bit) */
    int32_t       src_offset, weights_offset;
    int32_t       pad_value;
    mi355_requant requant;
    int32_t       path; /* mi355_conv_path */
    int32_t       layout; /* mi355_conv_layout of src, weights and dst */
    /* Bytes from one pixel (one tap of the weights) to the next when the tensors carry padding along the channel
     * dimension, as the reference's own fixtures give them (add_padding_x, tests/validation/Helpers.cpp:335-357;
     * ITensorInfo::strides_in_bytes()[1]). 0 = dense (C, C, OFM x element size). For MI355_NCHW tensors the same field
     * is the stride of dimension 1 there: bytes from one row of W (KW, OW) elements to the next. The strides of
     * dimensions 2 and 3 are the *_stride2 / *_stride3 fields at the end of this struct. The pointers passed to
     * prepare / run address the first element. Padded tensors are gathered into dense device buffers first (one
     * extra pass) and the result is scattered into dst, leaving its padding untouched. */
    int64_t       src_pixel_stride, weights_pixel_stride, dst_pixel_stride;
    /* dst_dtype MI355_F32 only - the dequantising convolution (CpuGemmConv2d with a QASYMM8_SIGNED input and an F32
     * destination, src/cpu/operators/CpuGemmConv2d.cpp:297-305,391-393): no requantisation, dst = float(acc) * scale
     * (+ float bias) + float(offset terms) * scale, clamped to [act_min, act_max] as MI355_EPI_F32 does; flags takes
     * MI355_GEMM_ACT_TWICE. The bias passed to mi355_conv_prepare is then OFM floats. */
    float         scale, act_min, act_max;
    int32_t       flags;
    /* ITensorInfo::strides_in_bytes()[2] and [3] of the three tensors (arm_compute/core/ITensorInfo.h:81-334): NHWC -
     * from one row of pixels to the next and from one image (one output channel's filter) to the next; NCHW - from one
     * channel plane to the next and from one image (filter) to the next. 0 = follows without a gap from the stride of
     * the dimension below (tensors padded along y, between planes or between images have larger values). */
    int64_t       src_stride2, src_stride3, weights_stride2, weights_stride3, dst_stride2, dst_stride3;
} mi355_conv_desc;

typedef struct mi355_conv_handle mi355_conv_handle;

int  mi355_conv_create(const mi355_conv_desc *desc, mi355_conv_handle **out);
/* bias: OFM int32 (8-bit destinations) or OFM floats (F32 destination), or NULL */
int  mi355_conv_prepare(mi355_conv_handle *h, const void *weights, const void *bias, const int32_t *mult,
                        const int32_t *shift, void *stream);
/* Replaces CpuGemmConv2d::update_quantization_parameters (:858-908): new offsets, pad value and requantisation without
 * touching the packed weights. mult / shift (OFM int32 each) are read only when requant->per_channel. */
int  mi355_conv_update_quant(mi355_conv_handle *h, int32_t src_offset, int32_t weights_offset, int32_t pad_value,
                             const mi355_requant *requant, const int32_t *mult, const int32_t *shift, void *stream);
/* New pixel strides (see mi355_conv_desc) for the calls that follow: weights_pixel_stride is read by the next
 * mi355_conv_prepare, the other two by the next mi355_conv_run. The reference reads strides when it runs and its
 * fixtures pad the tensors after configure (tests/validation/fixtures/CpuGemmConv2dFixture.h:315-319). */
int  mi355_conv_set_strides(mi355_conv_handle *h, int64_t src_pixel_stride, int64_t weights_pixel_stride,
                            int64_t dst_pixel_stride);
/* The same for all three strides of each tensor: { strides_in_bytes()[1], [2], [3] } of src, weights and dst, 0 = dense.
 * mi355_conv_set_strides(h, a, b, c) is this call with { a, 0, 0 }, { b, 0, 0 }, { c, 0, 0 }. Both layouts. */
int  mi355_conv_set_strides_nd(mi355_conv_handle *h, const int64_t src[3], const int64_t weights[3], const int64_t dst[3]);
int  mi355_conv_run(mi355_conv_handle *h, const void *src, void *dst, void *stream);
void mi355_conv_out_dims(const mi355_conv_desc *desc, int32_t *OH, int32_t *OW);
void mi355_conv_destroy(mi355_conv_handle *h);
const char *mi355_conv_kernel_name(const mi355_conv_handle *h);

/* The im2col kernel on its own. Replaces CpuIm2ColKernel::run_op for NHWC
 * (src/cpu/kernels/CpuIm2ColKernel.cpp:408-420 -> src/cpu/kernels/directconv2d/impl.h:307-389).
 * dst is [batch*OH*OW][KH*KW*C], K ordered (ky, kx, c). */
int mi355_im2col_nhwc_run(const mi355_conv_desc *desc, const void *src, void *dst, void *stream);

/* Thread-local text of the last error on this thread ("" if none). */
const char *mi355_last_error(void);

/* Library / device identification: fills name with the HIP device's gcnArchName; returns its CU count or -1. */
int mi355_device_info(char *name, size_t name_len);

#ifdef __cplusplus
}
#endif
#endif /* MI355_GEMMLOWP_H */
