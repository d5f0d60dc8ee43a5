/*
 * TEST INFRASTRUCTURE ONLY — C-callable doorway into the reference's own portable test oracle.
 *
 * This translation unit contains no arithmetic of its own: it copies caller buffers into the
 * reference's SimpleTensor objects, calls the reference functions named in each comment, and
 * copies the result back. It is compiled together with the reference's sources where they lie
 * under /root/reference (see oracle/Makefile); the product is oracle/_ref/libaclref.so, which is
 * git-ignored. Used to pin oracle/gemmlowp_oracle.c and to write the fixtures in tests/golden/.
 */
#include "arm_compute/core/utils/quantization/AsymmHelpers.h"
#include "tests/SimpleTensor.h"
#include "tests/validation/reference/ArithmeticOperations.h"
#include "tests/validation/reference/Convolution3d.h"
#include "tests/validation/reference/DequantizationLayer.h"
#include "tests/validation/reference/GEMMLowp.h"
#include "tests/validation/reference/Im2Col.h"
#include "tests/validation/reference/UtilsQuantizedAsymm.h"

#include <cstdint>
#include <cstring>
#include <vector>

using namespace arm_compute;
using namespace arm_compute::test;
using namespace arm_compute::test::validation;

namespace
{
template <typename T>
SimpleTensor<T> make(const TensorShape &shape, DataType dt, const void *data, QuantizationInfo q = QuantizationInfo(),
                     DataLayout layout = DataLayout::NCHW)
{
    SimpleTensor<T> t(shape, dt, 1, q, layout);
    if (data != nullptr)
        std::memcpy(t.data(), data, sizeof(T) * t.num_elements());
    return t;
}
} // namespace

#pragma GCC visibility push(default)
extern "C"
{
    /* tests/validation/reference/UtilsQuantizedAsymm.h:51-88 */
    int32_t ref_asymm_int_mult(int32_t a, int32_t b) { return asymm_int_mult(a, b); }
    int32_t ref_asymm_rounding_divide_by_pow2(int32_t x, int e) { return asymm_rounding_divide_by_pow2(x, e); }
    int32_t ref_quantize_down_scalar(int32_t v, int32_t mult, int32_t shift, int32_t off, int32_t lo, int32_t hi)
    {
        return quantize_down_scale_by_fixedpoint(v, mult, shift, off, lo, hi);
    }

    /* src/core/utils/quantization/AsymmHelpers.cpp:43-55 */
    int ref_calculate_quantized_multiplier(float m, int32_t *qm, int32_t *shift)
    {
        const Status s = quantization::calculate_quantized_multiplier(m, qm, shift);
        return bool(s) ? 0 : 1;
    }

    /* tests/validation/reference/GEMMLowp.cpp:203-255 ; batch > 1 with b_batched = 0 shares one B */
    void ref_gemmlowp_core(const void *a, const void *b, int is_signed, int M, int N, int K, int batch, int b_batched,
                           int32_t a_offset, int32_t b_offset, int32_t *out)
    {
        const TensorShape sa(K, M, batch), sc(N, M, batch);
        const TensorShape sb = b_batched ? TensorShape(N, K, batch) : TensorShape(N, K);
        SimpleTensor<int32_t> c;
        if (is_signed)
            c = reference::gemmlowp_matrix_multiply_core<int32_t, int8_t, int8_t>(
                make<int8_t>(sa, DataType::QASYMM8_SIGNED, a), make<int8_t>(sb, DataType::QASYMM8_SIGNED, b), sc,
                a_offset, b_offset);
        else
            c = reference::gemmlowp_matrix_multiply_core<int32_t, uint8_t, uint8_t>(
                make<uint8_t>(sa, DataType::QASYMM8, a), make<uint8_t>(sb, DataType::QASYMM8, b), sc, a_offset,
                b_offset);
        std::memcpy(out, c.data(), sizeof(int32_t) * c.num_elements());
    }

    /* uint8 A x int8 B, zero offsets: the only mixed-sign instantiation the reference exports
     * (tests/validation/reference/GEMMLowp.cpp:487-489) */
    void ref_gemmlowp_u8s8(const void *a, const void *b, int M, int N, int K, int32_t *out)
    {
        const SimpleTensor<int32_t> c = reference::gemmlowp<int32_t, uint8_t, int8_t>(
            make<uint8_t>(TensorShape(K, M), DataType::QASYMM8, a),
            make<int8_t>(TensorShape(N, K), DataType::QASYMM8_SIGNED, b), TensorShape(N, M));
        std::memcpy(out, c.data(), sizeof(int32_t) * c.num_elements());
    }

    /* tests/validation/reference/GEMMLowp.cpp:110-157 (with and without bias) */
    void ref_quantize_down_fixedpoint(const int32_t *in, const int32_t *bias, int M, int N, const int32_t *mult,
                                      const int32_t *shift, int n_qparams, int32_t result_offset, int32_t lo,
                                      int32_t hi, int dst_signed, void *out)
    {
        const SimpleTensor<int32_t> t = make<int32_t>(TensorShape(N, M), DataType::S32, in);
        const std::vector<int32_t>  m(mult, mult + n_qparams), s(shift, shift + n_qparams);
        if (dst_signed)
        {
            const SimpleTensor<int8_t> d =
                bias ? reference::gemmlowp_quantize_down_scale_by_fixedpoint<int32_t, int8_t>(
                           t, make<int32_t>(TensorShape(N), DataType::S32, bias), m, s, result_offset, lo, hi)
                     : reference::gemmlowp_quantize_down_scale_by_fixedpoint<int32_t, int8_t>(t, m, s, result_offset,
                                                                                              lo, hi);
            std::memcpy(out, d.data(), d.num_elements());
        }
        else
        {
            const SimpleTensor<uint8_t> d =
                bias ? reference::gemmlowp_quantize_down_scale_by_fixedpoint<int32_t, uint8_t>(
                           t, make<int32_t>(TensorShape(N), DataType::S32, bias), m, s, result_offset, lo, hi)
                     : reference::gemmlowp_quantize_down_scale_by_fixedpoint<int32_t, uint8_t>(t, m, s, result_offset,
                                                                                               lo, hi);
            std::memcpy(out, d.data(), d.num_elements());
        }
    }

    /* the same template with a 16-bit destination (tests/validation/reference/GEMMLowp.cpp:110-157,423-437); note that it
     * multiplies with the non-rounding SQDMULH model whereas the NEON int16 kernel uses the rounding one */
    void ref_quantize_down_fixedpoint_s16(const int32_t *in, const int32_t *bias, int M, int N, int32_t mult, int32_t shift,
                                          int32_t lo, int32_t hi, int16_t *out)
    {
        const SimpleTensor<int32_t> t = make<int32_t>(TensorShape(N, M), DataType::S32, in);
        const std::vector<int32_t>  m(1, mult), s(1, shift);
        const SimpleTensor<int16_t> d =
            bias ? reference::gemmlowp_quantize_down_scale_by_fixedpoint<int32_t, int16_t>(
                       t, make<int32_t>(TensorShape(N), DataType::S32, bias), m, s, 0, lo, hi)
                 : reference::gemmlowp_quantize_down_scale_by_fixedpoint<int32_t, int16_t>(t, m, s, 0, lo, hi);
        std::memcpy(out, d.data(), sizeof(int16_t) * d.num_elements());
    }

    /* tests/validation/reference/GEMMLowp.cpp:66-104,278-307: QUANTIZE_DOWN with an integer multiplier */
    void ref_quantize_down_scale(const int32_t *in, const int32_t *bias, int M, int N, const int32_t *mult,
                                 const int32_t *shift, int n_qparams, int32_t result_offset, int32_t lo, int32_t hi,
                                 int dst_signed, void *out)
    {
        const SimpleTensor<int32_t> t = make<int32_t>(TensorShape(N, M), DataType::S32, in);
        const std::vector<int32_t>  m(mult, mult + n_qparams), s(shift, shift + n_qparams);
        if (dst_signed)
        {
            const SimpleTensor<int8_t> d =
                bias ? reference::gemmlowp_quantize_down_scale<int32_t, int8_t>(
                           t, make<int32_t>(TensorShape(N), DataType::S32, bias), result_offset, m, s, lo, hi)
                     : reference::gemmlowp_quantize_down_scale<int32_t, int8_t>(t, result_offset, m, s, lo, hi);
            std::memcpy(out, d.data(), d.num_elements());
        }
        else
        {
            const SimpleTensor<uint8_t> d =
                bias ? reference::gemmlowp_quantize_down_scale<int32_t, uint8_t>(
                           t, make<int32_t>(TensorShape(N), DataType::S32, bias), result_offset, m, s, lo, hi)
                     : reference::gemmlowp_quantize_down_scale<int32_t, uint8_t>(t, result_offset, m, s, lo, hi);
            std::memcpy(out, d.data(), d.num_elements());
        }
    }

    /* tests/validation/reference/DequantizationLayer.cpp:69-116 on an S32 tensor, as
     * tests/validation/fixtures/GEMMLowpFixture.h:868-910 uses it for the F32 GEMMLowp reference */
    void ref_dequantize_s32(const int32_t *in, int count, float scale, float *out)
    {
        const SimpleTensor<int32_t> t =
            make<int32_t>(TensorShape(count), DataType::S32, in, QuantizationInfo(scale, 0));
        const SimpleTensor<float> d = reference::dequantization_layer<float, int32_t>(t);
        std::memcpy(out, d.data(), sizeof(float) * d.num_elements());
    }

    /* tests/validation/reference/DequantizationLayer.cpp:69-116 with a half destination, and - when prev is given -
     * tests/validation/reference/ArithmeticOperations.cpp (ADD, SATURATE) on halfs: the F16 GEMMLowp reference of
     * tests/validation/fixtures/GEMMLowpFixture.h:908-920. Halfs travel as their 16 bits. */
    void ref_dequantize_s32_f16(const int32_t *in, int count, float scale, const uint16_t *prev, uint16_t *out)
    {
        const SimpleTensor<int32_t> t =
            make<int32_t>(TensorShape(count), DataType::S32, in, QuantizationInfo(scale, 0));
        SimpleTensor<half> d = reference::dequantization_layer<half, int32_t>(t);
        if (prev != nullptr)
        {
            SimpleTensor<half> o = make<half>(TensorShape(count), DataType::F16, prev);
            reference::arithmetic_operation<half>(reference::ArithmeticOperation::ADD, o, d, o, ConvertPolicy::SATURATE);
            std::memcpy(out, o.data(), sizeof(half) * o.num_elements());
            return;
        }
        std::memcpy(out, d.data(), sizeof(half) * d.num_elements());
    }

    /* tests/validation/reference/Im2Col.cpp:108-170 (NHWC branch; instantiated for uint8 storage only,
     * which is enough: im2col moves bytes and pads with the low byte of the zero point) */
    void ref_im2col_nhwc(const uint8_t *src, uint8_t *dst, int batch, int H, int W, int C, int KH, int KW, int sx,
                         int sy, int pl, int pt, int pr, int pb, int OH, int OW, int zero_point)
    {
        const QuantizationInfo q(1.f, zero_point);
        const SimpleTensor<uint8_t> s =
            make<uint8_t>(TensorShape(C, W, H, batch), DataType::QASYMM8, src, q, DataLayout::NHWC);
        SimpleTensor<uint8_t> d = make<uint8_t>(TensorShape(KH * KW * C, OH * OW, 1, batch), DataType::QASYMM8,
                                                nullptr, q, DataLayout::NHWC);
        reference::im2col<uint8_t>(s, d, Size2D(KW, KH), PadStrideInfo(sx, sy, pl, pr, pt, pb, DimensionRoundingType::FLOOR),
                                   false, 1, 0);
        std::memcpy(dst, d.data(), d.num_elements());
    }

    /* One output element per call of tests/validation/reference/Convolution3d.h:120-245, walked over the output the
     * way tests/validation/reference/ConvolutionLayer.cpp:44-113 does (that file itself needs the test framework).
     * All tensors NCHW as the reference's convolution reference requires. w_scales has n_scales entries (1 = per
     * tensor). Output dtype = input dtype. */
    void ref_conv_nchw_quantized(const void *src, const void *weights, const int32_t *bias, void *dst, int is_signed,
                                 int per_channel, int batch, int C, int H, int W, int OFM, int KH, int KW, int OH,
                                 int OW, int sx, int sy, int pl, int pt, int dx, int dy, float in_scale,
                                 int32_t in_zp, const float *w_scales, int n_scales, int32_t w_zp, float out_scale,
                                 int32_t out_zp)
    {
        const QuantizationInfo   iq(in_scale, in_zp), oq(out_scale, out_zp);
        const std::vector<float> ws(w_scales, w_scales + n_scales);
        const QuantizationInfo   wq = per_channel ? QuantizationInfo(ws) : QuantizationInfo(ws[0], w_zp);
        const TensorShape        s_in(W, H, C, batch), s_w(KW, KH, C, OFM), s_out(OW, OH, OFM, batch);
        const SimpleTensor<int32_t> b = make<int32_t>(TensorShape(OFM), DataType::S32, bias);
        const int start_xi = (dx * (KW - 1) + 1) / 2 - pl;
        const int start_yi = (dy * (KH - 1) + 1) / 2 - pt;
        auto run = [&](auto tag_in, auto tag_w, DataType dt_in, DataType dt_w)
        {
            using TI                 = decltype(tag_in);
            using TW                 = decltype(tag_w);
            const SimpleTensor<TI> s = make<TI>(s_in, dt_in, src, iq);
            const SimpleTensor<TW> w = make<TW>(s_w, dt_w, weights, wq);
            SimpleTensor<TI>       d = make<TI>(s_out, dt_in, nullptr, oq);
            for (int r = 0; r < batch; ++r)
                for (int yo = 0; yo < OH; ++yo)
                    for (int xo = 0; xo < OW; ++xo)
                        for (int ofm = 0; ofm < OFM; ++ofm)
                            convolution_3d::detail::convolution3d<TI, TW, int32_t, TI>(
                                s, w, b, d, r * W * H * C, ofm * KW * KH * C, ofm,
                                xo + yo * OW + ofm * OW * OH + r * OW * OH * OFM, start_xi + xo * sx,
                                start_yi + yo * sy, W, H, C, KW, KH, dx, dy, ofm);
            std::memcpy(dst, d.data(), d.num_elements());
        };
        if (is_signed)
            run(int8_t(0), int8_t(0), DataType::QASYMM8_SIGNED,
                per_channel ? DataType::QSYMM8_PER_CHANNEL : DataType::QASYMM8_SIGNED);
        else if (per_channel)
            run(uint8_t(0), int8_t(0), DataType::QASYMM8, DataType::QSYMM8_PER_CHANNEL);
        else
            run(uint8_t(0), uint8_t(0), DataType::QASYMM8, DataType::QASYMM8);
    }
}
#pragma GCC visibility pop
