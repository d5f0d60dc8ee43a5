// Tests of the arm_compute-compatible host layer, written the way the reference's validation suites are
// (tests/validation/NEON/GEMMLowp.cpp, ConvolutionLayer.cpp): build the function on real Tensors, fill them from a
// seed, run, and compare against the oracle (oracle/gemmlowp_oracle.h) with tolerance zero.
//   test_host_api --cpu   : validate() tables, TensorInfo layout, quantization helpers (no GPU needed)
//   test_host_api --gpu   : configure / prepare / run on the device, host buffers and imported device buffers
#include "arm_compute/core/utils/quantization/AsymmHelpers.h"
#include "arm_compute/runtime/NEON/NEFunctions.h"
#include "arm_compute/runtime/experimental/operators/CpuGEMMLowp.h"
#include "arm_compute/runtime/experimental/operators/CpuGemmConv2d.h"
#include "arm_compute/runtime/Tensor.h"
#include "gemmlowp_oracle.h"

#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <string>
#include <vector>

using namespace arm_compute;

static int g_failures = 0, g_checks = 0;
#define EXPECT(cond)                                                              \
    do                                                                            \
    {                                                                             \
        ++g_checks;                                                               \
        if (!(cond))                                                              \
        {                                                                         \
            ++g_failures;                                                         \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);         \
        }                                                                         \
    } while (0)
#define SECTION(name) std::printf("[case] %s\n", name), std::fflush(stdout)

// ---------------------------------------------------------------------------------------------------------------------
static void test_tensor_info()
{
    SECTION("TensorInfo strides, padding, shapes");
    TensorInfo info(TensorShape(21U, 13U), 1, DataType::QASYMM8);
    EXPECT(info.dimension(0) == 21 && info.dimension(1) == 13 && info.num_dimensions() == 2);
    EXPECT(info.strides_in_bytes()[0] == 1 && info.strides_in_bytes()[1] == 21 && info.total_size() == 21 * 13);
    EXPECT(info.offset_first_element_in_bytes() == 0);
    info.extend_padding(PaddingSize(0, 3, 0, 2)); // top, right, bottom, left
    EXPECT(info.strides_in_bytes()[1] == 26 && info.offset_first_element_in_bytes() == 2 && info.has_padding());
    TensorInfo s32(TensorShape(33U, 13U, 4U), 1, DataType::S32);
    EXPECT(s32.element_size() == 4 && s32.strides_in_bytes()[1] == 132 && s32.strides_in_bytes()[2] == 132 * 13);
    EXPECT(s32.total_size() == 132u * 13 * 4);
    EXPECT(TensorShape(5U, 1U, 1U).num_dimensions() == 1); // trailing ones are not counted
    EXPECT(TensorShape(5U, 3U, 2U).total_size_upper(1) == 6);
    EXPECT(info.clone()->set_is_resizable(false).is_resizable() == false);
    TensorInfo nhwc(TensorShape(64U, 56U, 48U, 2U), 1, DataType::QASYMM8_SIGNED, DataLayout::NHWC);
    EXPECT(nhwc.dimension(DataLayoutDimension::CHANNEL) == 64 && nhwc.dimension(DataLayoutDimension::WIDTH) == 56 &&
           nhwc.dimension(DataLayoutDimension::HEIGHT) == 48 && nhwc.dimension(DataLayoutDimension::BATCHES) == 2);
    QuantizationInfo q(0.5f, -3);
    EXPECT(q.uniform().scale == 0.5f && q.uniform().offset == -3 && !q.is_dynamic());
    QuantizationInfo pc(std::vector<float>{0.1f, 0.2f});
    EXPECT(pc.scale().size() == 2 && pc.offset().empty() && pc.uniform().offset == 0);
}

static void test_quant_helpers()
{
    SECTION("calculate_quantized_multiplier against the oracle");
    std::mt19937                          rng(7);
    std::uniform_real_distribution<float> u(std::log(1e-6f), std::log(8.f));
    for (int i = 0; i < 20000; ++i)
    {
        const float real = std::exp(u(rng));
        int32_t     m = 0, s = 0, om = 0, os = 0;
        const bool  ok  = bool(quantization::calculate_quantized_multiplier(real, &m, &s));
        const bool  ook = orc_calculate_quantized_multiplier(real, &om, &os) == 0;
        EXPECT(ok == ook);
        if (ok && ook)
            EXPECT(m == om && s == os);
    }
    int32_t m = 0, s = 0;
    EXPECT(bool(quantization::calculate_quantized_multiplier(0.0007f, &m, &s)) && m == 1539316224 && s == 10);
    EXPECT(bool(quantization::calculate_quantized_multiplier(1.0f, &m, &s)) && m == (1 << 30) && s == -1);
    EXPECT(!bool(quantization::calculate_quantized_multiplier(-0.5f, &m, &s)));

    SECTION("calculate_quantized_multipliers pads per-channel vectors by 32");
    GEMMLowpOutputStageInfo st;
    EXPECT(bool(quantization::calculate_quantized_multipliers(QuantizationInfo(0.02f, 1),
                                                              QuantizationInfo(std::vector<float>{0.1f, 0.5f, 0.9f}),
                                                              QuantizationInfo(0.5f, 3), st)));
    EXPECT(st.gemmlowp_multipliers.size() == 3 + 32 && st.gemmlowp_shifts.size() == 3 + 32);
    EXPECT(st.gemmlowp_multiplier == st.gemmlowp_multipliers[0] && st.gemmlowp_shift == st.gemmlowp_shifts[0]);

    SECTION("get_quantized_activation_min_max");
    const UniformQuantizationInfo oq(0.1f, 10);
    auto r = get_quantized_activation_min_max(ActivationLayerInfo(ActivationLayerInfo::ActivationFunction::RELU),
                                              DataType::QASYMM8, oq);
    EXPECT(r.first == 10 && r.second == 255);
    r = get_quantized_activation_min_max(ActivationLayerInfo(ActivationLayerInfo::ActivationFunction::BOUNDED_RELU, 6.f),
                                         DataType::QASYMM8, oq);
    EXPECT(r.first == 10 && r.second == 70);
    r = get_quantized_activation_min_max(
        ActivationLayerInfo(ActivationLayerInfo::ActivationFunction::LU_BOUNDED_RELU, 6.f, -1.f), DataType::QASYMM8_SIGNED, oq);
    EXPECT(r.first == 0 && r.second == 70);
    auto d = scaled_dimensions(56, 56, 3, 3, PadStrideInfo(1, 1, 1, 1));
    EXPECT(d.first == 56 && d.second == 56);
    d = scaled_dimensions(23, 27, 3, 3, PadStrideInfo(2, 1, 0, 0));
    EXPECT(d.first == 11 && d.second == 25);
}

// the reference's own validate tables: tests/validation/NEON/GEMMLowp.cpp:168-200 and :533-568
static void test_validate_tables()
{
    SECTION("NEGEMMLowpMatrixMultiplyCore::validate table (S32)");
    const QuantizationInfo qa(1.f / 255, 10), qb(1.f / 256, 10);
    struct Row
    {
        TensorInfo a, b, o;
        bool       expected;
    };
    const std::vector<Row> rows = {
        {TensorInfo(TensorShape(21U, 13U), 1, DataType::QASYMM8, qa), TensorInfo(TensorShape(33U, 21U), 1, DataType::QASYMM8, qb),
         TensorInfo(TensorShape(33U, 13U), 1, DataType::S32), true},
        {TensorInfo(TensorShape(21U, 13U), 1, DataType::S32), TensorInfo(TensorShape(33U, 21U), 1, DataType::QASYMM8, qb),
         TensorInfo(TensorShape(33U, 13U), 1, DataType::S32), false},
        {TensorInfo(TensorShape(20U, 13U), 1, DataType::QASYMM8, qa), TensorInfo(TensorShape(33U, 21U), 1, DataType::QASYMM8, qb),
         TensorInfo(TensorShape(33U, 13U), 1, DataType::S32), false},
        {TensorInfo(TensorShape(21U, 13U), 1, DataType::QASYMM8, qa), TensorInfo(TensorShape(33U, 21U), 1, DataType::QASYMM8, qb),
         TensorInfo(TensorShape(8U, 11U), 1, DataType::S32), false},
        {TensorInfo(TensorShape(16U, 32U), 1, DataType::QASYMM8, qa), TensorInfo(TensorShape(64U, 16U), 1, DataType::QASYMM8, qb),
         TensorInfo(TensorShape(64U, 32U), 1, DataType::S32), true},
        {TensorInfo(TensorShape(16U, 32U), 1, DataType::QASYMM8_SIGNED, qa), TensorInfo(TensorShape(64U, 16U), 1, DataType::QASYMM8, qb),
         TensorInfo(TensorShape(64U, 32U), 1, DataType::S32), false},
    };
    for (const Row &r : rows)
    {
        const Status st = NEGEMMLowpMatrixMultiplyCore::validate(&r.a.clone()->set_is_resizable(false),
                                                                 &r.b.clone()->set_is_resizable(false), nullptr,
                                                                 &r.o.clone()->set_is_resizable(false));
        EXPECT(bool(st) == r.expected);
    }
    SECTION("NEGEMMLowpMatrixMultiplyCore::validate table (F32 dequant)");
    const std::vector<Row> frows = {
        {TensorInfo(TensorShape(16U, 32U), 1, DataType::QASYMM8, qa), TensorInfo(TensorShape(64U, 16U), 1, DataType::QASYMM8_SIGNED, qb),
         TensorInfo(TensorShape(64U, 32U), 1, DataType::F32), true},
        {TensorInfo(TensorShape(16U, 32U), 1, DataType::QASYMM8_SIGNED, qa), TensorInfo(TensorShape(64U, 16U), 1, DataType::QASYMM8_SIGNED, qb),
         TensorInfo(TensorShape(64U, 32U), 1, DataType::F32), true},
        {TensorInfo(TensorShape(16U, 32U), 1, DataType::QASYMM8_SIGNED, qa), TensorInfo(TensorShape(64U, 16U), 1, DataType::QASYMM8, qb),
         TensorInfo(TensorShape(64U, 32U), 1, DataType::F32), false},
    };
    for (const Row &r : frows)
        EXPECT(bool(NEGEMMLowpMatrixMultiplyCore::validate(&r.a, &r.b, nullptr, &r.o)) == r.expected);

    SECTION("validate: bias, reshape flags, accumulate, output stage rules");
    const TensorInfo a(TensorShape(16U, 32U), 1, DataType::QASYMM8, qa), b(TensorShape(64U, 16U), 1, DataType::QASYMM8, qb);
    const TensorInfo o32(TensorShape(64U, 32U), 1, DataType::S32), o8(TensorShape(64U, 32U), 1, DataType::QASYMM8, qa);
    const TensorInfo bias(TensorShape(64U), 1, DataType::S32), bias_bad(TensorShape(63U), 1, DataType::S32);
    // bias with S32 output and no output stage: CpuGemmLowpMatrixMultiplyCore.cpp:376-378
    EXPECT(!bool(NEGEMMLowpMatrixMultiplyCore::validate(&a, &b, &bias, &o32)));
    EXPECT(!bool(NEGEMMLowpMatrixMultiplyCore::validate(&a, &b, nullptr, &o32, GEMMInfo(true, false, true))));
    EXPECT(!bool(NEGEMMLowpMatrixMultiplyCore::validate(&a, &b, nullptr, &o32, GEMMInfo(false, true, true))));
    GEMMInfo pre;
    pre.set_pretranspose_B(true);
    EXPECT(!bool(NEGEMMLowpMatrixMultiplyCore::validate(&a, &b, nullptr, &o32, pre)));
    EXPECT(!bool(NEGEMMLowpMatrixMultiplyCore::validate(&a, &b, nullptr, &o8))); // quantized output without a stage
    GEMMLowpOutputStageInfo st;
    st.type = GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT;
    st.gemmlowp_multiplier = 1518500250, st.gemmlowp_shift = 8, st.gemmlowp_offset = 10;
    st.gemmlowp_min_bound = 0, st.gemmlowp_max_bound = 255, st.output_data_type = DataType::QASYMM8;
    GEMMInfo fused(false, false, true, 0, false, false, st);
    EXPECT(bool(NEGEMMLowpMatrixMultiplyCore::validate(&a, &b, &bias, &o8, fused)));
    EXPECT(!bool(NEGEMMLowpMatrixMultiplyCore::validate(&a, &b, &bias_bad, &o8, fused)));
    EXPECT(!bool(NEGEMMLowpMatrixMultiplyCore::validate(&a, &b, &bias, &o32, fused)));
    st.gemmlowp_min_bound = 5, st.gemmlowp_max_bound = 4;
    EXPECT(!bool(NEGEMMLowpMatrixMultiplyCore::validate(&a, &b, &bias, &o8, GEMMInfo(false, false, true, 0, false, false, st))));
    // bounds with one end inside the output type's range and one outside are refused (the reference's kernels disagree
    // on them); bounds that cover the range only saturate and are accepted
    st.gemmlowp_min_bound = -5, st.gemmlowp_max_bound = 200;
    EXPECT(!bool(NEGEMMLowpMatrixMultiplyCore::validate(&a, &b, &bias, &o8, GEMMInfo(false, false, true, 0, false, false, st))));
    st.gemmlowp_min_bound = 10, st.gemmlowp_max_bound = 300;
    EXPECT(!bool(NEGEMMLowpMatrixMultiplyCore::validate(&a, &b, &bias, &o8, GEMMInfo(false, false, true, 0, false, false, st))));
    st.gemmlowp_min_bound = std::numeric_limits<int32_t>::lowest(), st.gemmlowp_max_bound = std::numeric_limits<int32_t>::max();
    EXPECT(bool(NEGEMMLowpMatrixMultiplyCore::validate(&a, &b, &bias, &o8, GEMMInfo(false, false, true, 0, false, false, st))));
    st.gemmlowp_min_bound = 5, st.gemmlowp_max_bound = 4;
    GEMMInfo acc;
    acc.set_accumulate(true);
    EXPECT(!bool(NEGEMMLowpMatrixMultiplyCore::validate(&a, &b, nullptr, &o8, acc)));
    // the reference's accumulation validate test (tests/validation/NEON/GEMMLowp.cpp:135-163): S32 yes, quantized no
    EXPECT(bool(NEGEMMLowpMatrixMultiplyCore::validate(&a, &b, nullptr, &o32, acc)));
    GEMMInfo acc_fused(false, false, true, 0, false, false, st);
    acc_fused.set_accumulate(true);
    st.gemmlowp_min_bound = 0, st.gemmlowp_max_bound = 255;
    acc_fused.set_gemmlowp_output_stage(st);
    EXPECT(!bool(NEGEMMLowpMatrixMultiplyCore::validate(&a, &b, nullptr, &o8, acc_fused)));
    EXPECT(!bool(NEGEMMLowpMatrixMultiplyCore::validate(nullptr, &b, nullptr, &o32)));

    SECTION("NEGEMMLowpOutputStage::validate");
    GEMMLowpOutputStageInfo os;
    os.type = GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT;
    os.gemmlowp_multiplier = 1 << 30, os.gemmlowp_shift = 3, os.gemmlowp_min_bound = 0, os.gemmlowp_max_bound = 255;
    os.output_data_type = DataType::QASYMM8;
    EXPECT(bool(NEGEMMLowpOutputStage::validate(&o32, &bias, &o8, os)));
    EXPECT(!bool(NEGEMMLowpOutputStage::validate(&o8, &bias, &o8, os)));       // src must be S32
    EXPECT(!bool(NEGEMMLowpOutputStage::validate(&o32, &bias_bad, &o8, os)));  // bias length
    EXPECT(!bool(NEGEMMLowpOutputStage::validate(&o32, &bias, &o32, os)));     // dst type
    os.type = GEMMLowpOutputStageType::NONE;
    EXPECT(!bool(NEGEMMLowpOutputStage::validate(&o32, &bias, &o8, os)));
    os.type = GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT;
    os.gemmlowp_min_bound = 9, os.gemmlowp_max_bound = 1;
    EXPECT(!bool(NEGEMMLowpOutputStage::validate(&o32, &bias, &o8, os)));
    os.gemmlowp_min_bound = -1, os.gemmlowp_max_bound = 254; // partly outside [0, 255]
    EXPECT(!bool(NEGEMMLowpOutputStage::validate(&o32, &bias, &o8, os)));
    os.gemmlowp_min_bound = -1000, os.gemmlowp_max_bound = 1000; // covers it: saturation only
    EXPECT(bool(NEGEMMLowpOutputStage::validate(&o32, &bias, &o8, os)));

    SECTION("NEGEMMConvolutionLayer::validate");
    TensorInfo src(TensorShape(64U, 8U, 8U, 2U), 1, DataType::QASYMM8_SIGNED, QuantizationInfo(0.02f, -1));
    TensorInfo w(TensorShape(64U, 3U, 3U, 32U), 1, DataType::QSYMM8_PER_CHANNEL, QuantizationInfo(std::vector<float>(32, 0.01f)));
    TensorInfo cb(TensorShape(32U), 1, DataType::S32);
    TensorInfo dst(TensorShape(32U, 8U, 8U, 2U), 1, DataType::QASYMM8_SIGNED, QuantizationInfo(0.5f, -5));
    for (TensorInfo *t : {&src, &w, &dst})
        t->set_data_layout(DataLayout::NHWC);
    const PadStrideInfo ps(1, 1, 1, 1);
    EXPECT(bool(NEGEMMConvolutionLayer::validate(&src, &w, &cb, &dst, ps)));
    EXPECT(!bool(NEGEMMConvolutionLayer::validate(&src, &w, &cb, &dst, ps, WeightsInfo(true, 3, 3, 32))));
    EXPECT(!bool(NEGEMMConvolutionLayer::validate(&src, &w, &cb, &dst, ps, WeightsInfo(), Size2D(1, 1), ActivationLayerInfo(), false, 2)));
    TensorInfo w_badc(TensorShape(32U, 3U, 3U, 32U), 1, DataType::QSYMM8_PER_CHANNEL, QuantizationInfo(std::vector<float>(32, 0.01f)));
    w_badc.set_data_layout(DataLayout::NHWC);
    EXPECT(!bool(NEGEMMConvolutionLayer::validate(&src, &w_badc, &cb, &dst, ps)));
    TensorInfo cb_bad(TensorShape(31U), 1, DataType::S32);
    EXPECT(!bool(NEGEMMConvolutionLayer::validate(&src, &w, &cb_bad, &dst, ps)));
    TensorInfo dst_bad(TensorShape(32U, 7U, 8U, 2U), 1, DataType::QASYMM8_SIGNED, QuantizationInfo(0.5f, -5));
    dst_bad.set_data_layout(DataLayout::NHWC);
    EXPECT(!bool(NEGEMMConvolutionLayer::validate(&src, &w, &cb, &dst_bad, ps)));
}

// accept / reject rules of CpuFullyConnected::validate (src/cpu/operators/CpuFullyConnected.cpp:384-489 of the reference)
static void test_fully_connected_validate()
{
    SECTION("NEFullyConnectedLayer::validate accept / reject");
    const QuantizationInfo q(0.1f, 3);
    TensorInfo src(TensorShape(200U, 4U), 1, DataType::QASYMM8, q), w(TensorShape(200U, 30U), 1, DataType::QASYMM8, q);
    TensorInfo b(TensorShape(30U), 1, DataType::S32), dst(TensorShape(30U, 4U), 1, DataType::QASYMM8, q);
    EXPECT(bool(NEFullyConnectedLayer::validate(&src, &w, &b, &dst)));
    EXPECT(bool(NEFullyConnectedLayer::validate(&src, &w, nullptr, &dst)));
    TensorInfo w_bad_k(TensorShape(201U, 30U), 1, DataType::QASYMM8, q);
    EXPECT(!bool(NEFullyConnectedLayer::validate(&src, &w_bad_k, &b, &dst)));          // num_inputs mismatch
    TensorInfo w3(TensorShape(200U, 30U, 2U), 1, DataType::QASYMM8, q);
    EXPECT(!bool(NEFullyConnectedLayer::validate(&src, &w3, &b, &dst)));               // weights with more than 2 dimensions
    TensorInfo w_s8(TensorShape(200U, 30U), 1, DataType::QASYMM8_SIGNED, q);
    EXPECT(!bool(NEFullyConnectedLayer::validate(&src, &w_s8, &b, &dst)));             // mismatching data types
    TensorInfo b_f32(TensorShape(30U), 1, DataType::F32);
    EXPECT(!bool(NEFullyConnectedLayer::validate(&src, &w, &b_f32, &dst)));            // quantized needs S32 biases
    TensorInfo b2(TensorShape(30U, 2U), 1, DataType::S32);
    EXPECT(!bool(NEFullyConnectedLayer::validate(&src, &w, &b2, &dst)));               // biases with more than 1 dimension
    TensorInfo dst_bad(TensorShape(31U, 4U), 1, DataType::QASYMM8, q);
    EXPECT(!bool(NEFullyConnectedLayer::validate(&src, &w, &b, &dst_bad)));
    FullyConnectedLayerInfo tanh_info;
    tanh_info.activation_info = ActivationLayerInfo(ActivationLayerInfo::ActivationFunction::TANH);
    EXPECT(!bool(NEFullyConnectedLayer::validate(&src, &w, &b, &dst, tanh_info)));     // only the RELU family fuses
    FullyConnectedLayerInfo relu_info;
    relu_info.activation_info = ActivationLayerInfo(ActivationLayerInfo::ActivationFunction::LU_BOUNDED_RELU, 6.f, -1.f);
    EXPECT(bool(NEFullyConnectedLayer::validate(&src, &w, &b, &dst, relu_info)));
    TensorInfo f_src(TensorShape(200U, 4U), 1, DataType::F32), f_w(TensorShape(200U, 30U), 1, DataType::F32);
    TensorInfo f_dst(TensorShape(30U, 4U), 1, DataType::F32);
    const Status st = NEFullyConnectedLayer::validate(&f_src, &f_w, nullptr, &f_dst);
    EXPECT(!bool(st) && st.error_description().find("not built") != std::string::npos); // out of scope, and says so
    // after a convolution: the flattened input must match the weights
    TensorInfo conv_src(TensorShape(16U, 3U, 5U, 4U), 1, DataType::QASYMM8, q), conv_w(TensorShape(240U, 30U), 1, DataType::QASYMM8, q);
    conv_src.set_data_layout(DataLayout::NHWC);
    EXPECT(bool(NEFullyConnectedLayer::validate(&conv_src, &conv_w, &b, &dst)));
    EXPECT(!bool(NEFullyConnectedLayer::validate(&conv_src, &w, &b, &dst)));
    WeightFormat wf = WeightFormat::ANY;
    EXPECT(!bool(NEFullyConnectedLayer::has_opt_impl(wf, &src, &w, &b, &dst, FullyConnectedLayerInfo(), WeightsInfo())));
    EXPECT(wf == WeightFormat::UNSPECIFIED);
}

// accept / reject rules of CpuGemmDirectConv2d::validate (src/cpu/operators/CpuGemmDirectConv2d.cpp:166-224 of the reference)
static void test_gemm_conv2d_validate()
{
    SECTION("NEGEMMConv2d::validate accept / reject");
    TensorInfo src(TensorShape(16U, 9U, 9U, 2U), 1, DataType::QASYMM8, QuantizationInfo(0.1f, 3));
    TensorInfo w(TensorShape(16U, 3U, 3U, 8U), 1, DataType::QASYMM8, QuantizationInfo(0.1f, 3));
    TensorInfo b(TensorShape(8U), 1, DataType::S32), dst(TensorShape(8U, 7U, 7U, 2U), 1, DataType::QASYMM8, QuantizationInfo(0.5f, 1));
    for (TensorInfo *t : {&src, &w, &dst})
        t->set_data_layout(DataLayout::NHWC);
    const PadStrideInfo ps(1, 1, 0, 0);
    EXPECT(bool(NEGEMMConv2d::validate(&src, &w, &b, &dst, Conv2dInfo(ps, Size2D(1, 1), ActivationLayerInfo(), false, 1))));
    EXPECT(!bool(NEGEMMConv2d::validate(&src, &w, &b, &dst, Conv2dInfo(ps, Size2D(2, 2), ActivationLayerInfo(), false, 1)))); // dilation
    EXPECT(!bool(NEGEMMConv2d::validate(&src, &w, &b, &dst, Conv2dInfo(ps, Size2D(1, 1), ActivationLayerInfo(), false, 2)))); // groups
    TensorInfo src_nchw(src);
    src_nchw.set_data_layout(DataLayout::NCHW);
    EXPECT(!bool(NEGEMMConv2d::validate(&src_nchw, &w, &b, &dst, Conv2dInfo(ps, Size2D(1, 1), ActivationLayerInfo(), false, 1))));
    TensorInfo w_bad(TensorShape(15U, 3U, 3U, 8U), 1, DataType::QASYMM8, QuantizationInfo(0.1f, 3));
    w_bad.set_data_layout(DataLayout::NHWC);
    EXPECT(!bool(NEGEMMConv2d::validate(&src, &w_bad, &b, &dst, Conv2dInfo(ps, Size2D(1, 1), ActivationLayerInfo(), false, 1))));
}

// ---------------------------------------------------------------------------------------------------------------------
// GPU tests
// ---------------------------------------------------------------------------------------------------------------------
template <typename T>
static void fill_uniform(Tensor &t, int lo, int hi, unsigned seed)
{
    // element-wise through the tensor's strides, so padded tensors are filled correctly
    std::mt19937                       rng(seed);
    std::uniform_int_distribution<int> u(lo, hi);
    const ITensorInfo                 *i = t.info();
    const size_t rows = i->tensor_shape().total_size_upper(1);
    for (size_t r = 0; r < rows; ++r)
    {
        // decompose r into coordinates of dims 1..5
        size_t  rem = r;
        int32_t off = static_cast<int32_t>(i->offset_first_element_in_bytes());
        for (size_t d = 1; d < MAX_DIMS; ++d)
        {
            const size_t dim = i->tensor_shape()[d];
            off += static_cast<int32_t>((rem % dim) * i->strides_in_bytes()[d]);
            rem /= dim;
        }
        T *row = reinterpret_cast<T *>(t.buffer() + off);
        for (size_t x = 0; x < i->dimension(0); ++x)
            row[x] = static_cast<T>(u(rng));
    }
}

template <typename T>
static std::vector<T> dense_copy(const Tensor &t)
{
    const ITensorInfo *i = t.info();
    std::vector<T>     out(i->tensor_shape().total_size());
    const size_t       rows = i->tensor_shape().total_size_upper(1), w = i->dimension(0);
    for (size_t r = 0; r < rows; ++r)
    {
        size_t  rem = r;
        int32_t off = static_cast<int32_t>(i->offset_first_element_in_bytes());
        for (size_t d = 1; d < MAX_DIMS; ++d)
        {
            const size_t dim = i->tensor_shape()[d];
            off += static_cast<int32_t>((rem % dim) * i->strides_in_bytes()[d]);
            rem /= dim;
        }
        std::memcpy(out.data() + r * w, t.buffer() + off, w * sizeof(T));
    }
    return out;
}

static void init_tensor(Tensor &t, const TensorShape &shape, DataType dt, const QuantizationInfo &q = QuantizationInfo(),
                        const PaddingSize &pad = PaddingSize(0))
{
    TensorInfo info(shape, 1, dt, q);
    t.allocator()->init(info);
    if (!pad.empty())
        t.info()->extend_padding(pad);
}

// the flow of examples/neon_gemm_qasymm8.cpp of the reference: configure first, allocate afterwards, run twice
static void test_gemmlowp_fused_u8(bool padded)
{
    SECTION(padded ? "NEGEMMLowpMatrixMultiplyCore fused QASYMM8 (x-padded tensors)" : "NEGEMMLowpMatrixMultiplyCore fused QASYMM8");
    const int   M = 72, N = 33, K = 52;
    Tensor      a, b, bias, dst;
    init_tensor(a, TensorShape(K, M), DataType::QASYMM8, QuantizationInfo(1.f / 255, -9));
    init_tensor(b, TensorShape(N, K), DataType::QASYMM8, QuantizationInfo(1.f / 255, 1));
    init_tensor(bias, TensorShape(N), DataType::S32);
    init_tensor(dst, TensorShape(N, M), DataType::QASYMM8, QuantizationInfo(0.3f, 10));
    GEMMLowpOutputStageInfo st;
    st.type = GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT;
    st.gemmlowp_multiplier = 1518500250, st.gemmlowp_shift = 8, st.gemmlowp_offset = 10;
    st.gemmlowp_min_bound = 0, st.gemmlowp_max_bound = 255, st.output_data_type = DataType::QASYMM8;
    NEGEMMLowpMatrixMultiplyCore gemm;
    gemm.configure(&a, &b, &bias, &dst, GEMMInfo(false, false, true, 0, false, false, st));
    if (padded)
    {
        // the order of the reference's fixture: configure, then add_padding_x, then allocate
        // (tests/validation/fixtures/GEMMLowpFixture.h:289-310)
        a.info()->extend_padding(PaddingSize(0, 5, 0, 3)), b.info()->extend_padding(PaddingSize(0, 11, 0, 2));
        dst.info()->extend_padding(PaddingSize(0, 1, 0, 16)), bias.info()->extend_padding(PaddingSize(0, 3, 0, 4));
    }
    a.allocator()->allocate(), b.allocator()->allocate(), bias.allocator()->allocate(), dst.allocator()->allocate();
    fill_uniform<uint8_t>(a, 0, 255, 1), fill_uniform<uint8_t>(b, 0, 255, 2), fill_uniform<int32_t>(bias, -1000, 1000, 3);
    const auto A = dense_copy<uint8_t>(a), B = dense_copy<uint8_t>(b);
    const auto C = dense_copy<int32_t>(bias);
    std::vector<uint8_t> want(M * N);
    const int32_t mult = st.gemmlowp_multiplier, shift = st.gemmlowp_shift;
    orc_gemmlowp_fixedpoint(A.data(), 0, K, B.data(), 0, N, C.data(), want.data(), N, 0, M, N, K, -9, 1, &mult, &shift, 1, 10, 0, 255);
    gemm.run();
    EXPECT(dense_copy<uint8_t>(dst) == want);
    EXPECT(!b.is_used()); // B was packed once and handed back (NEGEMMLowpMatrixMultiplyCore.cpp:176-183 of the reference)
    // run again with a new A: identical function object, new data
    fill_uniform<uint8_t>(a, 0, 255, 11);
    const auto A2 = dense_copy<uint8_t>(a);
    orc_gemmlowp_fixedpoint(A2.data(), 0, K, B.data(), 0, N, C.data(), want.data(), N, 0, M, N, K, -9, 1, &mult, &shift, 1, 10, 0, 255);
    gemm.run();
    EXPECT(dense_copy<uint8_t>(dst) == want);
    std::printf("       kernel: %s\n", gemm.kernel_name());
}

static void test_gemmlowp_s32_batched()
{
    SECTION("NEGEMMLowpMatrixMultiplyCore S32 output, batched, non-constant B");
    const int M = 17, N = 29, K = 15, batch = 3;
    Tensor    a, b, dst;
    init_tensor(a, TensorShape(K, M, batch), DataType::QASYMM8_SIGNED, QuantizationInfo(0.1f, 5));
    init_tensor(b, TensorShape(N, K, batch), DataType::QASYMM8_SIGNED, QuantizationInfo(0.2f, -7));
    init_tensor(dst, TensorShape(N, M, batch), DataType::S32);
    a.allocator()->allocate(), b.allocator()->allocate(), dst.allocator()->allocate();
    NEGEMMLowpMatrixMultiplyCore gemm;
    gemm.configure(&a, &b, nullptr, &dst, GEMMInfo(false, false, false /* B changes between runs */));
    for (int rep = 0; rep < 2; ++rep)
    {
        fill_uniform<int8_t>(a, -128, 127, 20 + rep), fill_uniform<int8_t>(b, -128, 127, 30 + rep);
        const auto A = dense_copy<int8_t>(a), B = dense_copy<int8_t>(b);
        std::vector<int32_t> want(batch * M * N);
        for (int z = 0; z < batch; ++z)
            orc_gemmlowp_s32(A.data() + z * M * K, 1, K, B.data() + z * K * N, 1, N, want.data() + z * M * N, N, M, N, K, 5, -7);
        gemm.run();
        EXPECT(dense_copy<int32_t>(dst) == want);
        EXPECT(b.is_used());
    }
}

// GEMMInfo::accumulate (the fixture of tests/validation/fixtures/GEMMLowpFixture.h:187-193,469-483: the destination is
// filled first and the product is added to it) and a [K, W, H, batch] input read as W*H rows with a 3D output
static void test_gemmlowp_accumulate_and_3d()
{
    SECTION("NEGEMMLowpMatrixMultiplyCore accumulate into S32 / F32; reinterpret_input_as_3d + depth_output_gemm3d");
    const int M = 23, N = 37, K = 40;
    {
        Tensor a, b, dst;
        init_tensor(a, TensorShape(K, M), DataType::QASYMM8, QuantizationInfo(1.f / 255, 3));
        init_tensor(b, TensorShape(N, K), DataType::QASYMM8, QuantizationInfo(1.f / 255, -9));
        init_tensor(dst, TensorShape(N, M), DataType::S32);
        a.allocator()->allocate(), b.allocator()->allocate(), dst.allocator()->allocate();
        fill_uniform<uint8_t>(a, 0, 255, 1), fill_uniform<uint8_t>(b, 0, 255, 2);
        fill_uniform<int32_t>(dst, -100000, 100000, 3);
        const auto prev = dense_copy<int32_t>(dst);
        GEMMInfo   info;
        info.set_accumulate(true);
        EXPECT(bool(NEGEMMLowpMatrixMultiplyCore::validate(a.info(), b.info(), nullptr, dst.info(), info)));
        NEGEMMLowpMatrixMultiplyCore gemm;
        gemm.configure(&a, &b, nullptr, &dst, info);
        gemm.run();
        const auto A = dense_copy<uint8_t>(a), B = dense_copy<uint8_t>(b);
        std::vector<int32_t> want(M * N);
        orc_gemmlowp_s32(A.data(), 0, K, B.data(), 0, N, want.data(), N, M, N, K, 3, -9);
        for (int i = 0; i < M * N; ++i)
            want[i] += prev[i];
        EXPECT(dense_copy<int32_t>(dst) == want);
    }
    {
        Tensor a, b, dst;
        init_tensor(a, TensorShape(K, M), DataType::QASYMM8_SIGNED, QuantizationInfo(0.02f, 0));
        init_tensor(b, TensorShape(N, K), DataType::QASYMM8_SIGNED, QuantizationInfo(0.005f, 0));
        init_tensor(dst, TensorShape(N, M), DataType::F32);
        a.allocator()->allocate(), b.allocator()->allocate(), dst.allocator()->allocate();
        fill_uniform<int8_t>(a, -128, 127, 4), fill_uniform<int8_t>(b, -128, 127, 5);
        std::mt19937                    rng(6);
        std::normal_distribution<float> nd(0.f, 2.f);
        for (int i = 0; i < M * N; ++i)
            reinterpret_cast<float *>(dst.buffer())[i] = nd(rng);
        auto     want = dense_copy<float>(dst);
        GEMMInfo info(false, false, true);
        info.set_accumulate(true);
        NEGEMMLowpMatrixMultiplyCore gemm;
        gemm.configure(&a, &b, nullptr, &dst, info);
        gemm.run();
        const auto A = dense_copy<int8_t>(a), B = dense_copy<int8_t>(b);
        orc_gemmlowp_f32(A.data(), 1, K, B.data(), 1, N, nullptr, want.data(), N, M, N, K, 0, 0, 0.02f * 0.005f, -INFINITY,
                         INFINITY, 1, 0);
        EXPECT(dense_copy<float>(dst) == want);
    }
    for (int accumulate = 0; accumulate < 2; ++accumulate)
    {
        // F16 destination (tests/validation/NEON/GEMMLowp.cpp:598-621: the reference's small dataset, signed operands,
        // QuantizationInfo(1/255, a_offset) x QuantizationInfo(5/255, b_offset), with and without accumulation)
        Tensor a, b, dst;
        init_tensor(a, TensorShape(K, M), DataType::QASYMM8_SIGNED, QuantizationInfo(1.f / 255, -3));
        init_tensor(b, TensorShape(N, K), DataType::QASYMM8_SIGNED, QuantizationInfo(5.f / 255, 2));
        init_tensor(dst, TensorShape(N, M), DataType::F16);
        a.allocator()->allocate(), b.allocator()->allocate(), dst.allocator()->allocate();
        fill_uniform<int8_t>(a, -128, 127, 14), fill_uniform<int8_t>(b, -128, 127, 15);
        std::mt19937                    rng(16);
        std::normal_distribution<float> nd(0.f, 2.f);
        for (size_t y = 0; y < (size_t)M; ++y)
            for (size_t x = 0; x < (size_t)N; ++x)
                *reinterpret_cast<uint16_t *>(dst.ptr_to_element(Coordinates(x, y))) = orc_f32_to_f16(nd(rng));
        auto     want = dense_copy<uint16_t>(dst);
        GEMMInfo info(false, false, true);
        info.set_accumulate(accumulate != 0);
        EXPECT(bool(NEGEMMLowpMatrixMultiplyCore::validate(a.info(), b.info(), nullptr, dst.info(), info)));
        NEGEMMLowpMatrixMultiplyCore gemm;
        gemm.configure(&a, &b, nullptr, &dst, info);
        gemm.run();
        const auto A = dense_copy<int8_t>(a), B = dense_copy<int8_t>(b);
        orc_gemmlowp_f16(A.data(), 1, K, B.data(), 1, N, nullptr, want.data(), N, M, N, K, -3, 2, (1.f / 255) * (5.f / 255),
                         -INFINITY, INFINITY, accumulate, 0);
        EXPECT(dense_copy<uint16_t>(dst) == want);
        // unsigned operands are not part of the half leg
        Tensor ua;
        init_tensor(ua, TensorShape(K, M), DataType::QASYMM8, QuantizationInfo(1.f / 255, 3));
        EXPECT(!bool(NEGEMMLowpMatrixMultiplyCore::validate(ua.info(), b.info(), nullptr, dst.info(), info)));
    }
    {
        // a = [K, W, H, batch] -> M = W*H rows per batch; dst = [N, W, H, batch]
        const int W = 5, H = 4, batch = 2;
        Tensor    a, b, dst;
        init_tensor(a, TensorShape(K, W, H, batch), DataType::QASYMM8_SIGNED, QuantizationInfo(0.1f, 2));
        init_tensor(b, TensorShape(N, K), DataType::QASYMM8_SIGNED, QuantizationInfo(0.2f, -1));
        init_tensor(dst, TensorShape(N, W, H, batch), DataType::S32);
        a.allocator()->allocate(), b.allocator()->allocate(), dst.allocator()->allocate();
        fill_uniform<int8_t>(a, -128, 127, 7), fill_uniform<int8_t>(b, -128, 127, 8);
        GEMMInfo info(false, false, true, H /* depth_output_gemm3d */, true /* reinterpret_input_as_3d */);
        EXPECT(bool(NEGEMMLowpMatrixMultiplyCore::validate(a.info(), b.info(), nullptr, dst.info(), info)));
        NEGEMMLowpMatrixMultiplyCore gemm;
        gemm.configure(&a, &b, nullptr, &dst, info);
        gemm.run();
        const auto A = dense_copy<int8_t>(a), B = dense_copy<int8_t>(b);
        std::vector<int32_t> want(batch * W * H * N);
        orc_gemmlowp_s32(A.data(), 1, K, B.data(), 1, N, want.data(), N, batch * W * H, N, K, 2, -1);
        EXPECT(dense_copy<int32_t>(dst) == want);
        // the same with both 3D tensors padded along x and y after configure (gaps between the planes of W rows:
        // strides_in_bytes()[2] > W * strides_in_bytes()[1]), a fused output stage, and the padding of dst left alone
        {
            Tensor a2, dst2;
            init_tensor(a2, TensorShape(K, W, H, batch), DataType::QASYMM8_SIGNED, QuantizationInfo(0.1f, 2));
            init_tensor(dst2, TensorShape(N, W, H, batch), DataType::QASYMM8_SIGNED, QuantizationInfo(0.7f, 3));
            GEMMLowpOutputStageInfo st;
            EXPECT(bool(quantization::calculate_quantized_multipliers(QuantizationInfo(0.1f, 2), QuantizationInfo(0.2f, -1),
                                                                      QuantizationInfo(0.7f, 3), st)));
            st.type                = GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT;
            st.gemmlowp_offset     = 3;
            st.gemmlowp_min_bound  = -128;
            st.gemmlowp_max_bound  = 127;
            st.output_data_type    = DataType::QASYMM8_SIGNED;
            st.gemmlowp_multiplier = st.gemmlowp_multipliers[0];
            st.gemmlowp_shift      = st.gemmlowp_shifts[0];
            GEMMInfo info2(false, false, true, H, true);
            info2.set_gemmlowp_output_stage(st);
            NEGEMMLowpMatrixMultiplyCore gemm2;
            gemm2.configure(&a2, &b, nullptr, &dst2, info2);
            a2.info()->extend_padding(PaddingSize(2, 5, 1, 3)); // top, right, bottom, left
            dst2.info()->extend_padding(PaddingSize(1, 4, 2, 0));
            a2.allocator()->allocate(), dst2.allocator()->allocate();
            EXPECT(a2.info()->strides_in_bytes()[2] > W * a2.info()->strides_in_bytes()[1]);
            fill_uniform<int8_t>(a2, -128, 127, 9);
            std::memset(dst2.buffer(), 0x5A, dst2.info()->total_size());
            gemm2.run();
            const auto A2 = dense_copy<int8_t>(a2);
            std::vector<int8_t> want2(batch * W * H * N);
            orc_gemmlowp_fixedpoint(A2.data(), 1, K, B.data(), 1, N, nullptr, want2.data(), N, 1, batch * W * H, N, K, 2, -1,
                                    &st.gemmlowp_multiplier, &st.gemmlowp_shift, 1, 3, -128, 127);
            EXPECT(dense_copy<int8_t>(dst2) == want2);
            size_t untouched = 0, padding = dst2.info()->total_size() - (size_t)batch * W * H * N;
            for (size_t i = 0; i < dst2.info()->total_size(); ++i)
                untouched += dst2.buffer()[i] == 0x5A;
            EXPECT(untouched >= padding);
            std::printf("       kernel: %s (planes %zu bytes apart for %d rows of %zu)\n", gemm2.kernel_name(),
                        (size_t)a2.info()->strides_in_bytes()[2], W, (size_t)a2.info()->strides_in_bytes()[1]);
        }
        // a 3D input without a 3D output is not built
        Tensor flat;
        init_tensor(flat, TensorShape(N, W * H, batch), DataType::S32);
        EXPECT(!bool(NEGEMMLowpMatrixMultiplyCore::validate(a.info(), b.info(), nullptr, flat.info(),
                                                            GEMMInfo(false, false, true, 0, true))));
    }
}

// dynamic quantization info: offsets (and the F32 path's scale) are read again on every run
// (src/cpu/operators/CpuGemmLowpMatrixMultiplyCore.cpp:668-674,758-784; the fixture sets it after configure,
// tests/validation/fixtures/GEMMLowpFixture.h:171-185)
static void test_gemmlowp_dynamic_qinfo()
{
    SECTION("NEGEMMLowpMatrixMultiplyCore with dynamic quantization info (S32 and F32 destinations)");
    const int M = 19, N = 33, K = 48;
    for (int f32 = 0; f32 < 2; ++f32)
    {
        Tensor a, b, dst;
        init_tensor(a, TensorShape(K, M), DataType::QASYMM8_SIGNED, QuantizationInfo(1.f, 0, true));
        init_tensor(b, TensorShape(N, K), DataType::QASYMM8_SIGNED, QuantizationInfo(1.f, 0, true));
        init_tensor(dst, TensorShape(N, M), f32 ? DataType::F32 : DataType::S32);
        a.allocator()->allocate(), b.allocator()->allocate(), dst.allocator()->allocate();
        fill_uniform<int8_t>(a, -128, 127, 90 + f32), fill_uniform<int8_t>(b, -128, 127, 92 + f32);
        NEGEMMLowpMatrixMultiplyCore gemm;
        gemm.configure(&a, &b, nullptr, &dst, GEMMInfo(false, false, true));
        const auto A = dense_copy<int8_t>(a), B = dense_copy<int8_t>(b);
        const struct { float sa, sb; int ao, bo; } steps[] = {{0.5f, 0.25f, 0, 0}, {0.02f, 0.005f, 7, -4}, {0.1f, 0.005f, 7, -4},
                                                              {0.1f, 0.3f, -11, 0}};
        for (const auto &st : steps)
        {
            a.info()->set_quantization_info(QuantizationInfo(st.sa, st.ao, true));
            b.info()->set_quantization_info(QuantizationInfo(st.sb, st.bo, true));
            gemm.run();
            if (f32)
            {
                std::vector<float> want(M * N);
                orc_gemmlowp_f32(A.data(), 1, K, B.data(), 1, N, nullptr, want.data(), N, M, N, K, st.ao, st.bo, st.sa * st.sb,
                                 -INFINITY, INFINITY, 0, 0);
                EXPECT(dense_copy<float>(dst) == want);
            }
            else
            {
                std::vector<int32_t> want(M * N);
                orc_gemmlowp_s32(A.data(), 1, K, B.data(), 1, N, want.data(), N, M, N, K, st.ao, st.bo);
                EXPECT(dense_copy<int32_t>(dst) == want);
            }
        }
    }
}

// The shapes and offsets of the reference's small datasets, through the function classes with padded tensors:
// tests/datasets/SmallGEMMLowpDataset.h:42-65 (S32 output, 2D and 3D), tests/datasets/GEMMLowpFusedOffsetOutputDataset.h:
// 120-165 (fused fixed-point output; batched B that changes between runs)
static void test_reference_small_datasets()
{
    SECTION("the reference's SmallGEMMLowp / FusedOffsetOutput / BatchedMatMul dataset shapes");
    struct Cfg { int K, M, N, batch, depth3d, ao, bo; };
    const Cfg s32_cfgs[] = {{21, 1, 1, 1, 0, 0, 0},    {21, 13, 33, 1, 0, 0, 0},  {31, 3, 72, 1, 0, -2, 13}, {52, 13, 33, 1, 0, 0, 4},
                            {52, 26, 33, 1, 0, -2, 0}, {31, 27, 23, 1, 0, 5, 13}, {38, 43, 21, 1, 0, -3, -2}, {32, 72, 17, 1, 0, -9, 1},
                            {21, 14, 34, 1, 7, 0, 0},  {31, 1, 3, 1, 1, -2, 13}};
    unsigned seed = 500;
    for (const Cfg &c : s32_cfgs)
    {
        Tensor a, b, dst;
        init_tensor(a, TensorShape(c.K, c.M), DataType::QASYMM8, QuantizationInfo(1.f / 255, c.ao));
        init_tensor(b, TensorShape(c.N, c.K), DataType::QASYMM8, QuantizationInfo(1.f / 255, c.bo));
        init_tensor(dst, c.depth3d ? TensorShape(c.N, c.depth3d, c.M / c.depth3d) : TensorShape(c.N, c.M), DataType::S32);
        NEGEMMLowpMatrixMultiplyCore gemm;
        gemm.configure(&a, &b, nullptr, &dst, GEMMInfo(false, false, false, c.depth3d));
        a.info()->extend_padding(PaddingSize(0, 1 + seed % 16, 0, 1 + seed % 7)), b.info()->extend_padding(PaddingSize(0, 3, 0, 16));
        if (!c.depth3d)
            dst.info()->extend_padding(PaddingSize(0, 5, 0, 2));
        a.allocator()->allocate(), b.allocator()->allocate(), dst.allocator()->allocate();
        fill_uniform<uint8_t>(a, 0, 255, seed++), fill_uniform<uint8_t>(b, 0, 255, seed++);
        gemm.run();
        const auto A = dense_copy<uint8_t>(a), B = dense_copy<uint8_t>(b);
        std::vector<int32_t> want(c.M * c.N);
        orc_gemmlowp_s32(A.data(), 0, c.K, B.data(), 0, c.N, want.data(), c.N, c.M, c.N, c.K, c.ao, c.bo);
        EXPECT(dense_copy<int32_t>(dst) == want);
    }
    const Cfg fused_cfgs[] = {{21, 13, 1, 1, 0, 3, -7},   {52, 13, 33, 1, 0, -12, 5},  {31, 27, 23, 1, 0, 0, 9},    {32, 72, 16, 1, 0, -1, 0},
                              {21, 1, 43, 1, 0, 6, 6},    {31, 3, 72, 1, 0, -20, 11},  {32, 72, 17, 1, 0, 2, -3},
                              {4, 3, 2, 1, 0, 1, 1},      {12, 15, 7, 1, 0, -5, 2},    {59, 17, 36, 1, 0, 7, -8},   {2, 4, 5, 3, 0, -3, 4},
                              {15, 7, 29, 3, 0, 10, -2},  {56, 17, 5, 32, 0, -9, 9},   {13, 256, 19, 32, 0, 4, -6}};
    for (const Cfg &c : fused_cfgs)
        for (int sgn = 0; sgn < 2; ++sgn)
        {
            const DataType dt = sgn ? DataType::QASYMM8_SIGNED : DataType::QASYMM8;
            const int      ao = c.ao + (sgn ? 0 : -128), bo = c.bo + (sgn ? 0 : -128); // zero-mean products for both types
            Tensor         a, b, bias, dst;
            init_tensor(a, c.batch > 1 ? TensorShape(c.K, c.M, c.batch) : TensorShape(c.K, c.M), dt, QuantizationInfo(0.05f, ao));
            init_tensor(b, c.batch > 1 ? TensorShape(c.N, c.K, c.batch) : TensorShape(c.N, c.K), dt, QuantizationInfo(0.02f, bo));
            init_tensor(bias, TensorShape(c.N), DataType::S32);
            init_tensor(dst, c.batch > 1 ? TensorShape(c.N, c.M, c.batch) : TensorShape(c.N, c.M), dt, QuantizationInfo(1.f, sgn ? -3 : 120));
            GEMMLowpOutputStageInfo st;
            st.type = GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT, st.output_data_type = dt;
            st.gemmlowp_offset = sgn ? -3 : 120, st.gemmlowp_min_bound = sgn ? -128 : 0, st.gemmlowp_max_bound = sgn ? 127 : 255;
            // products of K terms of magnitude ~74*74: bring one standard deviation to about 60 output steps
            EXPECT(bool(quantization::calculate_quantized_multiplier(60.f / (5476.f * std::sqrt((float)c.K)), &st.gemmlowp_multiplier,
                                                                     &st.gemmlowp_shift)));
            NEGEMMLowpMatrixMultiplyCore gemm;
            gemm.configure(&a, &b, &bias, &dst, GEMMInfo(false, false, c.batch == 1 /* batched B changes */, 0, false, false, st));
            a.info()->extend_padding(PaddingSize(0, 2, 0, 9)), dst.info()->extend_padding(PaddingSize(0, 8, 0, 1));
            a.allocator()->allocate(), b.allocator()->allocate(), bias.allocator()->allocate(), dst.allocator()->allocate();
            for (int rep = 0; rep < (c.batch > 1 ? 2 : 1); ++rep)
            {
                if (sgn)
                    fill_uniform<int8_t>(a, -128, 127, seed++), fill_uniform<int8_t>(b, -128, 127, seed++);
                else
                    fill_uniform<uint8_t>(a, 0, 255, seed++), fill_uniform<uint8_t>(b, 0, 255, seed++);
                fill_uniform<int32_t>(bias, -2000, 2000, seed++);
                gemm.run();
                const auto A = dense_copy<uint8_t>(a), B = dense_copy<uint8_t>(b);
                const auto Cb = dense_copy<int32_t>(bias);
                std::vector<uint8_t> want((size_t)c.batch * c.M * c.N);
                for (int z = 0; z < c.batch; ++z)
                    orc_gemmlowp_fixedpoint(A.data() + (size_t)z * c.M * c.K, sgn, c.K, B.data() + (size_t)z * c.K * c.N, sgn, c.N,
                                            Cb.data(), want.data() + (size_t)z * c.M * c.N, c.N, sgn, c.M, c.N, c.K,
                                            ao, bo, &st.gemmlowp_multiplier,
                                            &st.gemmlowp_shift, 1, st.gemmlowp_offset, st.gemmlowp_min_bound, st.gemmlowp_max_bound);
                EXPECT(dense_copy<uint8_t>(dst) == want);
            }
        }
}

static void test_gemmlowp_per_channel_and_update()
{
    SECTION("NEGEMMLowpMatrixMultiplyCore per-channel QSYMM8_PER_CHANNEL rhs");
    const int M = 150, N = 130, K = 208;
    std::mt19937 rng(5);
    std::uniform_real_distribution<float> us(1e-4f, 2e-2f);
    std::vector<float> wscale(N);
    for (auto &v : wscale)
        v = us(rng);
    Tensor a, b, bias, dst;
    init_tensor(a, TensorShape(K, M), DataType::QASYMM8_SIGNED, QuantizationInfo(0.05f, -3)); // offsets are ADDED: zero point 3
    init_tensor(b, TensorShape(N, K), DataType::QSYMM8_PER_CHANNEL, QuantizationInfo(wscale));
    init_tensor(bias, TensorShape(N), DataType::S32);
    init_tensor(dst, TensorShape(N, M), DataType::QASYMM8_SIGNED, QuantizationInfo(0.7f, -5));
    GEMMLowpOutputStageInfo st;
    st.type = GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT;
    st.gemmlowp_offset = -5, st.gemmlowp_min_bound = -128, st.gemmlowp_max_bound = 127;
    st.is_quantized_per_channel = true, st.output_data_type = DataType::QASYMM8_SIGNED;
    EXPECT(bool(quantization::calculate_quantized_multipliers(QuantizationInfo(0.05f, 3), QuantizationInfo(wscale),
                                                              QuantizationInfo(0.7f, -5), st)));
    a.allocator()->allocate(), b.allocator()->allocate(), bias.allocator()->allocate(), dst.allocator()->allocate();
    fill_uniform<int8_t>(a, -128, 127, 41), fill_uniform<int8_t>(b, -127, 127, 42), fill_uniform<int32_t>(bias, -2000, 2000, 43);
    NEGEMMLowpMatrixMultiplyCore gemm;
    gemm.configure(&a, &b, &bias, &dst, GEMMInfo(false, false, true, 0, false, false, st));
    gemm.run();
    const auto A = dense_copy<int8_t>(a), B = dense_copy<int8_t>(b);
    const auto C = dense_copy<int32_t>(bias);
    std::vector<int8_t> want(M * N);
    orc_gemmlowp_fixedpoint(A.data(), 1, K, B.data(), 1, N, C.data(), want.data(), N, 1, M, N, K, -3, 0,
                            st.gemmlowp_multipliers.data(), st.gemmlowp_shifts.data(), N, -5, -128, 127);
    EXPECT(dense_copy<int8_t>(dst) == want);

    SECTION("update_quantization_parameters (per tensor) after configure");
    Tensor a2, b2, dst2;
    init_tensor(a2, TensorShape(K, M), DataType::QASYMM8, QuantizationInfo(0.05f, 2));
    init_tensor(b2, TensorShape(N, K), DataType::QASYMM8, QuantizationInfo(0.01f, 4));
    init_tensor(dst2, TensorShape(N, M), DataType::QASYMM8, QuantizationInfo(0.9f, 7));
    GEMMLowpOutputStageInfo st2;
    st2.type = GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT;
    st2.gemmlowp_multiplier = 1 << 30, st2.gemmlowp_shift = 12, st2.gemmlowp_offset = 0;
    st2.gemmlowp_min_bound = 0, st2.gemmlowp_max_bound = 255, st2.output_data_type = DataType::QASYMM8;
    a2.allocator()->allocate(), b2.allocator()->allocate(), dst2.allocator()->allocate();
    fill_uniform<uint8_t>(a2, 0, 255, 51), fill_uniform<uint8_t>(b2, 0, 255, 52);
    NEGEMMLowpMatrixMultiplyCore g2;
    g2.configure(&a2, &b2, nullptr, &dst2, GEMMInfo(false, false, true, 0, false, false, st2));
    g2.run();
    // new quantization on the tensors, as the reference's UpdateStaticQuantInfoAfterConfigure tests do
    a2.info()->set_quantization_info(QuantizationInfo(0.04f, -100));
    b2.info()->set_quantization_info(QuantizationInfo(0.02f, -120));
    dst2.info()->set_quantization_info(QuantizationInfo(1.3f, 17));
    g2.update_quantization_parameters();
    g2.run();
    int32_t m = 0, s = 0;
    EXPECT(bool(quantization::calculate_quantized_multiplier(0.04f * 0.02f / 1.3f, &m, &s)));
    const auto A2 = dense_copy<uint8_t>(a2), B2 = dense_copy<uint8_t>(b2);
    std::vector<uint8_t> want2(M * N);
    orc_gemmlowp_fixedpoint(A2.data(), 0, K, B2.data(), 0, N, nullptr, want2.data(), N, 0, M, N, K, -100, -120, &m, &s, 1, 17, 0, 255);
    EXPECT(dense_copy<uint8_t>(dst2) == want2);
}

static void test_gemmlowp_f32()
{
    SECTION("NEGEMMLowpMatrixMultiplyCore F32 dequantized output with F32 bias and fused RELU");
    const int M = 40, N = 65, K = 1000;
    Tensor    a, b, bias, dst;
    init_tensor(a, TensorShape(K, M), DataType::QASYMM8_SIGNED, QuantizationInfo(0.02f, 3));
    init_tensor(b, TensorShape(N, K), DataType::QASYMM8_SIGNED, QuantizationInfo(0.005f, -2));
    init_tensor(bias, TensorShape(N), DataType::F32);
    init_tensor(dst, TensorShape(N, M), DataType::F32);
    a.allocator()->allocate(), b.allocator()->allocate(), bias.allocator()->allocate(), dst.allocator()->allocate();
    fill_uniform<int8_t>(a, -128, 127, 61), fill_uniform<int8_t>(b, -128, 127, 62);
    std::mt19937 rng(63);
    std::normal_distribution<float> nd(0.f, 2.f);
    for (int j = 0; j < N; ++j)
        reinterpret_cast<float *>(bias.buffer())[j] = nd(rng);
    GEMMInfo info(false, false, true, 0, false, false, GEMMLowpOutputStageInfo(), false, false, false,
                  ActivationLayerInfo(ActivationLayerInfo::ActivationFunction::RELU));
    NEGEMMLowpMatrixMultiplyCore gemm;
    gemm.configure(&a, &b, &bias, &dst, info);
    gemm.run();
    const auto A = dense_copy<int8_t>(a), B = dense_copy<int8_t>(b);
    std::vector<float> want(M * N);
    orc_gemmlowp_f32(A.data(), 1, K, B.data(), 1, N, reinterpret_cast<const float *>(bias.buffer()), want.data(), N, M, N, K, 3,
                     -2, 0.02f * 0.005f, 0.f, INFINITY, 0, 1);
    const auto got = dense_copy<float>(dst);
    bool       ok  = true;
    for (size_t i = 0; i < want.size(); ++i)
        ok = ok && std::fabs(got[i] - want[i]) <= 1e-5f * std::fabs(want[i]) + 1e-30f; // the stated 1e-5 relative bar
    EXPECT(ok);
    EXPECT(got == want); // and in fact identical bits: same float operations in the same order
}

static void test_output_stage()
{
    SECTION("NEGEMMLowpOutputStage S32 -> QASYMM8_SIGNED with bias (output auto-initialised)");
    const int M = 13, N = 130;
    Tensor    src, bias, dst;
    init_tensor(src, TensorShape(N, M), DataType::S32);
    init_tensor(bias, TensorShape(N), DataType::S32);
    GEMMLowpOutputStageInfo os;
    os.type = GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT;
    os.gemmlowp_multiplier = 1288490240, os.gemmlowp_shift = 4, os.gemmlowp_offset = -3;
    os.gemmlowp_min_bound = -100, os.gemmlowp_max_bound = 120, os.output_data_type = DataType::QASYMM8_SIGNED;
    NEGEMMLowpOutputStage stage;
    stage.configure(&src, &bias, &dst, os);
    EXPECT(dst.info()->data_type() == DataType::QASYMM8_SIGNED && dst.info()->dimension(0) == (size_t)N);
    // padding after configure, before allocation, as the reference's fixture does
    src.info()->extend_padding(PaddingSize(0, 3, 0, 2)), dst.info()->extend_padding(PaddingSize(0, 9, 0, 5));
    src.allocator()->allocate(), bias.allocator()->allocate(), dst.allocator()->allocate();
    fill_uniform<int32_t>(src, -6000, 6000, 71), fill_uniform<int32_t>(bias, -6000, 6000, 72);
    stage.run();
    std::vector<int8_t> want(M * N);
    const auto src_d = dense_copy<int32_t>(src);
    orc_output_stage_fixedpoint(src_d.data(), N, reinterpret_cast<const int32_t *>(bias.buffer()),
                                want.data(), N, 1, M, N, &os.gemmlowp_multiplier, &os.gemmlowp_shift, 1, -3, -100, 120);
    EXPECT(dense_copy<int8_t>(dst) == want);

    SECTION("NEGEMMLowpOutputStage S32 -> QSYMM16 (rounding multiply, offset ignored)");
    Tensor dst16;
    os.gemmlowp_offset    = 9; // the int16 kernel is not given the offset (src/cpu/operators/CpuGemmLowpOutputStage.cpp:73-80)
    os.gemmlowp_min_bound = -30000, os.gemmlowp_max_bound = 32767, os.output_data_type = DataType::QSYMM16;
    os.gemmlowp_multiplier = 2000000000, os.gemmlowp_shift = 1;
    NEGEMMLowpOutputStage stage16;
    stage16.configure(&src, &bias, &dst16, os);
    EXPECT(dst16.info()->data_type() == DataType::QSYMM16);
    dst16.allocator()->allocate();
    fill_uniform<int32_t>(src, -100000, 100000, 73);
    stage16.run();
    std::vector<int16_t> want16(M * N);
    const auto src_d2 = dense_copy<int32_t>(src);
    orc_output_stage_fixedpoint_s16(src_d2.data(), N, reinterpret_cast<const int32_t *>(bias.buffer()), want16.data(), N, M, N,
                                    2000000000, 1, -30000, 32767);
    EXPECT(dense_copy<int16_t>(dst16) == want16);
    int lo_hits = 0, hi_hits = 0;
    for (int16_t v : want16)
        lo_hits += v == -30000, hi_hits += v == 32767;
    EXPECT(lo_hits > 0 && hi_hits > 0 && lo_hits + hi_hits < M * N / 2); // both bounds bite, most values are inside
    os.type = GEMMLowpOutputStageType::QUANTIZE_DOWN;
    EXPECT(!bool(NEGEMMLowpOutputStage::validate(src.info(), bias.info(), dst16.info(), os)));
}

// QUANTIZE_DOWN (integer multiplier): stand-alone stage without bounds (min == max) and fused into the GEMM
static void test_quantize_down_scale()
{
    SECTION("QUANTIZE_DOWN (integer multiplier): NEGEMMLowpOutputStage and fused NEGEMMLowpMatrixMultiplyCore");
    {
        const int M = 9, N = 77;
        Tensor    src, bias, dst;
        init_tensor(src, TensorShape(N, M), DataType::S32);
        init_tensor(bias, TensorShape(N), DataType::S32);
        init_tensor(dst, TensorShape(N, M), DataType::QASYMM8);
        GEMMLowpOutputStageInfo os;
        os.type = GEMMLowpOutputStageType::QUANTIZE_DOWN;
        os.gemmlowp_multiplier = 5, os.gemmlowp_shift = 9, os.gemmlowp_offset = -700;
        os.gemmlowp_min_bound = 0, os.gemmlowp_max_bound = 0, os.output_data_type = DataType::QASYMM8;
        EXPECT(bool(NEGEMMLowpOutputStage::validate(src.info(), bias.info(), dst.info(), os)));
        GEMMLowpOutputStageInfo bad = os;
        bad.gemmlowp_shift          = 32;
        EXPECT(!bool(NEGEMMLowpOutputStage::validate(src.info(), bias.info(), dst.info(), bad)));
        NEGEMMLowpOutputStage stage;
        stage.configure(&src, &bias, &dst, os);
        src.allocator()->allocate(), bias.allocator()->allocate(), dst.allocator()->allocate();
        fill_uniform<int32_t>(src, -20000, 30000, 81), fill_uniform<int32_t>(bias, -3000, 3000, 82);
        stage.run();
        std::vector<uint8_t> want(M * N);
        orc_output_stage_scale(reinterpret_cast<const int32_t *>(src.buffer()), N, reinterpret_cast<const int32_t *>(bias.buffer()),
                               want.data(), N, 0, M, N, &os.gemmlowp_multiplier, &os.gemmlowp_shift, 1, -700,
                               std::numeric_limits<int32_t>::lowest(), std::numeric_limits<int32_t>::max());
        EXPECT(dense_copy<uint8_t>(dst) == want);
    }
    {
        const int M = 40, N = 50, K = 96;
        Tensor    a, b, bias, dst;
        init_tensor(a, TensorShape(K, M), DataType::QASYMM8_SIGNED, QuantizationInfo(1.f, 4));
        init_tensor(b, TensorShape(N, K), DataType::QASYMM8_SIGNED, QuantizationInfo(1.f, -2));
        init_tensor(bias, TensorShape(N), DataType::S32);
        init_tensor(dst, TensorShape(N, M), DataType::QASYMM8_SIGNED, QuantizationInfo(1.f, 0));
        GEMMLowpOutputStageInfo st;
        st.type = GEMMLowpOutputStageType::QUANTIZE_DOWN;
        st.gemmlowp_multiplier = 3, st.gemmlowp_shift = 12, st.gemmlowp_offset = 250;
        st.gemmlowp_min_bound = -100, st.gemmlowp_max_bound = 90, st.output_data_type = DataType::QASYMM8_SIGNED;
        const GEMMInfo gi(false, false, true, 0, false, false, st);
        EXPECT(bool(NEGEMMLowpMatrixMultiplyCore::validate(a.info(), b.info(), bias.info(), dst.info(), gi)));
        NEGEMMLowpMatrixMultiplyCore gemm;
        gemm.configure(&a, &b, &bias, &dst, gi);
        a.allocator()->allocate(), b.allocator()->allocate(), bias.allocator()->allocate(), dst.allocator()->allocate();
        fill_uniform<int8_t>(a, -128, 127, 83), fill_uniform<int8_t>(b, -128, 127, 84), fill_uniform<int32_t>(bias, -2000, 2000, 85);
        const auto A = dense_copy<int8_t>(a), B = dense_copy<int8_t>(b);
        const auto Cb = dense_copy<int32_t>(bias);
        std::vector<int8_t> want(M * N);
        orc_gemmlowp_scale(A.data(), 1, K, B.data(), 1, N, Cb.data(), want.data(), N, 1, M, N, K, 4, -2, &st.gemmlowp_multiplier,
                           &st.gemmlowp_shift, 1, 250, -100, 90);
        gemm.run();
        EXPECT(dense_copy<int8_t>(dst) == want);
        size_t inside = 0;
        for (int8_t v : want)
            inside += (v > -100 && v < 90) ? 1 : 0;
        EXPECT(inside * 4 > want.size());
    }
}

// padded: src / weights / dst carry padding along x (the channels), as the reference's fixture adds it with
// add_padding_x (tests/validation/fixtures/ConvolutionLayerFixture.h:464-469)
// padded == 2: padding along y as well (rows above and below every plane; ITensorInfo::strides_in_bytes()[2] and the
// offset of the first element change, arm_compute/core/ITensorInfo.h:81-334)
static void test_convolution(DataType dt, bool per_channel, int C, const ActivationLayerInfo &act, int padded = 0)
{
    SECTION(padded == 2 ? "NEGEMMConvolutionLayer NHWC, tensors padded along x and y"
            : padded   ? "NEGEMMConvolutionLayer NHWC, tensors padded along x"
                   : per_channel ? "NEGEMMConvolutionLayer NHWC per-channel weights" : "NEGEMMConvolutionLayer NHWC per-tensor weights");
    const bool is_signed = dt == DataType::QASYMM8_SIGNED;
    const int  batch = 2, H = 9, W = 8, OFM = 24, KH = 3, KW = 3;
    const int  in_zp = is_signed ? -1 : 127, out_zp = is_signed ? -5 : 9, w_zp = (per_channel || is_signed) ? 0 : 120;
    std::mt19937 rng(81);
    std::uniform_real_distribution<float> us(0.01f, 1.f);
    std::vector<float> wscale(per_channel ? OFM : 1);
    for (auto &v : wscale)
        v = us(rng) * 0.05f;
    Tensor src, w, bias, dst;
    init_tensor(src, TensorShape(C, W, H, batch), dt, QuantizationInfo(0.02f, in_zp));
    init_tensor(w, TensorShape(C, KW, KH, OFM), per_channel ? DataType::QSYMM8_PER_CHANNEL : dt,
                per_channel ? QuantizationInfo(wscale) : QuantizationInfo(wscale[0], w_zp));
    init_tensor(bias, TensorShape(OFM), DataType::S32);
    init_tensor(dst, TensorShape(), dt, QuantizationInfo(0.9f, out_zp)); // shape filled in by configure()
    for (Tensor *t : {&src, &w, &dst})
        t->info()->set_data_layout(DataLayout::NHWC);
    NEGEMMConvolutionLayer conv;
    conv.configure(&src, &w, &bias, &dst, PadStrideInfo(1, 1, 1, 1), WeightsInfo(), Size2D(1, 1), act);
    EXPECT(dst.info()->dimension(0) == (size_t)OFM && dst.info()->dimension(1) == (size_t)W && dst.info()->dimension(2) == (size_t)H);
    if (padded)
    {
        // after configure and before allocation, like the fixture: PaddingSize(top, right, bottom, left)
        const unsigned y = padded == 2 ? 1 : 0;
        src.info()->extend_padding(PaddingSize(2 * y, 7, y, 3));
        w.info()->extend_padding(PaddingSize(y, 16, 3 * y, 1));
        bias.info()->extend_padding(PaddingSize(0, 2, 0, 5));
        dst.info()->extend_padding(PaddingSize(y, 4, 2 * y, 9));
    }
    src.allocator()->allocate(), w.allocator()->allocate(), bias.allocator()->allocate(), dst.allocator()->allocate();
    if (is_signed)
        fill_uniform<int8_t>(src, -128, 127, 82);
    else
        fill_uniform<uint8_t>(src, 0, 255, 82);
    if (per_channel || is_signed)
        fill_uniform<int8_t>(w, -127, 127, 83);
    else
        fill_uniform<uint8_t>(w, 0, 255, 83);
    fill_uniform<int32_t>(bias, -500, 500, 84);
    conv.run();
    EXPECT(!w.is_used());
    // expected: direct convolution of the oracle with the multipliers the reference's helper derives
    GEMMLowpOutputStageInfo st;
    EXPECT(bool(quantization::calculate_quantized_multipliers(
        QuantizationInfo(0.02f, in_zp), per_channel ? QuantizationInfo(wscale) : QuantizationInfo(wscale[0], w_zp),
        QuantizationInfo(0.9f, out_zp), st)));
    int32_t lo = is_signed ? -128 : 0, hi = is_signed ? 127 : 255;
    if (act.enabled())
        std::tie(lo, hi) = get_quantized_activation_min_max(act, dt, UniformQuantizationInfo(0.9f, out_zp));
    std::vector<uint8_t> want(batch * H * W * OFM);
    const auto src_d = dense_copy<uint8_t>(src), w_d = dense_copy<uint8_t>(w);
    const auto bias_d = dense_copy<int32_t>(bias);
    orc_conv_nhwc_direct(src_d.data(), is_signed, w_d.data(), (per_channel || is_signed) ? 1 : 0, bias_d.data(), want.data(),
                         is_signed, batch, H, W, C, OFM, KH, KW, 1, 1, 1, 1, 1, 1, 1, 1, in_zp, w_zp,
                         st.gemmlowp_multipliers.data(), st.gemmlowp_shifts.data(), per_channel ? OFM : 1, out_zp, lo, hi);
    EXPECT(dense_copy<uint8_t>(dst) == want);
    std::printf("       kernel: %s\n", conv.kernel_name());

    // new output quantization after configure
    dst.info()->set_quantization_info(QuantizationInfo(1.7f, out_zp + 2));
    conv.update_quantization_parameters();
    conv.run();
    EXPECT(bool(quantization::calculate_quantized_multipliers(
        QuantizationInfo(0.02f, in_zp), per_channel ? QuantizationInfo(wscale) : QuantizationInfo(wscale[0], w_zp),
        QuantizationInfo(1.7f, out_zp + 2), st)));
    lo = is_signed ? -128 : 0, hi = is_signed ? 127 : 255;
    if (act.enabled())
        std::tie(lo, hi) = get_quantized_activation_min_max(act, dt, UniformQuantizationInfo(1.7f, out_zp + 2));
    orc_conv_nhwc_direct(src_d.data(), is_signed, w_d.data(), (per_channel || is_signed) ? 1 : 0, bias_d.data(), want.data(),
                         is_signed, batch, H, W, C, OFM, KH, KW, 1, 1, 1, 1, 1, 1, 1, 1, in_zp, w_zp,
                         st.gemmlowp_multipliers.data(), st.gemmlowp_shifts.data(), per_channel ? OFM : 1, out_zp + 2, lo, hi);
    EXPECT(dense_copy<uint8_t>(dst) == want);
}

// NEFullyConnectedLayer against the oracle GEMM on explicitly transposed / re-ordered weights
// (the reference's own FullyConnectedLayer fixture compares against a reference built the same way:
//  tests/validation/fixtures/FullyConnectedLayerFixture.h of the reference)
enum class FcCase
{
    AfterFc,          // src [K, batch], weights [K, N] (one row of num_inputs per output), RELU
    AfterConvNhwc,    // src NHWC [C, W, H, batch], weights trained NCHW (the default): K re-ordered while packing
    AfterConvNchw,    // src NCHW [W, H, C, batch], weights trained NHWC
    WeightsReshaped   // transpose_weights = false: weights [N, K]
};

static void test_fully_connected(DataType dt, FcCase which)
{
    SECTION(which == FcCase::AfterFc         ? "NEFullyConnectedLayer after FC, RELU"
            : which == FcCase::AfterConvNhwc ? "NEFullyConnectedLayer after conv, NHWC input, NCHW-trained weights"
            : which == FcCase::AfterConvNchw ? "NEFullyConnectedLayer after conv, NCHW input, NHWC-trained weights, BOUNDED_RELU"
                                             : "NEFullyConnectedLayer with weights already transposed");
    const bool is_signed = dt == DataType::QASYMM8_SIGNED;
    const int  C = 16, W = 3, H = 5, batch = 7, N = 45;
    const int  K = (which == FcCase::AfterConvNhwc || which == FcCase::AfterConvNchw) ? C * W * H : 200;
    const int  in_zp = is_signed ? -7 : 120, w_zp = is_signed ? 3 : 131, out_zp = is_signed ? -2 : 9;
    const QuantizationInfo iq(0.02f, in_zp), wq(0.011f, w_zp), oq(0.31f, out_zp);
    Tensor src, weights, bias, dst;
    FullyConnectedLayerInfo fc;
    if (which == FcCase::AfterConvNhwc)
    {
        init_tensor(src, TensorShape(C, W, H, batch), dt, iq);
        src.info()->set_data_layout(DataLayout::NHWC);
    }
    else if (which == FcCase::AfterConvNchw)
    {
        init_tensor(src, TensorShape(W, H, C, batch), dt, iq);
        src.info()->set_data_layout(DataLayout::NCHW);
        fc.weights_trained_layout = DataLayout::NHWC;
        fc.activation_info        = ActivationLayerInfo(ActivationLayerInfo::ActivationFunction::BOUNDED_RELU, 60.f);
    }
    else
        init_tensor(src, TensorShape(K, batch), dt, iq);
    if (which == FcCase::WeightsReshaped)
    {
        init_tensor(weights, TensorShape(N, K), dt, wq);
        fc.transpose_weights = false;
    }
    else
        init_tensor(weights, TensorShape(K, N), dt, wq);
    if (which == FcCase::AfterFc)
        fc.activation_info = ActivationLayerInfo(ActivationLayerInfo::ActivationFunction::RELU);
    init_tensor(bias, TensorShape(N), DataType::S32);
    init_tensor(dst, TensorShape(N, batch), dt, oq);
    EXPECT(bool(NEFullyConnectedLayer::validate(src.info(), weights.info(), bias.info(), dst.info(), fc)));
    NEFullyConnectedLayer fcl;
    fcl.configure(&src, &weights, &bias, &dst, fc);
    // the reference's fixture pads every tensor along x after configure()
    // (tests/validation/fixtures/FullyConnectedLayerFixture.h:232-240); an input that has to be flattened stays dense here
    weights.info()->extend_padding(PaddingSize(0, 6, 0, 1)), bias.info()->extend_padding(PaddingSize(0, 2, 0, 2));
    dst.info()->extend_padding(PaddingSize(0, 3, 0, 7));
    if (which == FcCase::AfterFc || which == FcCase::WeightsReshaped)
        src.info()->extend_padding(PaddingSize(0, 4, 0, 12));
    src.allocator()->allocate(), weights.allocator()->allocate(), bias.allocator()->allocate(), dst.allocator()->allocate();
    if (is_signed)
        fill_uniform<int8_t>(src, -128, 127, 21), fill_uniform<int8_t>(weights, -128, 127, 22);
    else
        fill_uniform<uint8_t>(src, 0, 255, 21), fill_uniform<uint8_t>(weights, 0, 255, 22);
    fill_uniform<int32_t>(bias, -3000, 3000, 23);
    const auto A = dense_copy<uint8_t>(src), Wt = dense_copy<uint8_t>(weights);
    const auto Cb = dense_copy<int32_t>(bias);
    // B[k][n] as the GEMM of the reference sees it after transpose + layout conversion
    std::vector<uint8_t> B(static_cast<size_t>(K) * N);
    for (int k = 0; k < K; ++k)
        for (int n = 0; n < N; ++n)
        {
            int ks = k;
            if (which == FcCase::AfterConvNhwc) // flattened NHWC index k = (h*W + w)*C + c takes the NCHW-trained row
                ks = (k % C) * (W * H) + k / C;
            else if (which == FcCase::AfterConvNchw) // flattened NCHW index k = c*H*W + p takes the NHWC-trained row
                ks = (k % (W * H)) * C + k / (W * H);
            B[static_cast<size_t>(k) * N + n] =
                which == FcCase::WeightsReshaped ? Wt[static_cast<size_t>(ks) * N + n] : Wt[static_cast<size_t>(n) * K + ks];
        }
    int32_t mult = 0, shift = 0;
    EXPECT(bool(quantization::calculate_quantized_multiplier(0.02f * 0.011f / 0.31f, &mult, &shift)));
    int32_t lo = is_signed ? -128 : 0, hi = is_signed ? 127 : 255;
    if (which == FcCase::AfterFc)
        lo = out_zp;
    if (which == FcCase::AfterConvNchw)
    {
        lo = out_zp;
        hi = is_signed ? quantize_qasymm8_signed(60.f, oq.uniform()) : quantize_qasymm8(60.f, oq.uniform());
    }
    std::vector<uint8_t> want(static_cast<size_t>(batch) * N);
    orc_gemmlowp_fixedpoint(A.data(), is_signed, K, B.data(), is_signed, N, Cb.data(), want.data(), N, is_signed, batch, N, K,
                            -in_zp, -w_zp, &mult, &shift, 1, out_zp, lo, hi);
    fcl.run();
    EXPECT(dense_copy<uint8_t>(dst) == want);
    EXPECT(!weights.is_used());
    // second run with new input, same packed weights
    if (is_signed)
        fill_uniform<int8_t>(src, -128, 127, 31);
    else
        fill_uniform<uint8_t>(src, 0, 255, 31);
    const auto A2 = dense_copy<uint8_t>(src);
    orc_gemmlowp_fixedpoint(A2.data(), is_signed, K, B.data(), is_signed, N, Cb.data(), want.data(), N, is_signed, batch, N, K,
                            -in_zp, -w_zp, &mult, &shift, 1, out_zp, lo, hi);
    fcl.run();
    EXPECT(dense_copy<uint8_t>(dst) == want);
    size_t inside = 0;
    for (uint8_t v : want)
        inside += (is_signed ? (static_cast<int8_t>(v) > lo && static_cast<int8_t>(v) < hi) : (v > lo && v < hi)) ? 1 : 0;
    EXPECT(inside * 5 > want.size()); // a fair share of the outputs is not clamped: the comparison means something
    std::printf("       kernel: %s\n", fcl.kernel_name());
}

// NEGEMMConv2d: stride 2, asymmetric padding, fused RELU, against the oracle's direct convolution
static void test_gemm_conv2d()
{
    SECTION("NEGEMMConv2d NHWC stride 2, asymmetric padding, RELU");
    const int batch = 3, H = 17, W = 13, C = 32, OFM = 24, KH = 3, KW = 3;
    const int in_zp = 5, out_zp = -9;
    std::vector<float> wscale(OFM);
    for (int i = 0; i < OFM; ++i)
        wscale[i] = 0.002f + 0.0007f * i;
    Tensor src, w, bias, dst;
    init_tensor(src, TensorShape(C, W, H, batch), DataType::QASYMM8_SIGNED, QuantizationInfo(0.03f, in_zp));
    init_tensor(w, TensorShape(C, KW, KH, OFM), DataType::QSYMM8_PER_CHANNEL, QuantizationInfo(wscale));
    init_tensor(bias, TensorShape(OFM), DataType::S32);
    init_tensor(dst, TensorShape(), DataType::QASYMM8_SIGNED, QuantizationInfo(0.6f, out_zp));
    for (Tensor *t : {&src, &w, &dst})
        t->info()->set_data_layout(DataLayout::NHWC);
    const PadStrideInfo       ps(2, 2, 1, 0, 0, 1, DimensionRoundingType::FLOOR); // left 1, right 0, top 0, bottom 1
    const ActivationLayerInfo relu(ActivationLayerInfo::ActivationFunction::RELU);
    const Conv2dInfo          info(ps, Size2D(1, 1), relu, false, 1);
    NEGEMMConv2d conv;
    conv.configure(&src, &w, &bias, &dst, info);
    const int OW = (W + 1 + 0 - 3) / 2 + 1, OH = (H + 0 + 1 - 3) / 2 + 1;
    EXPECT(dst.info()->dimension(0) == (size_t)OFM && dst.info()->dimension(1) == (size_t)OW && dst.info()->dimension(2) == (size_t)OH);
    src.allocator()->allocate(), w.allocator()->allocate(), bias.allocator()->allocate(), dst.allocator()->allocate();
    fill_uniform<int8_t>(src, -128, 127, 91), fill_uniform<int8_t>(w, -127, 127, 92), fill_uniform<int32_t>(bias, -800, 800, 93);
    conv.run();
    GEMMLowpOutputStageInfo st;
    EXPECT(bool(quantization::calculate_quantized_multipliers(QuantizationInfo(0.03f, in_zp), QuantizationInfo(wscale),
                                                              QuantizationInfo(0.6f, out_zp), st)));
    int32_t lo = 0, hi = 0;
    std::tie(lo, hi) = get_quantized_activation_min_max(relu, DataType::QASYMM8_SIGNED, UniformQuantizationInfo(0.6f, out_zp));
    std::vector<uint8_t> want(static_cast<size_t>(batch) * OH * OW * OFM);
    orc_conv_nhwc_direct(src.buffer(), 1, w.buffer(), 1, reinterpret_cast<const int32_t *>(bias.buffer()), want.data(), 1, batch,
                         H, W, C, OFM, KH, KW, 2, 2, 1, 0, 0, 1, 1, 1, in_zp, 0, st.gemmlowp_multipliers.data(),
                         st.gemmlowp_shifts.data(), OFM, out_zp, lo, hi);
    EXPECT(dense_copy<uint8_t>(dst) == want);
    std::printf("       kernel: %s\n", conv.kernel_name());
}

// experimental::op::CpuGEMMLowp: configured on infos, run on an ITensorPack, re-quantised without re-packing B
static void test_stateless_operator()
{
    SECTION("experimental::op::CpuGEMMLowp on an ITensorPack, update_quantization_parameters with negated offsets");
    const int M = 45, N = 70, K = 160;
    const QuantizationInfo aq(0.02f, 7), bq(0.004f, -3), oq(0.05f, 11);
    TensorInfo ai(TensorShape(K, M), 1, DataType::QASYMM8_SIGNED, aq), bi(TensorShape(N, K), 1, DataType::QASYMM8_SIGNED, bq);
    TensorInfo ci(TensorShape(N), 1, DataType::S32), oi(TensorShape(N, M), 1, DataType::QASYMM8_SIGNED, oq);
    GEMMLowpOutputStageInfo st;
    st.type = GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT, st.output_data_type = DataType::QASYMM8_SIGNED;
    st.gemmlowp_offset = 11, st.gemmlowp_min_bound = -128, st.gemmlowp_max_bound = 127;
    EXPECT(bool(quantization::calculate_quantized_multipliers(aq, bq, oq, st)));
    const GEMMInfo gi(false, false, true, 0, false, false, st);
    EXPECT(bool(experimental::op::CpuGEMMLowp::validate(&ai, &bi, &ci, &oi, gi)));
    experimental::op::CpuGEMMLowp op;
    op.configure(&ai, &bi, &ci, &oi, gi);
    EXPECT(op.workspace().empty());
    Tensor a, b, c, dst;
    a.allocator()->init(ai), b.allocator()->init(bi), c.allocator()->init(ci), dst.allocator()->init(oi);
    a.allocator()->allocate(), b.allocator()->allocate(), c.allocator()->allocate(), dst.allocator()->allocate();
    fill_uniform<int8_t>(a, -128, 127, 101), fill_uniform<int8_t>(b, -128, 127, 102), fill_uniform<int32_t>(c, -3000, 3000, 103);
    ITensorPack pack{{ACL_SRC_0, &a}, {ACL_SRC_1, &b}, {ACL_SRC_2, &c}, {ACL_DST, &dst}};
    EXPECT(pack.size() == 4 && pack.get_const_tensor(ACL_SRC_1) == &b && pack.get_tensor(ACL_DST) == &dst);
    op.run(pack);
    const auto A = dense_copy<int8_t>(a), B = dense_copy<int8_t>(b);
    const auto Cb = dense_copy<int32_t>(c);
    std::vector<int8_t> want(M * N);
    orc_gemmlowp_fixedpoint(A.data(), 1, K, B.data(), 1, N, Cb.data(), want.data(), N, 1, M, N, K, 7, -3, &st.gemmlowp_multiplier,
                            &st.gemmlowp_shift, 1, 11, -128, 127);
    EXPECT(dense_copy<int8_t>(dst) == want);
    EXPECT(!b.is_used());
    // a different pack (other activations, other destination), same packed weights
    Tensor a2, dst2;
    a2.allocator()->init(ai), dst2.allocator()->init(oi);
    a2.allocator()->allocate(), dst2.allocator()->allocate();
    fill_uniform<int8_t>(a2, -128, 127, 104);
    ITensorPack pack2{{ACL_SRC_0, &a2}, {ACL_SRC_1, &b}, {ACL_SRC_2, &c}, {ACL_DST, &dst2}};
    op.run(pack2);
    const auto A2 = dense_copy<int8_t>(a2);
    orc_gemmlowp_fixedpoint(A2.data(), 1, K, B.data(), 1, N, Cb.data(), want.data(), N, 1, M, N, K, 7, -3, &st.gemmlowp_multiplier,
                            &st.gemmlowp_shift, 1, 11, -128, 127);
    EXPECT(dense_copy<int8_t>(dst2) == want);
    // new quantization; negated_offsets = true: the offsets handed over are already the added ones, which is how
    // NEGEMMLowpMatrixMultiplyCore and the reference's own fixture call this
    // (tests/validation/fixtures/CpuGEMMLowpFixture.h:109; src/cpu/operators/internal/CpuGemmAssemblyDispatch.cpp:213-215)
    const QuantizationInfo aq2(0.03f, -4), bq2(0.006f, 2), oq2(0.08f, -6);
    op.update_quantization_parameters(aq2, bq2, oq2, DataType::QASYMM8_SIGNED, true, true);
    op.run(pack2);
    GEMMLowpOutputStageInfo st2;
    EXPECT(bool(quantization::calculate_quantized_multipliers(aq2, bq2, oq2, st2)));
    orc_gemmlowp_fixedpoint(A2.data(), 1, K, B.data(), 1, N, Cb.data(), want.data(), N, 1, M, N, K, -4, 2, &st2.gemmlowp_multiplier,
                            &st2.gemmlowp_shift, 1, -6, -128, 127);
    EXPECT(dense_copy<int8_t>(dst2) == want);
    // negated_offsets = false: true zero points (what a CpuMatMul-style caller holds); they are subtracted
    const QuantizationInfo aq3(0.025f, 9), bq3(0.005f, -5), oq3(0.09f, 3);
    op.update_quantization_parameters(aq3, bq3, oq3, DataType::QASYMM8_SIGNED, true, false);
    op.run(pack2);
    GEMMLowpOutputStageInfo st3;
    EXPECT(bool(quantization::calculate_quantized_multipliers(aq3, bq3, oq3, st3)));
    orc_gemmlowp_fixedpoint(A2.data(), 1, K, B.data(), 1, N, Cb.data(), want.data(), N, 1, M, N, K, -9, 5, &st3.gemmlowp_multiplier,
                            &st3.gemmlowp_shift, 1, 3, -128, 127);
    EXPECT(dense_copy<int8_t>(dst2) == want);
}

// The flow of the reference's fixtures for the stateless operators: configure on tensor infos, THEN pad the tensors
// along x, allocate and run (tests/validation/fixtures/CpuGEMMLowpFixture.h:95-124, CpuGemmConv2dFixture.h:300-330).
// The strides the operator walks must be those of the tensors in the pack; dynamic offsets are re-read from them too.
static void test_stateless_operators_padded_after_configure()
{
    SECTION("experimental::op::CpuGEMMLowp / CpuGemmConv2d: x-padding added after configure, dynamic offsets");
    {
        const int M = 37, N = 50, K = 96;
        const QuantizationInfo aq(0.02f, 5, true), bq(0.004f, -2, true), oq(0.06f, 9);
        TensorInfo ai(TensorShape(K, M), 1, DataType::QASYMM8_SIGNED, aq), bi(TensorShape(N, K), 1, DataType::QASYMM8_SIGNED, bq);
        TensorInfo ci(TensorShape(N), 1, DataType::S32), oi(TensorShape(N, M), 1, DataType::QASYMM8_SIGNED, oq);
        GEMMLowpOutputStageInfo st;
        st.type = GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT, st.output_data_type = DataType::QASYMM8_SIGNED;
        st.gemmlowp_offset = 9, st.gemmlowp_min_bound = -128, st.gemmlowp_max_bound = 127;
        EXPECT(bool(quantization::calculate_quantized_multipliers(aq, bq, oq, st)));
        experimental::op::CpuGEMMLowp op;
        op.configure(&ai, &bi, &ci, &oi, GEMMInfo(false, false, true, 0, false, false, st));
        Tensor a, b, c, dst;
        a.allocator()->init(ai), b.allocator()->init(bi), c.allocator()->init(ci), dst.allocator()->init(oi);
        a.info()->extend_padding(PaddingSize(0, 7, 0, 4)), b.info()->extend_padding(PaddingSize(0, 13, 0, 1));
        dst.info()->extend_padding(PaddingSize(0, 2, 0, 16));
        a.allocator()->allocate(), b.allocator()->allocate(), c.allocator()->allocate(), dst.allocator()->allocate();
        EXPECT(a.info()->strides_in_bytes()[1] != (size_t)K && dst.info()->strides_in_bytes()[1] != (size_t)N);
        fill_uniform<int8_t>(a, -128, 127, 201), fill_uniform<int8_t>(b, -128, 127, 202), fill_uniform<int32_t>(c, -2000, 2000, 203);
        std::memset(dst.buffer(), 0x55, dst.info()->total_size());
        ITensorPack pack{{ACL_SRC_0, &a}, {ACL_SRC_1, &b}, {ACL_SRC_2, &c}, {ACL_DST, &dst}};
        op.run(pack);
        const auto A = dense_copy<int8_t>(a), B = dense_copy<int8_t>(b);
        const auto Cb = dense_copy<int32_t>(c);
        std::vector<int8_t> want(M * N);
        orc_gemmlowp_fixedpoint(A.data(), 1, K, B.data(), 1, N, Cb.data(), want.data(), N, 1, M, N, K, 5, -2, &st.gemmlowp_multiplier,
                                &st.gemmlowp_shift, 1, 9, -128, 127);
        EXPECT(dense_copy<int8_t>(dst) == want);
        // the destination's padding bytes are not touched
        bool pad_ok = true;
        const size_t ld = dst.info()->strides_in_bytes()[1], off0 = dst.info()->offset_first_element_in_bytes();
        for (size_t i = 0; i < dst.info()->total_size(); ++i)
        {
            const bool inside = i >= off0 && (i - off0) % ld < (size_t)N && (i - off0) / ld < (size_t)M;
            pad_ok = pad_ok && (inside || dst.buffer()[i] == 0x55);
        }
        EXPECT(pad_ok);
        // dynamic quantization info: new offsets on the pack's tensors are picked up by the next run
        a.info()->set_quantization_info(QuantizationInfo(0.02f, -11, true));
        b.info()->set_quantization_info(QuantizationInfo(0.004f, 6, true));
        op.run(pack);
        orc_gemmlowp_fixedpoint(A.data(), 1, K, B.data(), 1, N, Cb.data(), want.data(), N, 1, M, N, K, -11, 6, &st.gemmlowp_multiplier,
                                &st.gemmlowp_shift, 1, 9, -128, 127);
        EXPECT(dense_copy<int8_t>(dst) == want);
    }
    {
        const int batch = 2, H = 9, W = 8, C = 16, OFM = 24, KH = 3, KW = 3, in_zp = -4, out_zp = 6;
        const QuantizationInfo iq(0.03f, in_zp), wq(0.01f, 0), oq(0.9f, out_zp);
        TensorInfo si(TensorShape(C, W, H, batch), 1, DataType::QASYMM8_SIGNED, iq), wi(TensorShape(C, KW, KH, OFM), 1, DataType::QASYMM8_SIGNED, wq);
        TensorInfo bi(TensorShape(OFM), 1, DataType::S32), di(TensorShape(), 1, DataType::QASYMM8_SIGNED, oq);
        si.set_data_layout(DataLayout::NHWC), wi.set_data_layout(DataLayout::NHWC), di.set_data_layout(DataLayout::NHWC);
        const PadStrideInfo psi(1, 1, 1, 1);
        experimental::op::CpuGemmConv2d op;
        op.configure(&si, &wi, &bi, &di, psi);
        Tensor src, w, bias, dst;
        src.allocator()->init(si), w.allocator()->init(wi), bias.allocator()->init(bi), dst.allocator()->init(di);
        src.info()->extend_padding(PaddingSize(0, 5, 0, 3)), w.info()->extend_padding(PaddingSize(0, 16, 0, 2));
        dst.info()->extend_padding(PaddingSize(0, 8, 0, 1));
        src.allocator()->allocate(), w.allocator()->allocate(), bias.allocator()->allocate(), dst.allocator()->allocate();
        fill_uniform<int8_t>(src, -128, 127, 211), fill_uniform<int8_t>(w, -127, 127, 212), fill_uniform<int32_t>(bias, -500, 500, 213);
        ITensorPack pack{{ACL_SRC_0, &src}, {ACL_SRC_1, &w}, {ACL_SRC_2, &bias}, {ACL_DST, &dst}};
        op.run(pack);
        const auto S = dense_copy<int8_t>(src), Wd = dense_copy<int8_t>(w);
        const auto Bv = dense_copy<int32_t>(bias);
        GEMMLowpOutputStageInfo st;
        EXPECT(bool(quantization::calculate_quantized_multipliers(iq, wq, oq, st)));
        std::vector<int8_t> want(batch * H * W * OFM);
        orc_conv_nhwc_direct(S.data(), 1, Wd.data(), 1, Bv.data(), want.data(), 1, batch, H, W, C, OFM, KH, KW, 1, 1, 1, 1, 1, 1, 1, 1,
                             in_zp, 0, &st.gemmlowp_multiplier, &st.gemmlowp_shift, 1, out_zp, -128, 127);
        EXPECT(dense_copy<int8_t>(dst) == want);
    }
}

// the channel-planar layout through NEGEMMConvolutionLayer and the stateless operator on an ITensorPack: both against
// the oracle's direct convolution of the same data in NHWC order
static void test_convolution_nchw_and_stateless()
{
    SECTION("NEGEMMConvolutionLayer NCHW; experimental::op::CpuGemmConv2d on an ITensorPack");
    const int batch = 2, H = 10, W = 7, C = 16, OFM = 20, KH = 3, KW = 2, in_zp = 3, out_zp = -4;
    std::mt19937 rng(140);
    std::uniform_int_distribution<int> u8(-128, 127), uw(-127, 127), ub(-400, 400);
    std::uniform_real_distribution<float> us(0.0005f, 0.05f);
    std::vector<int8_t> src_nhwc(batch * H * W * C), w_nhwc(OFM * KH * KW * C);
    std::vector<int32_t> biasv(OFM);
    std::vector<float> wscale(OFM);
    for (auto &v : src_nhwc) v = (int8_t)u8(rng);
    for (auto &v : w_nhwc) v = (int8_t)uw(rng);
    for (auto &v : biasv) v = ub(rng);
    for (auto &v : wscale) v = us(rng);
    const PadStrideInfo psi(2, 1, 1, 0, 2, 1, DimensionRoundingType::FLOOR); // stride (2,1), pad l1 r0 t2 b1
    int OH = 0, OW = 0;
    orc_conv_out_dims(H, W, KH, KW, 2, 1, 1, 2, 0, 1, 1, 1, &OH, &OW);
    const QuantizationInfo iq(0.02f, in_zp), wq(wscale), oq(0.7f, out_zp);
    GEMMLowpOutputStageInfo st;
    EXPECT(bool(quantization::calculate_quantized_multipliers(iq, wq, oq, st)));
    std::vector<int8_t> want(batch * OH * OW * OFM);
    auto expect = [&](const GEMMLowpOutputStageInfo &stage, int ozp)
    {
        orc_conv_nhwc_direct(src_nhwc.data(), 1, w_nhwc.data(), 1, biasv.data(), want.data(), 1, batch, H, W, C, OFM, KH, KW, 2,
                             1, 1, 2, 0, 1, 1, 1, in_zp, 0, stage.gemmlowp_multipliers.data(), stage.gemmlowp_shifts.data(), OFM,
                             ozp, -128, 127);
    };
    expect(st, out_zp);
    {
        Tensor src, w, bias, dst;
        init_tensor(src, TensorShape(W, H, C, batch), DataType::QASYMM8_SIGNED, iq);
        init_tensor(w, TensorShape(KW, KH, C, OFM), DataType::QSYMM8_PER_CHANNEL, wq);
        init_tensor(bias, TensorShape(OFM), DataType::S32);
        init_tensor(dst, TensorShape(), DataType::QASYMM8_SIGNED, oq);
        for (Tensor *t : {&src, &w, &dst})
            t->info()->set_data_layout(DataLayout::NCHW);
        NEGEMMConvolutionLayer conv;
        conv.configure(&src, &w, &bias, &dst, psi);
        EXPECT(dst.info()->dimension(0) == (size_t)OW && dst.info()->dimension(1) == (size_t)OH &&
               dst.info()->dimension(2) == (size_t)OFM && dst.info()->dimension(3) == (size_t)batch);
        src.allocator()->allocate(), w.allocator()->allocate(), bias.allocator()->allocate(), dst.allocator()->allocate();
        for (int n = 0; n < batch; ++n)
            for (int c = 0; c < C; ++c)
                for (int y = 0; y < H; ++y)
                    for (int x = 0; x < W; ++x)
                        reinterpret_cast<int8_t *>(src.buffer())[((n * C + c) * H + y) * W + x] = src_nhwc[((n * H + y) * W + x) * C + c];
        for (int o = 0; o < OFM; ++o)
            for (int c = 0; c < C; ++c)
                for (int t = 0; t < KH * KW; ++t)
                    reinterpret_cast<int8_t *>(w.buffer())[(o * C + c) * KH * KW + t] = w_nhwc[(o * KH * KW + t) * C + c];
        std::memcpy(bias.buffer(), biasv.data(), sizeof(int32_t) * OFM);
        conv.run();
        bool ok = true;
        for (int n = 0; n < batch; ++n)
            for (int o = 0; o < OFM; ++o)
                for (int p = 0; p < OH * OW; ++p)
                    ok = ok && reinterpret_cast<const int8_t *>(dst.buffer())[(n * OFM + o) * OH * OW + p] == want[(n * OH * OW + p) * OFM + o];
        EXPECT(ok);
        std::printf("       kernel: %s\n", conv.kernel_name());
    }
    {
        TensorInfo si(TensorShape(C, W, H, batch), 1, DataType::QASYMM8_SIGNED, iq), wi(TensorShape(C, KW, KH, OFM), 1, DataType::QSYMM8_PER_CHANNEL, wq);
        TensorInfo bi(TensorShape(OFM), 1, DataType::S32), di(TensorShape(), 1, DataType::QASYMM8_SIGNED, oq);
        si.set_data_layout(DataLayout::NHWC), wi.set_data_layout(DataLayout::NHWC), di.set_data_layout(DataLayout::NHWC);
        experimental::op::CpuGemmConv2d op;
        op.configure(&si, &wi, &bi, &di, psi);
        EXPECT(di.dimension(0) == (size_t)OFM && di.dimension(1) == (size_t)OW && di.dimension(2) == (size_t)OH);
        EXPECT(bool(experimental::op::CpuGemmConv2d::validate(&si, &wi, &bi, &di, psi)));
        EXPECT(op.workspace().empty());
        Tensor src, w, bias, dst;
        src.allocator()->init(si), w.allocator()->init(wi), bias.allocator()->init(bi), dst.allocator()->init(di);
        src.allocator()->allocate(), w.allocator()->allocate(), bias.allocator()->allocate(), dst.allocator()->allocate();
        std::memcpy(src.buffer(), src_nhwc.data(), src_nhwc.size());
        std::memcpy(w.buffer(), w_nhwc.data(), w_nhwc.size());
        std::memcpy(bias.buffer(), biasv.data(), sizeof(int32_t) * OFM);
        ITensorPack pack{{ACL_SRC_0, &src}, {ACL_SRC_1, &w}, {ACL_SRC_2, &bias}, {ACL_DST, &dst}};
        op.run(pack);
        EXPECT(dense_copy<int8_t>(dst) == want);
        EXPECT(!w.is_used());
        // the output's quantization changes after configure: re-derived from the pack's tensors, weights stay packed
        const QuantizationInfo oq2(1.3f, out_zp + 7);
        dst.info()->set_quantization_info(oq2);
        op.update_quantization_parameters(pack);
        op.run(pack);
        GEMMLowpOutputStageInfo st2;
        EXPECT(bool(quantization::calculate_quantized_multipliers(iq, wq, oq2, st2)));
        expect(st2, out_zp + 7);
        EXPECT(dense_copy<int8_t>(dst) == want);
    }
}

// QASYMM8_SIGNED convolution with an F32 destination and a fused RELU (the dequantising path of CpuGemmConv2d)
static void test_convolution_f32_destination()
{
    SECTION("NEGEMMConvolutionLayer QASYMM8_SIGNED -> F32 with F32 bias and RELU");
    const int batch = 2, H = 8, W = 9, C = 16, OFM = 12, KH = 3, KW = 3, in_zp = 5, w_zp = -2;
    Tensor src, w, bias, dst;
    init_tensor(src, TensorShape(C, W, H, batch), DataType::QASYMM8_SIGNED, QuantizationInfo(0.02f, in_zp));
    init_tensor(w, TensorShape(C, KW, KH, OFM), DataType::QASYMM8_SIGNED, QuantizationInfo(0.005f, w_zp));
    init_tensor(bias, TensorShape(OFM), DataType::F32);
    init_tensor(dst, TensorShape(OFM, W, H, batch), DataType::F32);
    for (Tensor *t : {&src, &w, &dst})
        t->info()->set_data_layout(DataLayout::NHWC);
    const ActivationLayerInfo relu(ActivationLayerInfo::ActivationFunction::RELU);
    EXPECT(bool(NEGEMMConvolutionLayer::validate(src.info(), w.info(), bias.info(), dst.info(), PadStrideInfo(1, 1, 1, 1), WeightsInfo(),
                                                 Size2D(1, 1), relu)));
    NEGEMMConvolutionLayer conv;
    conv.configure(&src, &w, &bias, &dst, PadStrideInfo(1, 1, 1, 1), WeightsInfo(), Size2D(1, 1), relu);
    src.allocator()->allocate(), w.allocator()->allocate(), bias.allocator()->allocate(), dst.allocator()->allocate();
    fill_uniform<int8_t>(src, -128, 127, 151), fill_uniform<int8_t>(w, -127, 127, 152);
    std::mt19937                    rng(153);
    std::normal_distribution<float> nd(0.f, 2.f);
    for (int j = 0; j < OFM; ++j)
        reinterpret_cast<float *>(bias.buffer())[j] = nd(rng);
    conv.run();
    const int K = KH * KW * C, M = batch * H * W;
    std::vector<uint8_t> cols((size_t)M * K);
    orc_im2col_nhwc(src.buffer(), cols.data(), batch, H, W, C, KH, KW, 1, 1, 1, 1, 1, 1, 1, 1, (uint8_t)in_zp);
    std::vector<int8_t> Bm((size_t)K * OFM); // weights [OFM][K] -> B [K][OFM]
    for (int o = 0; o < OFM; ++o)
        for (int k = 0; k < K; ++k)
            Bm[(size_t)k * OFM + o] = reinterpret_cast<const int8_t *>(w.buffer())[(size_t)o * K + k];
    std::vector<float> want((size_t)M * OFM);
    orc_gemmlowp_f32(cols.data(), 1, K, Bm.data(), 1, OFM, reinterpret_cast<const float *>(bias.buffer()), want.data(), OFM, M, OFM,
                     K, -in_zp, -w_zp, 0.02f * 0.005f, 0.f, INFINITY, 0, 1);
    EXPECT(dense_copy<float>(dst) == want);
    std::printf("       kernel: %s\n", conv.kernel_name());
    // an F32 destination with per-channel or unsigned weights has no kernel
    Tensor wpc;
    init_tensor(wpc, TensorShape(C, KW, KH, OFM), DataType::QSYMM8_PER_CHANNEL, QuantizationInfo(std::vector<float>(OFM, 0.01f)));
    wpc.info()->set_data_layout(DataLayout::NHWC);
    EXPECT(!bool(NEGEMMConvolutionLayer::validate(src.info(), wpc.info(), bias.info(), dst.info(), PadStrideInfo(1, 1, 1, 1))));
}

static void test_error_paths()
{
    SECTION("configure() throws on invalid input; run() before configure() throws");
    Tensor a, b, dst;
    init_tensor(a, TensorShape(20U, 13U), DataType::QASYMM8, QuantizationInfo(1.f, 0));
    init_tensor(b, TensorShape(33U, 21U), DataType::QASYMM8, QuantizationInfo(1.f, 0));
    init_tensor(dst, TensorShape(33U, 13U), DataType::S32);
    NEGEMMLowpMatrixMultiplyCore gemm;
    bool threw = false;
    try
    {
        gemm.configure(&a, &b, nullptr, &dst);
    }
    catch (const std::runtime_error &)
    {
        threw = true;
    }
    EXPECT(threw);
    threw = false;
    try
    {
        gemm.run();
    }
    catch (const std::runtime_error &)
    {
        threw = true;
    }
    EXPECT(threw);
}

// Every case has a name so that the runner (tests/test_host_api.py) can start each one in a process of its own and
// report it on its own: --list-cpu / --list-gpu print the names, --case NAME runs one, --cpu / --gpu run a whole group.
struct Case
{
    const char *name;
    bool        gpu;
    void (*fn)();
};

static const Case g_cases[] = {
    {"tensor_info", false, [] { test_tensor_info(); }},
    {"quant_helpers", false, [] { test_quant_helpers(); }},
    {"validate_tables", false, [] { test_validate_tables(); }},
    {"fully_connected_validate", false, [] { test_fully_connected_validate(); }},
    {"gemm_conv2d_validate", false, [] { test_gemm_conv2d_validate(); }},
    {"error_paths", false, [] { test_error_paths(); }},
    {"gemmlowp_fused_u8_host", true, [] { test_gemmlowp_fused_u8(false); }},
    {"gemmlowp_fused_u8_device", true, [] { test_gemmlowp_fused_u8(true); }},
    {"gemmlowp_s32_batched", true, [] { test_gemmlowp_s32_batched(); }},
    {"reference_small_datasets", true, [] { test_reference_small_datasets(); }},
    {"gemmlowp_accumulate_and_3d", true, [] { test_gemmlowp_accumulate_and_3d(); }},
    {"gemmlowp_dynamic_qinfo", true, [] { test_gemmlowp_dynamic_qinfo(); }},
    {"gemmlowp_per_channel_and_update", true, [] { test_gemmlowp_per_channel_and_update(); }},
    {"gemmlowp_f32", true, [] { test_gemmlowp_f32(); }},
    {"output_stage", true, [] { test_output_stage(); }},
    {"quantize_down_scale", true, [] { test_quantize_down_scale(); }},
    {"convolution_s8_per_channel_64", true, [] { test_convolution(DataType::QASYMM8_SIGNED, true, 64, ActivationLayerInfo()); }},
    {"convolution_s8_relu_16", true,
     [] { test_convolution(DataType::QASYMM8_SIGNED, false, 16, ActivationLayerInfo(ActivationLayerInfo::ActivationFunction::RELU)); }},
    {"convolution_u8_6", true, [] { test_convolution(DataType::QASYMM8, false, 6, ActivationLayerInfo()); }},
    {"convolution_u8_per_channel_bounded_relu_32", true,
     [] {
         test_convolution(DataType::QASYMM8, true, 32, ActivationLayerInfo(ActivationLayerInfo::ActivationFunction::BOUNDED_RELU, 20.f));
     }},
    {"convolution_s8_per_channel_32_variant1", true, [] { test_convolution(DataType::QASYMM8_SIGNED, true, 32, ActivationLayerInfo(), 1); }},
    {"convolution_u8_relu_6_variant1", true,
     [] { test_convolution(DataType::QASYMM8, false, 6, ActivationLayerInfo(ActivationLayerInfo::ActivationFunction::RELU), 1); }},
    {"convolution_s8_per_channel_16_variant2", true, [] { test_convolution(DataType::QASYMM8_SIGNED, true, 16, ActivationLayerInfo(), 2); }},
    {"convolution_u8_6_variant2", true, [] { test_convolution(DataType::QASYMM8, false, 6, ActivationLayerInfo(), 2); }},
    {"gemm_conv2d", true, [] { test_gemm_conv2d(); }},
    {"stateless_operator", true, [] { test_stateless_operator(); }},
    {"stateless_operators_padded_after_configure", true, [] { test_stateless_operators_padded_after_configure(); }},
    {"convolution_nchw_and_stateless", true, [] { test_convolution_nchw_and_stateless(); }},
    {"convolution_f32_destination", true, [] { test_convolution_f32_destination(); }},
    {"fully_connected_s8_after_fc", true, [] { test_fully_connected(DataType::QASYMM8_SIGNED, FcCase::AfterFc); }},
    {"fully_connected_u8_after_fc", true, [] { test_fully_connected(DataType::QASYMM8, FcCase::AfterFc); }},
    {"fully_connected_s8_after_conv_nhwc", true, [] { test_fully_connected(DataType::QASYMM8_SIGNED, FcCase::AfterConvNhwc); }},
    {"fully_connected_u8_after_conv_nchw", true, [] { test_fully_connected(DataType::QASYMM8, FcCase::AfterConvNchw); }},
    {"fully_connected_s8_weights_reshaped", true, [] { test_fully_connected(DataType::QASYMM8_SIGNED, FcCase::WeightsReshaped); }},
};

int main(int argc, char **argv)
{
    const std::string mode = argc > 1 ? argv[1] : "--cpu";
    const std::string want = argc > 2 ? argv[2] : "";
    if (mode == "--list-cpu" || mode == "--list-gpu")
    {
        for (const Case &c : g_cases)
            if (c.gpu == (mode == "--list-gpu"))
                std::printf("%s\n", c.name);
        return 0;
    }
    if (mode != "--cpu" && mode != "--gpu" && mode != "--case")
    {
        std::printf("usage: %s --cpu | --gpu | --case NAME | --list-cpu | --list-gpu\n", argv[0]);
        return 2;
    }
    int ran = 0;
    try
    {
        for (const Case &c : g_cases)
            if (mode == "--case" ? want == c.name : c.gpu == (mode == "--gpu"))
            {
                c.fn();
                ++ran;
            }
    }
    catch (const std::exception &e)
    {
        std::printf("FAILED: unexpected exception: %s\n", e.what());
        ++g_failures;
    }
    if (ran == 0)
    {
        std::printf("no such case: %s\n", want.c_str());
        return 2;
    }
    std::printf("%d checks, %d failures\n", g_checks, g_failures);
    return g_failures == 0 ? 0 : 1;
}
