// NEGEMMLowpMatrixMultiplyCore, NEGEMMLowpOutputStage, NEGEMMConvolutionLayer and NEFullyConnectedLayer on top of the
// MI355X C ABI
// (include/mi355_gemmlowp.h). The classes keep the reference's calling conventions: non-owning tensor pointers captured
// at configure() and dereferenced at run(), buffers that may be allocated after configure(), validate() that returns a
// Status and never throws, configure() that throws std::runtime_error on invalid input, synchronous run().
#include "arm_compute/core/utils/quantization/AsymmHelpers.h"
#include "arm_compute/runtime/NEON/NEFunctions.h"
#include "arm_compute/runtime/experimental/operators/CpuGEMMLowp.h"
#include "arm_compute/runtime/experimental/operators/CpuGemmConv2d.h"
#include "mi355_gemmlowp.h"

#include <cmath>
#include <limits>
#include <set>
#include <string>
#include <vector>

namespace arm_compute
{
namespace
{
int to_mi355(DataType dt)
{
    switch (dt)
    {
        case DataType::QASYMM8:
        case DataType::U8:
            return MI355_U8;
        case DataType::QASYMM8_SIGNED:
        case DataType::QSYMM8:
        case DataType::QSYMM8_PER_CHANNEL:
        case DataType::S8:
            return MI355_S8;
        case DataType::QSYMM16:
            return MI355_S16;
        case DataType::S32:
            return MI355_S32;
        case DataType::F32:
            return MI355_F32;
        case DataType::F16:
            return MI355_F16;
        default:
            return -1;
    }
}

bool is_one_of(DataType dt, std::initializer_list<DataType> list)
{
    for (DataType d : list)
        if (d == dt)
            return true;
    return false;
}

void check_abi(int rc, const char *what)
{
    if (rc != 0)
        throw std::runtime_error(std::string(what) + ": " + mi355_last_error());
}

uint8_t *first_element(const ITensor *t)
{
    return t->buffer() + t->info()->offset_first_element_in_bytes();
}

mi355_requant make_requant(const GEMMLowpOutputStageInfo &s)
{
    mi355_requant rq{};
    rq.per_channel   = s.is_quantized_per_channel ? 1 : 0;
    rq.multiplier    = s.gemmlowp_multiplier;
    rq.shift         = s.gemmlowp_shift;
    rq.result_offset = s.gemmlowp_offset;
    rq.min_bound     = s.gemmlowp_min_bound;
    rq.max_bound     = s.gemmlowp_max_bound;
    rq.stage         = s.type == GEMMLowpOutputStageType::QUANTIZE_DOWN ? MI355_STAGE_SCALE : MI355_STAGE_FIXEDPOINT;
    if (s.type == GEMMLowpOutputStageType::QUANTIZE_DOWN && s.gemmlowp_min_bound == s.gemmlowp_max_bound)
    {
        // equal bounds mean "no bounded activation": only the saturation to the output type remains
        // (src/cpu/kernels/CpuGemmLowpQuantizeDownInt32ScaleKernel.cpp:299-300, tests/validation/reference/GEMMLowp.cpp:95-99)
        rq.min_bound = std::numeric_limits<int32_t>::lowest();
        rq.max_bound = std::numeric_limits<int32_t>::max();
    }
    return rq;
}

// rows of the matrix must be contiguous along x, everything above dimension 1 is one batch index
Status check_matrix_layout(const ITensorInfo *t, const char *name)
{
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(t->strides_in_bytes()[0] != t->element_size(),
                                    std::string(name) + ": elements of a row must be contiguous");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(t->strides_in_bytes()[1] % t->element_size() != 0,
                                    std::string(name) + ": row stride must be a whole number of elements");
    return Status{};
}

// Clamp bounds of an 8-bit output stage must lie inside the destination type's range (a bounded activation) or cover it
// (saturation only). With one end inside and one outside, the reference's own paths disagree: the stand-alone kernel
// narrows the bound to 8 bits (src/cpu/kernels/CpuGemmLowpOffsetContributionOutputStageKernel.cpp:502-503), the assembly
// path clamps in int32 and keeps the low byte (src/core/NEON/kernels/arm_gemm/quantized.cpp:36-46,254-261).
Status check_8bit_bounds(const GEMMLowpOutputStageInfo &stage, DataType dt)
{
    if (dt != DataType::QASYMM8 && dt != DataType::QASYMM8_SIGNED)
        return Status{};
    if (stage.type == GEMMLowpOutputStageType::QUANTIZE_DOWN && stage.gemmlowp_min_bound == stage.gemmlowp_max_bound)
        return Status{}; // "no bounded activation" for that stage
    const int32_t lo = dt == DataType::QASYMM8 ? 0 : -128, hi = dt == DataType::QASYMM8 ? 255 : 127;
    const bool    covers = stage.gemmlowp_min_bound <= lo && stage.gemmlowp_max_bound >= hi;
    const bool    inside = stage.gemmlowp_min_bound >= lo && stage.gemmlowp_max_bound <= hi;
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(!covers && !inside, "Output stage bounds partly outside the output type's range");
    return Status{};
}

const std::set<ActivationLayerInfo::ActivationFunction> fusable_acts = {
    ActivationLayerInfo::ActivationFunction::RELU, ActivationLayerInfo::ActivationFunction::BOUNDED_RELU,
    ActivationLayerInfo::ActivationFunction::LU_BOUNDED_RELU};

// Row and batch strides of the three matrices as the tensor infos give them now; an info that is not at hand (nullptr)
// leaves its fields as they are
void read_gemm_strides(const ITensorInfo *ai, const ITensorInfo *bi, const ITensorInfo *oi, const GEMMInfo &gemm_info,
                       mi355_gemm_desc &d)
{
    const bool a3d = gemm_info.reinterpret_input_as_3d();
    if (ai != nullptr)
    {
        d.lda            = ai->strides_in_bytes()[1];
        d.a_batch_stride = ai->strides_in_bytes()[a3d ? 3 : 2];
        // [K, W, H, batch] read as W*H rows: planes of W rows, strides_in_bytes()[2] apart (more than W rows when the
        // tensor is padded along y)
        d.a_plane_rows   = a3d ? static_cast<int32_t>(ai->dimension(1)) : 0;
        d.a_plane_stride = a3d ? static_cast<int64_t>(ai->strides_in_bytes()[2]) : 0;
    }
    if (bi != nullptr)
    {
        d.ldb            = bi->strides_in_bytes()[1];
        d.b_batch_stride = bi->num_dimensions() > 2 ? bi->strides_in_bytes()[2] : 0;
    }
    if (oi != nullptr)
    {
        d.ldd = oi->strides_in_bytes()[1] / oi->element_size();
        if (gemm_info.depth_output_gemm3d() != 0)
        {
            // [N, W, H, batch]: planes of W rows
            d.d_batch_stride = oi->strides_in_bytes()[3] / oi->element_size();
            d.d_plane_rows   = static_cast<int32_t>(oi->dimension(1));
            d.d_plane_stride = static_cast<int64_t>(oi->strides_in_bytes()[2] / oi->element_size());
        }
        else
        {
            d.d_batch_stride = oi->strides_in_bytes()[2] / oi->element_size();
            d.d_plane_rows = 0, d.d_plane_stride = 0;
        }
    }
}

// Padding may be added to a tensor between configure() and the first run (the reference's fixtures do exactly that:
// tests/validation/fixtures/GEMMLowpFixture.h:300-304, CpuGEMMLowpFixture.h:117) and the reference reads strides when
// it runs. Re-reads them from the infos at hand and tells the handle when they differ from what it holds. Once B is
// packed its strides no longer matter.
void sync_gemm_strides(const ITensorInfo *ai, const ITensorInfo *bi, const ITensorInfo *oi, const GEMMInfo &info,
                       mi355_gemm_desc &d, mi355_gemm_handle *handle, bool b_is_packed, const char *where)
{
    mi355_gemm_desc now = d;
    read_gemm_strides(ai, b_is_packed ? nullptr : bi, oi, info, now);
    if (now.lda == d.lda && now.ldb == d.ldb && now.ldd == d.ldd && now.a_batch_stride == d.a_batch_stride &&
        now.b_batch_stride == d.b_batch_stride && now.d_batch_stride == d.d_batch_stride &&
        now.a_plane_stride == d.a_plane_stride && now.d_plane_stride == d.d_plane_stride)
        return;
    check_abi(mi355_gemmlowp_set_strides_3d(handle, now.lda, now.ldb, now.ldd, now.a_batch_stride, now.b_batch_stride,
                                            now.d_batch_stride, now.a_plane_stride, now.d_plane_stride),
              where);
    d = now;
}

// the C-ABI descriptor of a GEMMLowp on these tensor infos (shapes are x-fastest: a = [K, M, batch], b = [N, K(, batch)],
// output = [N, M, batch]); per-channel multipliers / shifts are cut to exactly N entries
void fill_gemm_desc(const ITensorInfo *ai, const ITensorInfo *bi, const ITensorInfo *oi, const GEMMInfo &gemm_info,
                    mi355_gemm_desc &d, std::vector<int32_t> &multipliers, std::vector<int32_t> &shifts)
{
    multipliers.clear(), shifts.clear();
    const GEMMLowpOutputStageInfo stage = gemm_info.gemmlowp_output_stage();
    d = mi355_gemm_desc{};
    d.K                = static_cast<int32_t>(ai->dimension(0));
    d.N                = static_cast<int32_t>(bi->dimension(0));
    const bool a3d     = gemm_info.reinterpret_input_as_3d(); // [K, W, H, batch]: M = W * H
    d.M                = static_cast<int32_t>(a3d ? ai->dimension(1) * ai->dimension(2) : ai->dimension(1));
    d.batch            = static_cast<int32_t>(ai->tensor_shape().total_size_upper(a3d ? 3 : 2));
    d.a_dtype          = to_mi355(ai->data_type());
    d.b_dtype          = to_mi355(bi->data_type());
    d.dst_dtype        = to_mi355(oi->data_type());
    read_gemm_strides(ai, bi, oi, gemm_info, d);
    d.a_offset = ai->quantization_info().uniform().offset;
    d.b_offset = is_data_type_quantized_per_channel(bi->data_type()) ? 0 : bi->quantization_info().uniform().offset;
    d.act_min  = -std::numeric_limits<float>::infinity();
    d.act_max  = std::numeric_limits<float>::infinity();
    d.scale    = 1.f;
    d.path     = MI355_PATH_AUTO;
    d.flags    = gemm_info.accumulate() ? MI355_GEMM_ACCUMULATE : 0;
    if (stage.type == GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT || stage.type == GEMMLowpOutputStageType::QUANTIZE_DOWN)
    {
        d.epilogue = MI355_EPI_FIXEDPOINT;
        d.requant  = make_requant(stage);
        if (stage.is_quantized_per_channel)
        {
            multipliers.assign(stage.gemmlowp_multipliers.begin(), stage.gemmlowp_multipliers.begin() + d.N);
            shifts.assign(stage.gemmlowp_shifts.begin(), stage.gemmlowp_shifts.begin() + d.N);
        }
    }
    else if (oi->data_type() == DataType::F32 || oi->data_type() == DataType::F16)
    {
        d.epilogue = MI355_EPI_F32;
        d.scale    = ai->quantization_info().uniform().scale * bi->quantization_info().uniform().scale;
        const ActivationLayerInfo act = gemm_info.activation_info();
        if (act.enabled())
        {
            switch (act.activation())
            {
                case ActivationLayerInfo::ActivationFunction::RELU:
                    d.act_min = 0.f;
                    break;
                case ActivationLayerInfo::ActivationFunction::BOUNDED_RELU:
                    d.act_min = 0.f, d.act_max = act.a();
                    break;
                case ActivationLayerInfo::ActivationFunction::LU_BOUNDED_RELU:
                    d.act_min = act.b(), d.act_max = act.a();
                    break;
                default:
                    ARM_COMPUTE_ERROR("Only RELU, BOUNDED_RELU and LU_BOUNDED_RELU can be fused");
            }
            // the reference's assembly GEMM takes these three when the lower bound is 0 and clamps inside its merge
            // step, before the offset term is added; the CpuActivation post-op then clamps again
            // (src/core/utils/AssemblyUtils.cpp:32-62, src/cpu/operators/CpuGemmLowpMatrixMultiplyCore.cpp:326-332)
            if (act.b() == 0.f)
                d.flags |= MI355_GEMM_ACT_TWICE;
        }
    }
    else
        d.epilogue = MI355_EPI_S32;
}
} // namespace

// =====================================================================================================================
// NEGEMMLowpMatrixMultiplyCore
// =====================================================================================================================
struct NEGEMMLowpMatrixMultiplyCore::Impl
{
    const ITensor      *a{nullptr}, *b{nullptr}, *c{nullptr};
    ITensor            *output{nullptr};
    GEMMInfo            info{};
    mi355_gemm_desc     desc{};
    mi355_gemm_handle  *handle{nullptr};
    bool                is_prepared{false};
    bool                b_constant{true};
    std::vector<int32_t> multipliers, shifts; // per-channel, exactly N entries

    ~Impl()
    {
        if (handle)
            mi355_gemmlowp_destroy(handle);
    }
};

NEGEMMLowpMatrixMultiplyCore::NEGEMMLowpMatrixMultiplyCore(std::shared_ptr<IMemoryManager> memory_manager,
                                                           IWeightsManager                *weights_manager)
    : _impl(std::make_unique<Impl>())
{
    // device workspace is owned by the handle; a host memory manager has nothing to manage here
    ARM_COMPUTE_UNUSED(memory_manager, weights_manager);
}
NEGEMMLowpMatrixMultiplyCore::~NEGEMMLowpMatrixMultiplyCore() = default;

// Accept / reject rules of src/cpu/operators/CpuGemmLowpMatrixMultiplyCore.cpp:362-645 and of the kernels it validates
// (CpuGemmLowpOffsetContributionOutputStageKernel.cpp:829-905, CpuGemmLowpMatrixMultiplyKernel.cpp:690-692).
Status NEGEMMLowpMatrixMultiplyCore::validate(const ITensorInfo *a, const ITensorInfo *b, const ITensorInfo *c,
                                              const ITensorInfo *output, const GEMMInfo &gemm_info)
{
    ARM_COMPUTE_RETURN_ERROR_ON_NULLPTR(a, b, output);
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(a->is_dynamic() || b->is_dynamic() || output->is_dynamic() ||
                                        (c != nullptr && c->is_dynamic()),
                                    "Dynamic tensor shapes are not supported");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(!is_one_of(a->data_type(), {DataType::QASYMM8, DataType::QASYMM8_SIGNED}) ||
                                        a->num_channels() != 1,
                                    "Matrix A must be QASYMM8 or QASYMM8_SIGNED");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(!is_one_of(b->data_type(), {DataType::QASYMM8, DataType::QASYMM8_SIGNED,
                                                                DataType::QSYMM8, DataType::QSYMM8_PER_CHANNEL}) ||
                                        b->num_channels() != 1,
                                    "Matrix B must be QASYMM8, QASYMM8_SIGNED, QSYMM8 or QSYMM8_PER_CHANNEL");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(!is_one_of(output->data_type(), {DataType::S32, DataType::QASYMM8,
                                                                     DataType::QASYMM8_SIGNED, DataType::F32, DataType::F16}),
                                    "Output must be S32, QASYMM8, QASYMM8_SIGNED, F32 or F16");
    // the half leg of the dequantising GEMM is exercised by the reference with signed operands only
    // (tests/validation/NEON/GEMMLowp.cpp:598-607)
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(output->data_type() == DataType::F16 &&
                                        (a->data_type() != DataType::QASYMM8_SIGNED || b->data_type() != DataType::QASYMM8_SIGNED),
                                    "An F16 output needs QASYMM8_SIGNED operands");
    const GEMMLowpOutputStageInfo stage = gemm_info.gemmlowp_output_stage();
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(c != nullptr && output->data_type() != DataType::F32 &&
                                        stage.type == GEMMLowpOutputStageType::NONE,
                                    "Bias addition not supported in NEGEMMLowpMatrixMultiplyCore for output S32");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(
        a->dimension(0) != b->dimension(1),
        "The product AB is defined only if the number of columns in A is equal to the number of rows in B");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(gemm_info.is_a_reshaped(), "Matrix A already reshaped is not supported");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(gemm_info.is_b_reshaped(), "Matrix B already reshaped is not supported");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(gemm_info.pretranspose_A(), "Matrix A already pretransposed is not supported");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(gemm_info.pretranspose_B(), "Matrix B already pretransposed is not supported");
    // signed A with unsigned B has no kernel in the reference (CpuGemmLowpMatrixMultiplyKernel.cpp:690-692)
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(a->data_type() == DataType::QASYMM8_SIGNED && b->data_type() == DataType::QASYMM8,
                                    "QASYMM8_SIGNED lhs with QASYMM8 rhs is not supported");
    if (gemm_info.accumulate())
    {
        ARM_COMPUTE_RETURN_ERROR_ON_MSG(stage.type != GEMMLowpOutputStageType::NONE,
                                        "Accumulation is not supported for output QASYMM8/QASYMM8_SIGNED");
    }

    // shapes
    ARM_COMPUTE_RETURN_ERROR_ON(b->dimension(0) != output->dimension(0));
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(gemm_info.reinterpret_input_as_3d() && gemm_info.depth_output_gemm3d() == 0,
                                    "reinterpret_input_as_3d is only built together with a 3D output");
    if (gemm_info.depth_output_gemm3d() != 0)
    {
        if (gemm_info.reinterpret_input_as_3d())
        {
            ARM_COMPUTE_RETURN_ERROR_ON(a->dimension(1) != output->dimension(1));
            ARM_COMPUTE_RETURN_ERROR_ON(a->dimension(2) != output->dimension(2));
            ARM_COMPUTE_RETURN_ERROR_ON(a->tensor_shape().total_size_upper(3) != output->tensor_shape().total_size_upper(3));
        }
        else
            ARM_COMPUTE_RETURN_ERROR_ON(a->dimension(1) != output->dimension(1) * output->dimension(2));
    }
    else
    {
        ARM_COMPUTE_RETURN_ERROR_ON(a->dimension(1) != output->dimension(1));
        ARM_COMPUTE_RETURN_ERROR_ON(a->tensor_shape().total_size_upper(2) != output->tensor_shape().total_size_upper(2));
    }
    const size_t a_batch_dim = gemm_info.reinterpret_input_as_3d() ? 3 : 2;
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(b->num_dimensions() > 2 && b->tensor_shape().total_size_upper(2) !=
                                                                   a->tensor_shape().total_size_upper(a_batch_dim),
                                    "Batched B must have as many matrices as A");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(a->num_dimensions() > a_batch_dim + 1 || b->num_dimensions() > 3,
                                    "More than one batch dimension is not supported");
    ARM_COMPUTE_RETURN_ON_ERROR(check_matrix_layout(a, "a"));
    ARM_COMPUTE_RETURN_ON_ERROR(check_matrix_layout(b, "b"));
    ARM_COMPUTE_RETURN_ON_ERROR(check_matrix_layout(output, "output"));

    // output stage
    switch (stage.type)
    {
        case GEMMLowpOutputStageType::NONE:
            ARM_COMPUTE_RETURN_ERROR_ON_MSG(!is_one_of(output->data_type(), {DataType::S32, DataType::F32, DataType::F16}),
                                            "A quantized output needs an output stage");
            if (c != nullptr)
            {
                ARM_COMPUTE_RETURN_ERROR_ON(c->data_type() != DataType::F32);
                ARM_COMPUTE_RETURN_ERROR_ON(c->num_dimensions() > 1 || c->dimension(0) != b->dimension(0));
            }
            break;
        case GEMMLowpOutputStageType::QUANTIZE_DOWN:
            if (stage.is_quantized_per_channel)
            {
                for (size_t j = 0; j < b->dimension(0) && j < stage.gemmlowp_shifts.size(); ++j)
                    ARM_COMPUTE_RETURN_ERROR_ON_MSG(stage.gemmlowp_shifts[j] < 0 || stage.gemmlowp_shifts[j] > 31,
                                                    "QUANTIZE_DOWN needs shifts in [0, 31]");
            }
            else
                ARM_COMPUTE_RETURN_ERROR_ON_MSG(stage.gemmlowp_shift < 0 || stage.gemmlowp_shift > 31,
                                                "QUANTIZE_DOWN needs a shift in [0, 31]");
            // the same rules otherwise (CpuGemmLowpOffsetContributionOutputStageKernel.cpp:829-905)
            [[fallthrough]];
        case GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT:
            ARM_COMPUTE_RETURN_ERROR_ON_MSG(!is_one_of(output->data_type(), {DataType::QASYMM8, DataType::QASYMM8_SIGNED}),
                                            "The integer output stages write QASYMM8 or QASYMM8_SIGNED");
            ARM_COMPUTE_RETURN_ERROR_ON(stage.gemmlowp_min_bound > stage.gemmlowp_max_bound);
            ARM_COMPUTE_RETURN_ON_ERROR(check_8bit_bounds(stage, output->data_type()));
            if (c != nullptr)
            {
                ARM_COMPUTE_RETURN_ERROR_ON(c->data_type() != DataType::S32);
                ARM_COMPUTE_RETURN_ERROR_ON(c->num_dimensions() > 1 || c->dimension(0) != b->dimension(0));
            }
            if (stage.is_quantized_per_channel)
            {
                ARM_COMPUTE_RETURN_ERROR_ON_MSG(stage.gemmlowp_multipliers.size() < b->dimension(0) ||
                                                    stage.gemmlowp_shifts.size() < b->dimension(0),
                                                "Per-channel multipliers / shifts shorter than the number of columns");
                // CpuGemmLowpOffsetContributionOutputStageKernel.cpp:832-836
                ARM_COMPUTE_RETURN_ERROR_ON_MSG(b->quantization_info().uniform().offset != 0 &&
                                                    !is_data_type_quantized_per_channel(b->data_type()),
                                                "Per-channel requantization needs a zero rhs offset");
            }
            break;
        default:
            ARM_COMPUTE_RETURN_ERROR_MSG("Unsupported output stage");
    }
    return Status{};
}

void NEGEMMLowpMatrixMultiplyCore::configure(const ITensor *a, const ITensor *b, const ITensor *c, ITensor *output,
                                             const GEMMInfo &gemm_info)
{
    ARM_COMPUTE_ERROR_ON_NULLPTR(a, b, output);
    ARM_COMPUTE_ERROR_THROW_ON(
        validate(a->info(), b->info(), c != nullptr ? c->info() : nullptr, output->info(), gemm_info));
    Impl &s = *_impl;
    if (s.handle)
    {
        mi355_gemmlowp_destroy(s.handle);
        s.handle = nullptr;
    }
    s.a = a, s.b = b, s.c = c, s.output = output, s.info = gemm_info;
    s.is_prepared = false;
    s.b_constant  = gemm_info.reshape_b_only_on_first_run(); // NEGEMMLowpMatrixMultiplyCore.cpp:77-81 of the reference

    fill_gemm_desc(a->info(), b->info(), output->info(), gemm_info, s.desc, s.multipliers, s.shifts);
    mi355_gemm_desc &d = s.desc;
    check_abi(mi355_gemmlowp_create(&d, &s.handle), "NEGEMMLowpMatrixMultiplyCore::configure");
}

void NEGEMMLowpMatrixMultiplyCore::prepare()
{
    Impl &s = *_impl;
    ARM_COMPUTE_ERROR_ON_MSG(s.handle == nullptr, "NEGEMMLowpMatrixMultiplyCore::prepare() before configure()");
    ARM_COMPUTE_ERROR_THROW_ON(check_matrix_layout(s.a->info(), "a"));
    ARM_COMPUTE_ERROR_THROW_ON(check_matrix_layout(s.output->info(), "output"));
    sync_gemm_strides(s.a->info(), s.b->info(), s.output->info(), s.info, s.desc, s.handle, s.is_prepared,
                      "NEGEMMLowpMatrixMultiplyCore::prepare");
    if (s.is_prepared)
        return;
    ARM_COMPUTE_ERROR_THROW_ON(check_matrix_layout(s.b->info(), "b"));
    ARM_COMPUTE_ERROR_ON_MSG(s.b->buffer() == nullptr, "matrix B has no memory");
    const int32_t *bias = nullptr;
    if (s.desc.epilogue == MI355_EPI_FIXEDPOINT && s.c != nullptr)
    {
        ARM_COMPUTE_ERROR_ON_MSG(s.c->buffer() == nullptr, "bias has no memory");
        bias = reinterpret_cast<const int32_t *>(first_element(s.c));
    }
    check_abi(mi355_gemmlowp_prepare(s.handle, first_element(s.b), bias,
                                     s.multipliers.empty() ? nullptr : s.multipliers.data(),
                                     s.shifts.empty() ? nullptr : s.shifts.data(), nullptr),
              "NEGEMMLowpMatrixMultiplyCore::prepare");
    if (s.b_constant)
    {
        s.b->mark_as_unused(); // the packed copy lives on the device from here on
        s.is_prepared = true;
    }
}

void NEGEMMLowpMatrixMultiplyCore::update_quantization_parameters()
{
    Impl &s = *_impl;
    ARM_COMPUTE_ERROR_ON_MSG(s.handle == nullptr, "update_quantization_parameters() before configure()");
    const QuantizationInfo iq = s.a->info()->quantization_info();
    const QuantizationInfo wq = s.b->info()->quantization_info();
    const QuantizationInfo oq = (s.output->info()->total_size() == 0) ? iq : s.output->info()->quantization_info();
    const DataType         dt = s.a->info()->data_type();
    int32_t                lo = get_min_max(dt).first, hi = get_min_max(dt).second;
    const UniformQuantizationInfo uo = oq.uniform();
    if (fusable_acts.count(s.info.activation_info().activation()) != 0)
        std::tie(lo, hi) = get_quantized_activation_min_max(s.info.activation_info(), dt, uo);
    s.desc.a_offset = iq.uniform().offset;
    s.desc.b_offset = is_data_type_quantized_per_channel(s.b->info()->data_type()) ? 0 : wq.uniform().offset;
    if (s.desc.epilogue == MI355_EPI_FIXEDPOINT)
    {
        ARM_COMPUTE_ERROR_ON_MSG(s.desc.requant.per_channel, "per-channel output stages cannot be updated in place");
        GEMMLowpOutputStageInfo out;
        out.type                     = GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT;
        out.gemmlowp_offset          = uo.offset;
        out.gemmlowp_min_bound       = lo;
        out.gemmlowp_max_bound       = hi;
        out.is_quantized_per_channel = false;
        out.output_data_type         = s.output->info()->data_type();
        ARM_COMPUTE_ERROR_THROW_ON(quantization::calculate_quantized_multipliers(iq, wq, oq, out));
        s.desc.requant = make_requant(out);
        s.info.set_gemmlowp_output_stage(out);
    }
    if (s.desc.epilogue == MI355_EPI_F32)
        s.desc.scale = iq.uniform().scale * wq.uniform().scale;
    check_abi(mi355_gemmlowp_update_quant(s.handle, s.desc.a_offset, s.desc.b_offset,
                                          s.desc.epilogue == MI355_EPI_FIXEDPOINT ? &s.desc.requant : nullptr,
                                          s.desc.scale, nullptr),
              "NEGEMMLowpMatrixMultiplyCore::update_quantization_parameters");
}

void NEGEMMLowpMatrixMultiplyCore::run()
{
    Impl &s = *_impl;
    ARM_COMPUTE_ERROR_ON_MSG(s.handle == nullptr, "NEGEMMLowpMatrixMultiplyCore::run() before configure()");
    ARM_COMPUTE_ERROR_ON_MSG(s.a->buffer() == nullptr || s.output->buffer() == nullptr, "tensor without memory");
    // dynamic quantization: offsets are re-read on every run (CpuGemmLowpMatrixMultiplyCore.cpp:668-674 of the reference)
    if (s.a->info()->quantization_info().is_dynamic() || s.b->info()->quantization_info().is_dynamic())
    {
        const int32_t ao = s.a->info()->quantization_info().uniform().offset;
        const int32_t bo = is_data_type_quantized_per_channel(s.b->info()->data_type())
                               ? 0
                               : s.b->info()->quantization_info().uniform().offset;
        // ... and so is the dequantisation scale of the F32 path (:776-784)
        const float sc = s.desc.epilogue == MI355_EPI_F32 ? s.a->info()->quantization_info().uniform().scale *
                                                                s.b->info()->quantization_info().uniform().scale
                                                          : s.desc.scale;
        if (ao != s.desc.a_offset || bo != s.desc.b_offset || sc != s.desc.scale)
        {
            s.desc.a_offset = ao, s.desc.b_offset = bo, s.desc.scale = sc;
            check_abi(mi355_gemmlowp_update_quant(s.handle, ao, bo, nullptr, s.desc.scale, nullptr),
                      "NEGEMMLowpMatrixMultiplyCore::run");
        }
    }
    prepare();
    const float *bias_f32 = nullptr;
    if (s.desc.epilogue == MI355_EPI_F32 && s.c != nullptr)
        bias_f32 = reinterpret_cast<const float *>(first_element(s.c));
    check_abi(mi355_gemmlowp_run(s.handle, first_element(s.a), bias_f32, first_element(s.output), nullptr),
              "NEGEMMLowpMatrixMultiplyCore::run");
}

const char *NEGEMMLowpMatrixMultiplyCore::kernel_name() const
{
    return _impl->handle ? mi355_gemmlowp_kernel_name(_impl->handle) : "";
}

// =====================================================================================================================
// NEGEMMLowpOutputStage
// =====================================================================================================================
struct NEGEMMLowpOutputStage::Impl
{
    const ITensor          *src{nullptr}, *bias{nullptr};
    ITensor                *dst{nullptr};
    mi355_output_stage_desc desc{};
    bool                    configured{false};
};

NEGEMMLowpOutputStage::NEGEMMLowpOutputStage() : _impl(std::make_unique<Impl>()) {}
NEGEMMLowpOutputStage::~NEGEMMLowpOutputStage() = default;

// src/cpu/operators/CpuGemmLowpOutputStage.cpp:114-161 and
// src/cpu/kernels/CpuGemmLowpQuantizeDownInt32ToInt8ScaleByFixedPointKernel.cpp:52-76 of the reference
Status NEGEMMLowpOutputStage::validate(const ITensorInfo *input, const ITensorInfo *bias, const ITensorInfo *output,
                                       const GEMMLowpOutputStageInfo &info)
{
    ARM_COMPUTE_RETURN_ERROR_ON_NULLPTR(input, output);
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(output->data_type() == DataType::UNKNOWN,
                                    "NEGEMMLowpOutputStage cannot be used with UNKNOWN output data type.");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(!is_one_of(output->data_type(), {DataType::QASYMM8, DataType::QASYMM8_SIGNED,
                                                                     DataType::QSYMM16}),
                                    "Output must be QASYMM8, QASYMM8_SIGNED or QSYMM16");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(info.type != GEMMLowpOutputStageType::QUANTIZE_DOWN &&
                                        info.type != GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT,
                                    "Unsupported output stage type");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(info.type == GEMMLowpOutputStageType::QUANTIZE_DOWN &&
                                        (info.gemmlowp_shift < 0 || info.gemmlowp_shift > 31),
                                    "QUANTIZE_DOWN needs a shift in [0, 31]");
    // QSYMM16 only has a fixed-point kernel (src/cpu/operators/CpuGemmLowpOutputStage.cpp:73-80,91-107)
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(output->data_type() == DataType::QSYMM16 &&
                                        info.type != GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT,
                                    "Unsupported output data type.");
    if (output->data_type() == DataType::QSYMM16)
    {
        // the int16 kernel narrows the bounds with a plain cast: accept what survives it
        const bool whole = info.gemmlowp_min_bound <= -32768 && info.gemmlowp_max_bound >= 32767;
        ARM_COMPUTE_RETURN_ERROR_ON_MSG(!whole && (info.gemmlowp_min_bound < -32768 || info.gemmlowp_max_bound > 32767),
                                        "QSYMM16 bounds partly outside the int16 range");
    }
    ARM_COMPUTE_RETURN_ERROR_ON(input->data_type() != DataType::S32 || input->num_channels() != 1);
    ARM_COMPUTE_RETURN_ERROR_ON(info.gemmlowp_min_bound > info.gemmlowp_max_bound);
    ARM_COMPUTE_RETURN_ON_ERROR(check_8bit_bounds(info, output->data_type()));
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(info.is_quantized_per_channel, "The stand-alone output stage is per-tensor");
    if (bias != nullptr)
    {
        ARM_COMPUTE_RETURN_ERROR_ON(bias->data_type() != input->data_type());
        ARM_COMPUTE_RETURN_ERROR_ON(bias->num_dimensions() > 1);
        ARM_COMPUTE_RETURN_ERROR_ON(input->dimension(0) != bias->dimension(0));
    }
    if (output->total_size() != 0)
        ARM_COMPUTE_RETURN_ERROR_ON(output->tensor_shape() != input->tensor_shape());
    ARM_COMPUTE_RETURN_ON_ERROR(check_matrix_layout(input, "input"));
    ARM_COMPUTE_RETURN_ON_ERROR(check_matrix_layout(output, "output"));
    return Status{};
}

void NEGEMMLowpOutputStage::configure(const ITensor *input, const ITensor *bias, ITensor *output,
                                      const GEMMLowpOutputStageInfo &info)
{
    ARM_COMPUTE_ERROR_ON_NULLPTR(input, output);
    // like the reference, an uninitialised output takes the input's shape and the requested data type
    if (output->info()->total_size() == 0 && output->info()->is_resizable())
    {
        output->info()->set_tensor_shape(input->info()->tensor_shape());
        output->info()->set_num_channels(1);
        output->info()->set_data_type(info.output_data_type);
    }
    ARM_COMPUTE_ERROR_THROW_ON(validate(input->info(), bias != nullptr ? bias->info() : nullptr, output->info(), info));
    Impl &s = *_impl;
    s.src = input, s.bias = bias, s.dst = output;
    const ITensorInfo *ii = input->info(), *oi = output->info();
    // every dimension above x is a row as long as rows are evenly spaced
    const size_t rows = ii->tensor_shape().total_size_upper(1);
    for (size_t i = 2; i < ii->num_dimensions(); ++i)
    {
        ARM_COMPUTE_ERROR_ON_MSG(ii->strides_in_bytes()[i] != ii->dimension(i - 1) * ii->strides_in_bytes()[i - 1] ||
                                     oi->strides_in_bytes()[i] != oi->dimension(i - 1) * oi->strides_in_bytes()[i - 1],
                                 "padding between planes is not supported by the stand-alone output stage");
    }
    s.desc           = mi355_output_stage_desc{};
    s.desc.M         = static_cast<int32_t>(rows);
    s.desc.N         = static_cast<int32_t>(ii->dimension(0));
    s.desc.ld_src    = ii->strides_in_bytes()[1] / ii->element_size();
    s.desc.ld_dst    = oi->strides_in_bytes()[1] / oi->element_size();
    s.desc.dst_dtype = to_mi355(oi->data_type());
    if (oi->data_type() == DataType::QSYMM16)
    {
        // no result offset on this path: the reference's int16 kernel is not given one (CpuGemmLowpOutputStage.cpp:73-80)
        s.desc.requant            = mi355_requant{};
        s.desc.requant.multiplier = info.gemmlowp_multiplier;
        s.desc.requant.shift      = info.gemmlowp_shift;
        s.desc.requant.min_bound  = info.gemmlowp_min_bound;
        s.desc.requant.max_bound  = info.gemmlowp_max_bound;
        s.desc.requant.stage      = MI355_STAGE_FIXEDPOINT;
    }
    else
        s.desc.requant = make_requant(info);
    s.configured = true;
}

void NEGEMMLowpOutputStage::run()
{
    Impl &s = *_impl;
    ARM_COMPUTE_ERROR_ON_MSG(!s.configured, "NEGEMMLowpOutputStage::run() before configure()");
    ARM_COMPUTE_ERROR_ON_MSG(s.src->buffer() == nullptr || s.dst->buffer() == nullptr, "tensor without memory");
    // strides are read when running, as the reference does: its fixtures pad the tensors after configure()
    s.desc.ld_src = s.src->info()->strides_in_bytes()[1] / s.src->info()->element_size();
    s.desc.ld_dst = s.dst->info()->strides_in_bytes()[1] / s.dst->info()->element_size();
    check_abi(mi355_output_stage_run(&s.desc, reinterpret_cast<const int32_t *>(first_element(s.src)),
                                     s.bias ? reinterpret_cast<const int32_t *>(first_element(s.bias)) : nullptr,
                                     first_element(s.dst), nullptr),
              "NEGEMMLowpOutputStage::run");
}

// =====================================================================================================================
// NEGEMMConvolutionLayer
// =====================================================================================================================
struct NEGEMMConvolutionLayer::Impl
{
    const ITensor       *src{nullptr}, *weights{nullptr}, *biases{nullptr};
    ITensor             *dst{nullptr};
    ActivationLayerInfo  act{};
    mi355_conv_desc      desc{};
    mi355_conv_handle   *handle{nullptr};
    bool                 is_prepared{false};
    std::vector<int32_t> multipliers, shifts;

    ~Impl()
    {
        if (handle)
            mi355_conv_destroy(handle);
    }
};

NEGEMMConvolutionLayer::NEGEMMConvolutionLayer(const std::shared_ptr<IMemoryManager> &memory_manager,
                                               IWeightsManager                       *weights_manager)
    : _impl(std::make_unique<Impl>())
{
    ARM_COMPUTE_UNUSED(memory_manager, weights_manager);
}
NEGEMMConvolutionLayer::~NEGEMMConvolutionLayer() = default;

namespace
{
// positions of width / height / channels in a 4D tensor shape (get_data_layout_dimension_index of the reference)
struct ConvDims
{
    size_t w, h, c;
    explicit ConvDims(DataLayout l) : w(l == DataLayout::NHWC ? 1 : 0), h(l == DataLayout::NHWC ? 2 : 1), c(l == DataLayout::NHWC ? 0 : 2) {}
};

// requantisation of a quantized convolution, as CpuGemmConv2d::configure_mm derives it
// (src/cpu/operators/CpuGemmConv2d.cpp:266-313 of the reference)
Status conv_output_stage(const ITensorInfo *src, const ITensorInfo *weights, const ITensorInfo *dst,
                         const ActivationLayerInfo &act, GEMMLowpOutputStageInfo &out)
{
    const QuantizationInfo iq = src->quantization_info();
    const QuantizationInfo wq = weights->quantization_info();
    const QuantizationInfo oq = (dst->total_size() == 0) ? iq : dst->quantization_info();
    const DataType         dt = src->data_type();
    int32_t                lo = get_min_max(dt).first, hi = get_min_max(dt).second;
    if (fusable_acts.count(act.activation()) != 0)
        std::tie(lo, hi) = get_quantized_activation_min_max(act, dt, oq.uniform());
    out.type                     = GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT;
    out.gemmlowp_offset          = oq.uniform().offset;
    out.gemmlowp_min_bound       = lo;
    out.gemmlowp_max_bound       = hi;
    out.is_quantized_per_channel = weights->data_type() == DataType::QSYMM8_PER_CHANNEL;
    return quantization::calculate_quantized_multipliers(iq, wq, oq, out);
}
} // namespace

// src/cpu/operators/CpuGemmConv2d.cpp:697-856 of the reference, restricted to what this library builds
Status NEGEMMConvolutionLayer::validate(const ITensorInfo *input, const ITensorInfo *weights, const ITensorInfo *biases,
                                        const ITensorInfo *output, const PadStrideInfo &conv_info,
                                        const WeightsInfo &weights_info, const Size2D &dilation,
                                        const ActivationLayerInfo &act_info, bool enable_fast_math,
                                        unsigned int num_groups)
{
    ARM_COMPUTE_UNUSED(enable_fast_math);
    ARM_COMPUTE_RETURN_ERROR_ON_NULLPTR(input, weights, output);
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(weights_info.are_reshaped(), "Weights already reshaped are not supported!");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(is_one_of(input->data_type(), {DataType::BFLOAT16, DataType::F16, DataType::F32}),
                                    "Floating-point convolution is not built in this library");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(!is_one_of(input->data_type(), {DataType::QASYMM8, DataType::QASYMM8_SIGNED}),
                                    "Input must be QASYMM8 or QASYMM8_SIGNED");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(!is_one_of(weights->data_type(), {DataType::QASYMM8, DataType::QASYMM8_SIGNED,
                                                                      DataType::QSYMM8_PER_CHANNEL}),
                                    "Weights must be QASYMM8, QASYMM8_SIGNED or QSYMM8_PER_CHANNEL");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(input->data_layout() != weights->data_layout(), "Mismatching data layouts");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(num_groups > 1, "Grouping (num_groups != 1) is not supported");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(input->data_layout() != DataLayout::NHWC && input->data_layout() != DataLayout::NCHW,
                                    "Unknown data layout");
    const ConvDims dm(input->data_layout());
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(input->data_type() == DataType::QASYMM8_SIGNED && weights->data_type() == DataType::QASYMM8,
                                    "QASYMM8_SIGNED input with QASYMM8 weights is not supported");
    ARM_COMPUTE_RETURN_ERROR_ON(weights->dimension(dm.c) != input->dimension(dm.c)); // channels
    ARM_COMPUTE_RETURN_ERROR_ON(weights->num_dimensions() > 4);
    ARM_COMPUTE_RETURN_ERROR_ON(input->num_dimensions() > 4);
    // QASYMM8_SIGNED in, F32 out: the dequantising path (src/cpu/operators/CpuGemmConv2d.cpp:156-159,763-770 of the reference)
    const bool dequant = input->data_type() == DataType::QASYMM8_SIGNED && output->data_type() == DataType::F32;
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(output->data_type() != input->data_type() && !dequant,
                                    "Output must have the input's data type, or be F32 for a QASYMM8_SIGNED input");
    if (dequant)
    {
        ARM_COMPUTE_RETURN_ERROR_ON_MSG(weights->data_type() != DataType::QASYMM8_SIGNED,
                                        "The F32 destination needs QASYMM8_SIGNED weights");
    }
    if (biases != nullptr)
    {
        ARM_COMPUTE_RETURN_ERROR_ON(biases->data_type() != (dequant ? DataType::F32 : DataType::S32));
        ARM_COMPUTE_RETURN_ERROR_ON(biases->dimension(0) != weights->dimension(3));
        ARM_COMPUTE_RETURN_ERROR_ON(biases->num_dimensions() > 1);
    }
    if (weights->data_type() == DataType::QSYMM8_PER_CHANNEL)
        ARM_COMPUTE_RETURN_ERROR_ON_MSG(weights->quantization_info().scale().size() != weights->dimension(3),
                                        "One weight scale per output channel is required");
    if (act_info.enabled())
        ARM_COMPUTE_RETURN_ERROR_ON_MSG(fusable_acts.count(act_info.activation()) == 0,
                                        "Only RELU, BOUNDED_RELU and LU_BOUNDED_RELU can be fused");
    unsigned int conv_w = 0, conv_h = 0;
    std::tie(conv_w, conv_h) = scaled_dimensions(static_cast<int>(input->dimension(dm.w)), static_cast<int>(input->dimension(dm.h)),
                                                 static_cast<int>(weights->dimension(dm.w)), static_cast<int>(weights->dimension(dm.h)),
                                                 conv_info, dilation);
    if (output->total_size() != 0)
    {
        ARM_COMPUTE_RETURN_ERROR_ON_MSG(output->data_layout() != input->data_layout(), "Mismatching data layouts");
        ARM_COMPUTE_RETURN_ERROR_ON(output->dimension(dm.c) != weights->dimension(3));
        ARM_COMPUTE_RETURN_ERROR_ON(output->dimension(dm.w) != conv_w || output->dimension(dm.h) != conv_h);
        ARM_COMPUTE_RETURN_ERROR_ON(output->dimension(3) != input->dimension(3));
    }
    // Padding in any dimension of either layout (what the reference's fixtures add is add_padding_x,
    // tests/validation/Helpers.cpp:335-357; its kernels read ITensorInfo::strides_in_bytes()) travels as the byte
    // strides of dimensions 1 to 3; the elements of dimension 0 must be contiguous
    for (const ITensorInfo *t : {input, weights, output})
    {
        if (t->total_size() == 0)
            continue;
        ARM_COMPUTE_RETURN_ERROR_ON_MSG(t->strides_in_bytes()[0] != t->element_size(),
                                        "The elements of dimension 0 must be contiguous");
    }
    if (!dequant)
    {
        GEMMLowpOutputStageInfo stage;
        ARM_COMPUTE_RETURN_ON_ERROR(conv_output_stage(input, weights, output, act_info, stage));
    }
    return Status{};
}

Status NEGEMMConvolutionLayer::has_opt_impl(WeightFormat &expected_weight_format, const ITensorInfo *src,
                                            const ITensorInfo *weights, const ITensorInfo *biases,
                                            const ITensorInfo *dst, const PadStrideInfo &conv_info,
                                            const WeightsInfo &weights_info, const Size2D &dilation,
                                            const ActivationLayerInfo &act_info, bool enable_fast_math)
{
    // no fixed-format weights in this library: the packed layout is private to the device workspace
    expected_weight_format = WeightFormat::UNSPECIFIED;
    ARM_COMPUTE_RETURN_ON_ERROR(validate(src, weights, biases, dst, conv_info, weights_info, dilation, act_info,
                                         enable_fast_math, 1));
    ARM_COMPUTE_RETURN_ERROR_MSG("No fixed-format kernel available");
}

namespace
{
// an uninitialised output takes the convolved shape, the input's type, layout and (unless it already has one) quantization
void conv_auto_init_output(const ITensorInfo *ii, const ITensorInfo *wi, ITensorInfo *oi, const PadStrideInfo &conv_info,
                           const Size2D &dilation)
{
    if (oi->total_size() != 0 || !oi->is_resizable())
        return;
    const ConvDims dm(ii->data_layout());
    unsigned int   conv_w = 0, conv_h = 0;
    std::tie(conv_w, conv_h) = scaled_dimensions(static_cast<int>(ii->dimension(dm.w)), static_cast<int>(ii->dimension(dm.h)),
                                                 static_cast<int>(wi->dimension(dm.w)), static_cast<int>(wi->dimension(dm.h)),
                                                 conv_info, dilation);
    const QuantizationInfo keep = oi->quantization_info();
    TensorShape            shape;
    shape.set(dm.c, wi->dimension(3)), shape.set(dm.w, conv_w), shape.set(dm.h, conv_h), shape.set(3, ii->dimension(3));
    oi->set_tensor_shape(shape);
    oi->set_num_channels(1);
    oi->set_data_type(ii->data_type());
    oi->set_data_layout(ii->data_layout());
    oi->set_quantization_info(keep.empty() ? ii->quantization_info() : keep);
}

// strides_in_bytes()[1..3] of the three tensors of a convolution (zeros, i.e. "dense", for an info that is not at hand)
struct ConvStrides
{
    int64_t src[3] = {0, 0, 0}, weights[3] = {0, 0, 0}, dst[3] = {0, 0, 0};
};
ConvStrides conv_strides_of(const ITensorInfo *ii, const ITensorInfo *wi, const ITensorInfo *oi)
{
    ConvStrides cs;
    const auto  take = [](const ITensorInfo *t, int64_t *out)
    {
        if (t == nullptr || t->total_size() == 0)
            return;
        for (int i = 0; i < 3; ++i)
            out[i] = static_cast<int64_t>(t->strides_in_bytes()[i + 1]);
    };
    take(ii, cs.src), take(wi, cs.weights), take(oi, cs.dst);
    return cs;
}

// the C-ABI descriptor of a (validated) convolution on these tensor infos
void fill_conv_desc(const ITensorInfo *ii, const ITensorInfo *wi, const ITensorInfo *oi, const PadStrideInfo &conv_info,
                    const Size2D &dilation, const ActivationLayerInfo &act_info, mi355_conv_desc &d,
                    std::vector<int32_t> &multipliers, std::vector<int32_t> &shifts)
{
    const bool              dequant = oi->data_type() == DataType::F32;
    GEMMLowpOutputStageInfo stage;
    if (!dequant)
        ARM_COMPUTE_ERROR_THROW_ON(conv_output_stage(ii, wi, oi, act_info, stage));
    const ConvDims dm(ii->data_layout());
    d        = mi355_conv_desc{};
    d.layout = ii->data_layout() == DataLayout::NHWC ? MI355_NHWC : MI355_NCHW;
    d.C = static_cast<int32_t>(ii->dimension(dm.c)), d.W = static_cast<int32_t>(ii->dimension(dm.w));
    d.H = static_cast<int32_t>(ii->dimension(dm.h)), d.batch = static_cast<int32_t>(ii->tensor_shape().total_size_upper(3));
    d.KW = static_cast<int32_t>(wi->dimension(dm.w)), d.KH = static_cast<int32_t>(wi->dimension(dm.h));
    d.OFM      = static_cast<int32_t>(wi->dimension(3));
    d.stride_x = conv_info.stride().first, d.stride_y = conv_info.stride().second;
    d.pad_left = conv_info.pad_left(), d.pad_top = conv_info.pad_top();
    d.pad_right = conv_info.pad_right(), d.pad_bottom = conv_info.pad_bottom();
    d.dilation_x = static_cast<int32_t>(dilation.x()), d.dilation_y = static_cast<int32_t>(dilation.y());
    d.src_dtype = to_mi355(ii->data_type()), d.weights_dtype = to_mi355(wi->data_type());
    d.dst_dtype = to_mi355(oi->data_type());
    // the GEMM adds its offsets: hand it the negated zero points (CpuGemmConv2d.cpp:266-280 of the reference);
    // im2col pads with the un-negated input zero point (src/cpu/kernels/directconv2d/impl.h:333-334)
    const int32_t in_zp = ii->quantization_info().uniform().offset;
    d.src_offset        = -in_zp;
    d.weights_offset =
        is_data_type_quantized_per_channel(wi->data_type()) ? 0 : -wi->quantization_info().uniform().offset;
    d.pad_value = in_zp;
    d.path      = 0;
    d.act_min   = -std::numeric_limits<float>::infinity();
    d.act_max   = std::numeric_limits<float>::infinity();
    d.scale     = 1.f;
    if (dequant)
    {
        // the GEMM's dequantisation scale and fused activation, as for NEGEMMLowpMatrixMultiplyCore with an F32 output
        d.scale = ii->quantization_info().uniform().scale * wi->quantization_info().uniform().scale;
        if (act_info.enabled())
        {
            switch (act_info.activation())
            {
                case ActivationLayerInfo::ActivationFunction::RELU:
                    d.act_min = 0.f;
                    break;
                case ActivationLayerInfo::ActivationFunction::BOUNDED_RELU:
                    d.act_min = 0.f, d.act_max = act_info.a();
                    break;
                default: // LU_BOUNDED_RELU (validate() admits no other)
                    d.act_min = act_info.b(), d.act_max = act_info.a();
                    break;
            }
            if (act_info.b() == 0.f)
                d.flags |= MI355_GEMM_ACT_TWICE;
        }
    }
    else
        d.requant = make_requant(stage);
    const ConvStrides cs = conv_strides_of(ii, wi, oi);
    d.src_pixel_stride = cs.src[0], d.src_stride2 = cs.src[1], d.src_stride3 = cs.src[2];
    d.weights_pixel_stride = cs.weights[0], d.weights_stride2 = cs.weights[1], d.weights_stride3 = cs.weights[2];
    d.dst_pixel_stride = cs.dst[0], d.dst_stride2 = cs.dst[1], d.dst_stride3 = cs.dst[2];
    if (stage.is_quantized_per_channel)
    {
        multipliers.assign(stage.gemmlowp_multipliers.begin(), stage.gemmlowp_multipliers.begin() + d.OFM);
        shifts.assign(stage.gemmlowp_shifts.begin(), stage.gemmlowp_shifts.begin() + d.OFM);
    }
    else
        multipliers.clear(), shifts.clear();
}

// new quantization of src / weights / dst into an existing descriptor
void refresh_conv_quant(const ITensorInfo *ii, const ITensorInfo *wi, const ITensorInfo *oi, const ActivationLayerInfo &act,
                        mi355_conv_desc &d, std::vector<int32_t> &multipliers, std::vector<int32_t> &shifts)
{
    ARM_COMPUTE_ERROR_ON_MSG(oi->data_type() == DataType::F32,
                             "A convolution with an F32 destination has to be configured again for new quantization");
    GEMMLowpOutputStageInfo stage;
    ARM_COMPUTE_ERROR_THROW_ON(conv_output_stage(ii, wi, oi, act, stage));
    const int32_t in_zp = ii->quantization_info().uniform().offset;
    d.src_offset        = -in_zp;
    d.pad_value         = in_zp;
    d.weights_offset =
        is_data_type_quantized_per_channel(wi->data_type()) ? 0 : -wi->quantization_info().uniform().offset;
    d.requant = make_requant(stage);
    if (stage.is_quantized_per_channel)
    {
        multipliers.assign(stage.gemmlowp_multipliers.begin(), stage.gemmlowp_multipliers.begin() + d.OFM);
        shifts.assign(stage.gemmlowp_shifts.begin(), stage.gemmlowp_shifts.begin() + d.OFM);
    }
}
} // namespace

void NEGEMMConvolutionLayer::configure(const ITensor *input, const ITensor *weights, const ITensor *biases,
                                       ITensor *output, const PadStrideInfo &conv_info, const WeightsInfo &weights_info,
                                       const Size2D &dilation, const ActivationLayerInfo &act_info,
                                       bool enable_fast_math, unsigned int num_groups)
{
    ARM_COMPUTE_ERROR_ON_NULLPTR(input, weights, output);
    const ITensorInfo *ii = input->info(), *wi = weights->info();
    conv_auto_init_output(ii, wi, output->info(), conv_info, dilation);
    ARM_COMPUTE_ERROR_THROW_ON(validate(ii, wi, biases != nullptr ? biases->info() : nullptr, output->info(), conv_info,
                                        weights_info, dilation, act_info, enable_fast_math, num_groups));
    Impl &s = *_impl;
    if (s.handle)
    {
        mi355_conv_destroy(s.handle);
        s.handle = nullptr;
    }
    s.src = input, s.weights = weights, s.biases = biases, s.dst = output, s.act = act_info;
    s.is_prepared = false;
    fill_conv_desc(ii, wi, output->info(), conv_info, dilation, act_info, s.desc, s.multipliers, s.shifts);
    check_abi(mi355_conv_create(&s.desc, &s.handle), "NEGEMMConvolutionLayer::configure");
}

namespace
{
// see sync_gemm_strides: the same for the convolution's pixel strides (an info that is not at hand, or weights that
// are already packed, leave their stride as it is)
void sync_conv_strides(const ITensorInfo *ii, const ITensorInfo *wi, const ITensorInfo *oi, mi355_conv_desc &d,
                       mi355_conv_handle *handle, const char *where)
{
    ConvStrides now = conv_strides_of(ii, wi, oi);
    const int64_t have[3][3] = {{d.src_pixel_stride, d.src_stride2, d.src_stride3},
                                {d.weights_pixel_stride, d.weights_stride2, d.weights_stride3},
                                {d.dst_pixel_stride, d.dst_stride2, d.dst_stride3}};
    if (!ii)
        std::copy(have[0], have[0] + 3, now.src);
    if (!wi)
        std::copy(have[1], have[1] + 3, now.weights);
    if (!oi)
        std::copy(have[2], have[2] + 3, now.dst);
    if (std::equal(now.src, now.src + 3, have[0]) && std::equal(now.weights, now.weights + 3, have[1]) &&
        std::equal(now.dst, now.dst + 3, have[2]))
        return;
    check_abi(mi355_conv_set_strides_nd(handle, now.src, now.weights, now.dst), where);
    d.src_pixel_stride = now.src[0], d.src_stride2 = now.src[1], d.src_stride3 = now.src[2];
    d.weights_pixel_stride = now.weights[0], d.weights_stride2 = now.weights[1], d.weights_stride3 = now.weights[2];
    d.dst_pixel_stride = now.dst[0], d.dst_stride2 = now.dst[1], d.dst_stride3 = now.dst[2];
}
} // namespace

void NEGEMMConvolutionLayer::prepare()
{
    Impl &s = *_impl;
    ARM_COMPUTE_ERROR_ON_MSG(s.handle == nullptr, "NEGEMMConvolutionLayer::prepare() before configure()");
    sync_conv_strides(s.src->info(), s.is_prepared ? nullptr : s.weights->info(), s.dst->info(), s.desc, s.handle,
                      "NEGEMMConvolutionLayer::prepare");
    if (s.is_prepared)
        return;
    ARM_COMPUTE_ERROR_ON_MSG(s.weights->buffer() == nullptr, "weights have no memory");
    check_abi(mi355_conv_prepare(s.handle, first_element(s.weights), s.biases ? first_element(s.biases) : nullptr,
                                 s.multipliers.empty() ? nullptr : s.multipliers.data(),
                                 s.shifts.empty() ? nullptr : s.shifts.data(), nullptr),
              "NEGEMMConvolutionLayer::prepare");
    s.weights->mark_as_unused();
    s.is_prepared = true;
}

void NEGEMMConvolutionLayer::update_quantization_parameters()
{
    Impl &s = *_impl;
    ARM_COMPUTE_ERROR_ON_MSG(s.handle == nullptr, "update_quantization_parameters() before configure()");
    refresh_conv_quant(s.src->info(), s.weights->info(), s.dst->info(), s.act, s.desc, s.multipliers, s.shifts);
    check_abi(mi355_conv_update_quant(s.handle, s.desc.src_offset, s.desc.weights_offset, s.desc.pad_value,
                                      &s.desc.requant, s.multipliers.empty() ? nullptr : s.multipliers.data(),
                                      s.shifts.empty() ? nullptr : s.shifts.data(), nullptr),
              "NEGEMMConvolutionLayer::update_quantization_parameters");
}

void NEGEMMConvolutionLayer::run()
{
    Impl &s = *_impl;
    ARM_COMPUTE_ERROR_ON_MSG(s.handle == nullptr, "NEGEMMConvolutionLayer::run() before configure()");
    ARM_COMPUTE_ERROR_ON_MSG(s.src->buffer() == nullptr || s.dst->buffer() == nullptr, "tensor without memory");
    prepare();
    check_abi(mi355_conv_run(s.handle, first_element(s.src), first_element(s.dst), nullptr), "NEGEMMConvolutionLayer::run");
}

const char *NEGEMMConvolutionLayer::kernel_name() const
{
    return _impl->handle ? mi355_conv_kernel_name(_impl->handle) : "";
}
// =====================================================================================================================
// NEFullyConnectedLayer
// =====================================================================================================================
struct NEFullyConnectedLayer::Impl
{
    const ITensor     *src{nullptr}, *weights{nullptr}, *biases{nullptr};
    ITensor           *dst{nullptr};
    mi355_gemm_desc    desc{};
    mi355_gemm_handle *handle{nullptr};
    bool               is_prepared{false};
    bool               dynamic_weights{false};
    FullyConnectedLayerInfo fc_info{};

    ~Impl()
    {
        if (handle)
            mi355_gemmlowp_destroy(handle);
    }
};

NEFullyConnectedLayer::NEFullyConnectedLayer(std::shared_ptr<IMemoryManager> memory_manager, IWeightsManager *weights_manager)
    : _impl(std::make_unique<Impl>())
{
    ARM_COMPUTE_UNUSED(memory_manager, weights_manager);
}
NEFullyConnectedLayer::~NEFullyConnectedLayer() = default;

namespace
{
// what CpuFullyConnected::validate / configure derive from the tensor infos
// (src/cpu/operators/CpuFullyConnected.cpp:232-262, 420-489 of the reference)
struct FcGeometry
{
    bool   weights_reshaped{true}; // the weights tensor is already [num_inputs rows][num_outputs], i.e. B itself
    bool   is_fc_after_conv{true};
    bool   convert_weights{false}; // trained in the other data layout
    size_t K{0}, N{0}, M{0};
    size_t k_interleave{0};        // _factor2 of CpuConvertFullyConnectedWeightsKernel
};

Status fc_geometry(const ITensorInfo *src, const ITensorInfo *weights, const ITensorInfo *dst,
                   const FullyConnectedLayerInfo &fc_info, FcGeometry &g)
{
    g.weights_reshaped             = fc_info.transpose_weights ? fc_info.are_weights_reshaped : true;
    const bool is_batched_fc_layer = dst->dimension(1) > 1;
    if (is_batched_fc_layer)
    {
        g.is_fc_after_conv = true;
        for (size_t i = 3; i < Dimensions<size_t>::num_max_dimensions; ++i)
            if (src->tensor_shape()[i] != dst->tensor_shape()[i - 2])
                g.is_fc_after_conv = false;
    }
    else
        g.is_fc_after_conv = src->num_dimensions() > 1;
    // after the (possibly implicit) transpose the weights are [K rows][N]
    g.K = g.weights_reshaped ? weights->dimension(1) : weights->dimension(0);
    g.N = g.weights_reshaped ? weights->dimension(0) : weights->dimension(1);
    if (g.is_fc_after_conv)
        ARM_COMPUTE_RETURN_ERROR_ON_MSG(g.K != src->dimension(0) * src->dimension(1) * src->dimension(2),
                                        "weights do not match the flattened input");
    else
        ARM_COMPUTE_RETURN_ERROR_ON_MSG(src->dimension(0) != g.K, "weights do not match the input");
    g.M = src->tensor_shape().total_size() / g.K;
    g.convert_weights = g.is_fc_after_conv && src->data_layout() != fc_info.weights_trained_layout;
    if (g.convert_weights)
    {
        ARM_COMPUTE_RETURN_ERROR_ON(fc_info.weights_trained_layout == DataLayout::UNKNOWN);
        // the tensor's own layout is the one the weights were NOT trained with
        const DataLayout in_layout = fc_info.weights_trained_layout == DataLayout::NCHW ? DataLayout::NHWC : DataLayout::NCHW;
        const size_t plane = src->dimension(get_data_layout_dimension_index(in_layout, DataLayoutDimension::WIDTH)) *
                             src->dimension(get_data_layout_dimension_index(in_layout, DataLayoutDimension::HEIGHT));
        const size_t chans = src->dimension(get_data_layout_dimension_index(in_layout, DataLayoutDimension::CHANNEL));
        g.k_interleave     = fc_info.weights_trained_layout == DataLayout::NCHW ? chans : plane;
    }
    return Status{};
}

// row strides of the three matrices; true when they differ from what d held
bool fc_strides(const ITensorInfo *ii, const ITensorInfo *wi, const ITensorInfo *oi, const FcGeometry &g, mi355_gemm_desc &d)
{
    // flattening an unpadded tensor is the identity on its bytes; a row that is a whole GEMM row keeps its own stride
    const int64_t lda = ii->dimension(0) == g.K ? static_cast<int64_t>(ii->strides_in_bytes()[1]) : static_cast<int64_t>(g.K);
    const int64_t ldb = static_cast<int64_t>(wi->strides_in_bytes()[1] / wi->element_size());
    const int64_t ldd = static_cast<int64_t>(g.M > 1 ? oi->strides_in_bytes()[1] / oi->element_size() : g.N);
    const bool    changed = lda != d.lda || ldb != d.ldb || ldd != d.ldd;
    d.lda = lda, d.ldb = ldb, d.ldd = ldd;
    return changed;
}

Status fc_output_stage(const ITensorInfo *src, const ITensorInfo *weights, const ITensorInfo *dst,
                       const ActivationLayerInfo &act, GEMMLowpOutputStageInfo &out)
{
    const UniformQuantizationInfo iq = src->quantization_info().uniform();
    const UniformQuantizationInfo wq = weights->quantization_info().uniform();
    const UniformQuantizationInfo oq = dst->quantization_info().uniform();
    const float                   multiplier = (iq.scale * wq.scale) / oq.scale;
    int32_t                       m = 0, sft = 0;
    ARM_COMPUTE_RETURN_ON_ERROR(quantization::calculate_quantized_multiplier(multiplier, &m, &sft));
    int32_t lo = get_min_max(src->data_type()).first, hi = get_min_max(src->data_type()).second;
    if (act.enabled())
    {
        // quantization::get_quantized_asymmetric_output_min_max (src/core/utils/quantization/AsymmHelpers.cpp:183-221)
        const bool is_signed = src->data_type() == DataType::QASYMM8_SIGNED;
        auto       q = [&](float v) -> int32_t { return is_signed ? quantize_qasymm8_signed(v, oq) : quantize_qasymm8(v, oq); };
        switch (act.activation())
        {
            case ActivationLayerInfo::ActivationFunction::RELU:
                lo = oq.offset;
                break;
            case ActivationLayerInfo::ActivationFunction::BOUNDED_RELU:
                lo = oq.offset;
                hi = q(act.a());
                break;
            case ActivationLayerInfo::ActivationFunction::LU_BOUNDED_RELU:
                lo = q(act.b());
                hi = q(act.a());
                break;
            default:
                ARM_COMPUTE_RETURN_ERROR_MSG("Activation function not supported.");
        }
    }
    out.type                = GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT;
    out.gemmlowp_multiplier = m;
    out.gemmlowp_shift      = sft;
    out.gemmlowp_offset     = oq.offset;
    out.gemmlowp_min_bound  = lo;
    out.gemmlowp_max_bound  = hi;
    return Status{};
}
} // namespace

// src/cpu/operators/CpuFullyConnected.cpp:384-489 of the reference, restricted to what this library builds
Status NEFullyConnectedLayer::validate(const ITensorInfo *input, const ITensorInfo *weights, const ITensorInfo *biases,
                                       const ITensorInfo *output, FullyConnectedLayerInfo fc_info,
                                       const WeightsInfo &weights_info)
{
    ARM_COMPUTE_RETURN_ERROR_ON_NULLPTR(input, weights, output);
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(weights_info.weight_format() != WeightFormat::UNSPECIFIED,
                                    "Fixed-format weights are not built in this library");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(is_one_of(input->data_type(), {DataType::F16, DataType::F32, DataType::BFLOAT16}),
                                    "Floating-point fully connected layers are not built in this library");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(!is_one_of(input->data_type(), {DataType::QASYMM8, DataType::QASYMM8_SIGNED}),
                                    "Input must be QASYMM8 or QASYMM8_SIGNED");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(weights->data_type() != input->data_type() || output->data_type() != input->data_type(),
                                    "Mismatching data types");
    ARM_COMPUTE_RETURN_ERROR_ON(weights->num_dimensions() > 2);
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(fc_info.activation_info.enabled() &&
                                        fusable_acts.count(fc_info.activation_info.activation()) == 0,
                                    "Only RELU, BOUNDED_RELU and LU_BOUNDED_RELU can be fused");
    if (biases != nullptr)
    {
        ARM_COMPUTE_RETURN_ERROR_ON(biases->num_dimensions() > 1);
        ARM_COMPUTE_RETURN_ERROR_ON_MSG(biases->data_type() != DataType::S32, "Biases must be S32");
    }
    FcGeometry g;
    ARM_COMPUTE_RETURN_ON_ERROR(fc_geometry(input, weights, output, fc_info, g));
    if (biases != nullptr)
        ARM_COMPUTE_RETURN_ERROR_ON(biases->dimension(0) != g.N);
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(output->dimension(0) != g.N, "The output's first dimension must be the number of outputs");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(output->tensor_shape().total_size() != g.M * g.N, "Mismatching number of batches");
    // a padded input is fine as long as one row of it is one row of the GEMM (nothing to flatten across the padding)
    if (input->has_padding())
    {
        ARM_COMPUTE_RETURN_ERROR_ON_MSG(input->dimension(0) != g.K, "A padded input cannot be flattened in place");
        for (size_t i = 2; i < input->num_dimensions(); ++i)
            ARM_COMPUTE_RETURN_ERROR_ON_MSG(input->strides_in_bytes()[i] != input->dimension(i - 1) * input->strides_in_bytes()[i - 1],
                                            "Padding between the rows' planes is not supported");
    }
    ARM_COMPUTE_RETURN_ON_ERROR(check_matrix_layout(weights, "weights"));
    ARM_COMPUTE_RETURN_ON_ERROR(check_matrix_layout(output, "output"));
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(g.M > 1 && output->num_dimensions() > 2 && output->has_padding(),
                                    "A padded output with more than two dimensions is not supported");
    GEMMLowpOutputStageInfo stage;
    ARM_COMPUTE_RETURN_ON_ERROR(fc_output_stage(input, weights, output, fc_info.activation_info, stage));
    return Status{};
}

Status NEFullyConnectedLayer::has_opt_impl(WeightFormat &expected_weight_format, const ITensorInfo *input,
                                           const ITensorInfo *weights, const ITensorInfo *biases, const ITensorInfo *output,
                                           const FullyConnectedLayerInfo &fc_info, const WeightsInfo &weights_info)
{
    // no fixed-format weights in this library: the packed layout is private to the device workspace
    expected_weight_format = WeightFormat::UNSPECIFIED;
    ARM_COMPUTE_RETURN_ON_ERROR(validate(input, weights, biases, output, fc_info, weights_info));
    ARM_COMPUTE_RETURN_ERROR_MSG("No fixed-format kernel available");
}

void NEFullyConnectedLayer::configure(const ITensor *input, const ITensor *weights, const ITensor *biases, ITensor *output,
                                      FullyConnectedLayerInfo fc_info, const WeightsInfo &weights_info)
{
    ARM_COMPUTE_ERROR_ON_NULLPTR(input, weights, output);
    const ITensorInfo *ii = input->info(), *wi = weights->info(), *oi = output->info();
    ARM_COMPUTE_ERROR_THROW_ON(validate(ii, wi, biases != nullptr ? biases->info() : nullptr, oi, fc_info, weights_info));
    FcGeometry g;
    ARM_COMPUTE_ERROR_THROW_ON(fc_geometry(ii, wi, oi, fc_info, g));
    GEMMLowpOutputStageInfo stage;
    ARM_COMPUTE_ERROR_THROW_ON(fc_output_stage(ii, wi, oi, fc_info.activation_info, stage));

    mi355_gemm_desc d{};
    d.M = static_cast<int32_t>(g.M), d.N = static_cast<int32_t>(g.N), d.K = static_cast<int32_t>(g.K), d.batch = 1;
    d.a_dtype = to_mi355(ii->data_type()), d.b_dtype = to_mi355(wi->data_type()), d.dst_dtype = to_mi355(oi->data_type());
    d.epilogue = MI355_EPI_FIXEDPOINT;
    fc_strides(ii, wi, oi, g, d);
    d.a_batch_stride = d.b_batch_stride = d.d_batch_stride = 0;
    // the GEMM adds its offsets: negated zero points (CpuFullyConnected.cpp:98-103,166-171 of the reference)
    d.a_offset       = -ii->quantization_info().uniform().offset;
    d.b_offset       = -wi->quantization_info().uniform().offset;
    d.requant        = make_requant(stage);
    d.scale          = 1.f;
    d.act_min        = -std::numeric_limits<float>::infinity();
    d.act_max        = std::numeric_limits<float>::infinity();
    d.path           = MI355_PATH_AUTO;
    d.b_transposed   = g.weights_reshaped ? 0 : 1; // [num_outputs rows][num_inputs]: the transpose happens while packing
    d.b_k_interleave = g.convert_weights ? static_cast<int32_t>(g.k_interleave) : 0;

    Impl      &s    = *_impl;
    const bool keep = fc_info.retain_internal_weights && s.handle != nullptr && s.is_prepared && s.desc.M == d.M &&
                      s.desc.N == d.N && s.desc.K == d.K && s.desc.b_dtype == d.b_dtype;
    s.src = input, s.weights = weights, s.biases = biases, s.dst = output, s.fc_info = fc_info;
    s.dynamic_weights = !wi->are_values_constant() && !g.weights_reshaped;
    if (keep)
    {
        // packed weights of the previous configuration stay; offsets and requantisation may have changed
        s.desc.a_offset = d.a_offset, s.desc.b_offset = d.b_offset, s.desc.requant = d.requant;
        check_abi(mi355_gemmlowp_update_quant(s.handle, d.a_offset, d.b_offset, &d.requant, 1.f, nullptr),
                  "NEFullyConnectedLayer::configure");
        return;
    }
    if (s.handle)
    {
        mi355_gemmlowp_destroy(s.handle);
        s.handle = nullptr;
    }
    s.desc        = d;
    s.is_prepared = false;
    check_abi(mi355_gemmlowp_create(&d, &s.handle), "NEFullyConnectedLayer::configure");
}

void NEFullyConnectedLayer::prepare()
{
    Impl &s = *_impl;
    ARM_COMPUTE_ERROR_ON_MSG(s.handle == nullptr, "NEFullyConnectedLayer::prepare() before configure()");
    {
        // padding added after configure() (see sync_gemm_strides)
        FcGeometry g;
        ARM_COMPUTE_ERROR_THROW_ON(fc_geometry(s.src->info(), s.weights->info(), s.dst->info(), s.fc_info, g));
        if (fc_strides(s.src->info(), s.weights->info(), s.dst->info(), g, s.desc))
        {
            ARM_COMPUTE_ERROR_THROW_ON(validate(s.src->info(), s.weights->info(), s.biases != nullptr ? s.biases->info() : nullptr,
                                                s.dst->info(), s.fc_info));
            mi355_gemmlowp_destroy(s.handle);
            s.handle = nullptr;
            check_abi(mi355_gemmlowp_create(&s.desc, &s.handle), "NEFullyConnectedLayer::prepare");
            s.is_prepared = false;
        }
    }
    if (s.is_prepared && !s.dynamic_weights)
        return;
    ARM_COMPUTE_ERROR_ON_MSG(s.weights->buffer() == nullptr, "weights have no memory");
    check_abi(mi355_gemmlowp_prepare(s.handle, first_element(s.weights),
                                     s.biases ? reinterpret_cast<const int32_t *>(first_element(s.biases)) : nullptr,
                                     nullptr, nullptr, nullptr),
              "NEFullyConnectedLayer::prepare");
    if (!s.dynamic_weights)
        s.weights->mark_as_unused();
    s.is_prepared = true;
}

void NEFullyConnectedLayer::run()
{
    Impl &s = *_impl;
    ARM_COMPUTE_ERROR_ON_MSG(s.handle == nullptr, "NEFullyConnectedLayer::run() before configure()");
    ARM_COMPUTE_ERROR_ON_MSG(s.src->buffer() == nullptr || s.dst->buffer() == nullptr, "tensor without memory");
    prepare();
    check_abi(mi355_gemmlowp_run(s.handle, first_element(s.src), nullptr, first_element(s.dst), nullptr),
              "NEFullyConnectedLayer::run");
}

const char *NEFullyConnectedLayer::kernel_name() const
{
    return _impl->handle ? mi355_gemmlowp_kernel_name(_impl->handle) : "";
}
// =====================================================================================================================
// NEGEMMConv2d
// =====================================================================================================================
NEGEMMConv2d::NEGEMMConv2d(const std::shared_ptr<IMemoryManager> &memory_manager)
    : _conv(std::make_unique<NEGEMMConvolutionLayer>(memory_manager))
{
}
NEGEMMConv2d::~NEGEMMConv2d() = default;

// src/cpu/operators/CpuGemmDirectConv2d.cpp:166-224 of the reference
Status NEGEMMConv2d::validate(const ITensorInfo *input, const ITensorInfo *weights, const ITensorInfo *biases,
                              const ITensorInfo *output, const Conv2dInfo &info)
{
    ARM_COMPUTE_RETURN_ERROR_ON_NULLPTR(input, weights, output);
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(info.num_groups > 1, "Grouping (num_groups != 1) is not supported on Cpu");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(input->data_layout() != DataLayout::NHWC, "Data layout supported is NHWC");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(info.dilation != Size2D(1U, 1U), "Dilation is not supported by NEGEMMConv2d");
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(info.weights_info.weight_format() != WeightFormat::UNSPECIFIED,
                                    "Fixed-format weights are not built in this library");
    return NEGEMMConvolutionLayer::validate(input, weights, biases, output, info.conv_info, WeightsInfo(), info.dilation,
                                            info.act_info, info.enable_fast_math, info.num_groups);
}

void NEGEMMConv2d::configure(ITensor *input, const ITensor *weights, const ITensor *biases, ITensor *output,
                             const Conv2dInfo &info)
{
    ARM_COMPUTE_ERROR_ON_NULLPTR(input, weights, output);
    if (output->info()->total_size() != 0)
        ARM_COMPUTE_ERROR_THROW_ON(validate(input->info(), weights->info(), biases != nullptr ? biases->info() : nullptr,
                                            output->info(), info));
    else
    {
        ARM_COMPUTE_ERROR_ON_MSG(info.dilation != Size2D(1U, 1U), "Dilation is not supported by NEGEMMConv2d");
        ARM_COMPUTE_ERROR_ON_MSG(info.num_groups > 1, "Grouping (num_groups != 1) is not supported on Cpu");
    }
    _conv->configure(input, weights, biases, output, info.conv_info, WeightsInfo(), info.dilation, info.act_info,
                     info.enable_fast_math, info.num_groups);
}

void NEGEMMConv2d::run()
{
    _conv->run();
}

void NEGEMMConv2d::prepare()
{
    _conv->prepare();
}

const char *NEGEMMConv2d::kernel_name() const
{
    return _conv->kernel_name();
}
// =====================================================================================================================
// experimental::op::CpuGEMMLowp
// =====================================================================================================================
namespace experimental
{
namespace op
{
struct CpuGEMMLowp::Impl
{
    mi355_gemm_desc      desc{};
    mi355_gemm_handle   *handle{nullptr};
    GEMMInfo             info{};
    bool                 b_per_channel{false};
    ActivationLayerInfo  act_info{};
    bool                 is_prepared{false};
    bool                 b_constant{true};
    bool                 has_bias{false};
    std::vector<int32_t> multipliers, shifts;

    ~Impl()
    {
        if (handle)
            mi355_gemmlowp_destroy(handle);
    }
};

CpuGEMMLowp::CpuGEMMLowp() : _impl(std::make_unique<Impl>()) {}
CpuGEMMLowp::~CpuGEMMLowp() = default;

MemoryRequirements CpuGEMMLowp::workspace() const
{
    return {}; // packed B, column sums and staging buffers live in device memory owned by the handle
}

Status CpuGEMMLowp::validate(const ITensorInfo *a, const ITensorInfo *b, const ITensorInfo *c, const ITensorInfo *output,
                             const GEMMInfo &gemm_info)
{
    return NEGEMMLowpMatrixMultiplyCore::validate(a, b, c, output, gemm_info);
}

void CpuGEMMLowp::configure(const ITensorInfo *a, const ITensorInfo *b, const ITensorInfo *c, ITensorInfo *output,
                            const GEMMInfo &gemm_info)
{
    ARM_COMPUTE_ERROR_ON_NULLPTR(a, b, output);
    ARM_COMPUTE_ERROR_THROW_ON(validate(a, b, c, output, gemm_info));
    Impl &s = *_impl;
    if (s.handle)
    {
        mi355_gemmlowp_destroy(s.handle);
        s.handle = nullptr;
    }
    s.act_info    = gemm_info.activation_info();
    s.info        = gemm_info;
    s.b_per_channel = is_data_type_quantized_per_channel(b->data_type());
    s.is_prepared = false;
    s.b_constant  = gemm_info.reshape_b_only_on_first_run(); // CpuGEMMLowp.cpp:60-66 of the reference
    s.has_bias    = c != nullptr;
    fill_gemm_desc(a, b, output, gemm_info, s.desc, s.multipliers, s.shifts);
    check_abi(mi355_gemmlowp_create(&s.desc, &s.handle), "CpuGEMMLowp::configure");
}

void CpuGEMMLowp::update_quantization_parameters(const QuantizationInfo &a, const QuantizationInfo &b,
                                                 const QuantizationInfo &c, const DataType data_type,
                                                 const bool is_prepared, const bool negated_offsets)
{
    Impl &s = *_impl;
    ARM_COMPUTE_ERROR_ON_MSG(s.handle == nullptr, "update_quantization_parameters() before configure()");
    ARM_COMPUTE_ERROR_ON_MSG(s.desc.epilogue != MI355_EPI_FIXEDPOINT || s.desc.requant.per_channel,
                             "only a per-tensor fixed-point output stage can be updated in place");
    int32_t                       lo = get_min_max(data_type).first, hi = get_min_max(data_type).second;
    const UniformQuantizationInfo uo = c.uniform();
    if (fusable_acts.count(s.act_info.activation()) != 0)
        std::tie(lo, hi) = get_quantized_activation_min_max(s.act_info, data_type, uo);
    GEMMLowpOutputStageInfo out;
    out.type                     = GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT;
    out.gemmlowp_offset          = uo.offset;
    out.gemmlowp_min_bound       = lo;
    out.gemmlowp_max_bound       = hi;
    out.is_quantized_per_channel = false;
    out.output_data_type         = data_type;
    ARM_COMPUTE_ERROR_THROW_ON(quantization::calculate_quantized_multipliers(a, b, c, out));
    // negated_offsets == true: the offsets in a / b are already the values ADDED to every element (what the tensors of
    // NEGEMMLowpMatrixMultiplyCore carry); false: they are true zero points, which are subtracted
    // (src/cpu/operators/internal/CpuGemmAssemblyDispatch.cpp:213-215: arm_gemm's subtracted zero point is
    // -offset * (negated ? 1 : -1))
    s.desc.a_offset = negated_offsets ? a.uniform().offset : -a.uniform().offset;
    s.desc.b_offset = negated_offsets ? b.uniform().offset : -b.uniform().offset;
    s.desc.requant  = make_requant(out);
    check_abi(mi355_gemmlowp_update_quant(s.handle, s.desc.a_offset, s.desc.b_offset, &s.desc.requant, s.desc.scale, nullptr),
              "CpuGEMMLowp::update_quantization_parameters");
    s.is_prepared = s.is_prepared && is_prepared;
}

void CpuGEMMLowp::prepare(ITensorPack &tensors)
{
    Impl &s = *_impl;
    ARM_COMPUTE_ERROR_ON_MSG(s.handle == nullptr, "CpuGEMMLowp::prepare() before configure()");
    if (s.is_prepared)
        return;
    const ITensor *b = tensors.get_const_tensor(ACL_SRC_1);
    ARM_COMPUTE_ERROR_ON_MSG(b == nullptr || b->buffer() == nullptr, "matrix B (ACL_SRC_1) is missing or has no memory");
    // the strides are those of the tensor in the pack, which may have been padded after configure()
    ARM_COMPUTE_ERROR_THROW_ON(check_matrix_layout(b->info(), "b"));
    sync_gemm_strides(nullptr, b->info(), nullptr, s.info, s.desc, s.handle, false, "CpuGEMMLowp::prepare");
    const int32_t *bias = nullptr;
    if (s.desc.epilogue == MI355_EPI_FIXEDPOINT && s.has_bias)
    {
        const ITensor *c = tensors.get_const_tensor(ACL_SRC_2);
        ARM_COMPUTE_ERROR_ON_MSG(c == nullptr || c->buffer() == nullptr, "bias (ACL_SRC_2) is missing or has no memory");
        bias = reinterpret_cast<const int32_t *>(first_element(c));
    }
    check_abi(mi355_gemmlowp_prepare(s.handle, first_element(b), bias, s.multipliers.empty() ? nullptr : s.multipliers.data(),
                                     s.shifts.empty() ? nullptr : s.shifts.data(), nullptr),
              "CpuGEMMLowp::prepare");
    if (s.b_constant)
    {
        b->mark_as_unused();
        s.is_prepared = true;
    }
}

void CpuGEMMLowp::run(ITensorPack &tensors)
{
    Impl &s = *_impl;
    ARM_COMPUTE_ERROR_ON_MSG(s.handle == nullptr, "CpuGEMMLowp::run() before configure()");
    const ITensor *a   = tensors.get_const_tensor(ACL_SRC_0);
    ITensor       *dst = tensors.get_tensor(ACL_DST);
    ARM_COMPUTE_ERROR_ON_MSG(a == nullptr || dst == nullptr || a->buffer() == nullptr || dst->buffer() == nullptr,
                             "ACL_SRC_0 / ACL_DST missing or without memory");
    // dynamic quantization: offsets (and the dequantisation scale) are those the tensors of this pack carry now
    // (src/cpu/operators/CpuGemmLowpMatrixMultiplyCore.cpp:668-674,776-784 of the reference)
    const ITensor *bq = tensors.get_const_tensor(ACL_SRC_1);
    if (a->info()->quantization_info().is_dynamic() || (bq != nullptr && bq->info()->quantization_info().is_dynamic()))
    {
        const int32_t ao = a->info()->quantization_info().uniform().offset;
        const int32_t bo = (s.b_per_channel || bq == nullptr) ? s.desc.b_offset : bq->info()->quantization_info().uniform().offset;
        const float   sc = (s.desc.epilogue == MI355_EPI_F32 && bq != nullptr)
                               ? a->info()->quantization_info().uniform().scale * bq->info()->quantization_info().uniform().scale
                               : s.desc.scale;
        if (ao != s.desc.a_offset || bo != s.desc.b_offset || sc != s.desc.scale)
        {
            s.desc.a_offset = ao, s.desc.b_offset = bo, s.desc.scale = sc;
            check_abi(mi355_gemmlowp_update_quant(s.handle, ao, bo, nullptr, sc, nullptr), "CpuGEMMLowp::run");
        }
    }
    prepare(tensors);
    // the strides of the tensors actually handed over (padding may have been added after configure())
    ARM_COMPUTE_ERROR_THROW_ON(check_matrix_layout(a->info(), "a"));
    ARM_COMPUTE_ERROR_THROW_ON(check_matrix_layout(dst->info(), "output"));
    sync_gemm_strides(a->info(), nullptr, dst->info(), s.info, s.desc, s.handle, true, "CpuGEMMLowp::run");
    const float *bias_f32 = nullptr;
    if (s.desc.epilogue == MI355_EPI_F32 && s.has_bias)
    {
        const ITensor *c = tensors.get_const_tensor(ACL_SRC_2);
        ARM_COMPUTE_ERROR_ON_MSG(c == nullptr || c->buffer() == nullptr, "bias (ACL_SRC_2) is missing or has no memory");
        bias_f32 = reinterpret_cast<const float *>(first_element(c));
    }
    check_abi(mi355_gemmlowp_run(s.handle, first_element(a), bias_f32, first_element(dst), nullptr), "CpuGEMMLowp::run");
}

// =====================================================================================================================
// experimental::op::CpuGemmConv2d
// =====================================================================================================================
struct CpuGemmConv2d::Impl
{
    mi355_conv_desc      desc{};
    mi355_conv_handle   *handle{nullptr};
    ActivationLayerInfo  act{};
    bool                 is_prepared{false};
    bool                 has_bias{false};
    std::vector<int32_t> multipliers, shifts;

    ~Impl()
    {
        if (handle)
            mi355_conv_destroy(handle);
    }
};

CpuGemmConv2d::CpuGemmConv2d() : _impl(std::make_unique<Impl>()) {}
CpuGemmConv2d::~CpuGemmConv2d() = default;

MemoryRequirements CpuGemmConv2d::workspace() const
{
    return {}; // packed weights, the lowered patch matrix (when one is needed) and staging buffers belong to the handle
}

Status CpuGemmConv2d::validate(const ITensorInfo *src, const ITensorInfo *weights, const ITensorInfo *biases,
                               const ITensorInfo *output, const PadStrideInfo &conv_info, const WeightsInfo &weights_info,
                               const Size2D &dilation, const ActivationLayerInfo &act_info, bool enable_fast_math,
                               unsigned int num_groups)
{
    return NEGEMMConvolutionLayer::validate(src, weights, biases, output, conv_info, weights_info, dilation, act_info,
                                            enable_fast_math, num_groups);
}

Status CpuGemmConv2d::has_opt_impl(arm_compute::WeightFormat &expected_weight_format, const ITensorInfo *src,
                                   const ITensorInfo *weights, const ITensorInfo *biases, const ITensorInfo *output,
                                   const PadStrideInfo &conv_info, const WeightsInfo &weights_info, const Size2D &dilation,
                                   const ActivationLayerInfo &act_info, bool enable_fast_math)
{
    return NEGEMMConvolutionLayer::has_opt_impl(expected_weight_format, src, weights, biases, output, conv_info,
                                                weights_info, dilation, act_info, enable_fast_math);
}

void CpuGemmConv2d::configure(const ITensorInfo *src, const ITensorInfo *weights, const ITensorInfo *biases,
                              ITensorInfo *dst, const PadStrideInfo &conv_info, const WeightsInfo &weights_info,
                              const Size2D &dilation, const ActivationLayerInfo &act_info, bool enable_fast_math,
                              unsigned int num_groups)
{
    ARM_COMPUTE_ERROR_ON_NULLPTR(src, weights, dst);
    conv_auto_init_output(src, weights, dst, conv_info, dilation);
    ARM_COMPUTE_ERROR_THROW_ON(
        validate(src, weights, biases, dst, conv_info, weights_info, dilation, act_info, enable_fast_math, num_groups));
    Impl &s = *_impl;
    if (s.handle)
    {
        mi355_conv_destroy(s.handle);
        s.handle = nullptr;
    }
    s.act = act_info, s.is_prepared = false, s.has_bias = biases != nullptr;
    fill_conv_desc(src, weights, dst, conv_info, dilation, act_info, s.desc, s.multipliers, s.shifts);
    check_abi(mi355_conv_create(&s.desc, &s.handle), "CpuGemmConv2d::configure");
}

void CpuGemmConv2d::prepare(ITensorPack &tensors)
{
    Impl &s = *_impl;
    ARM_COMPUTE_ERROR_ON_MSG(s.handle == nullptr, "CpuGemmConv2d::prepare() before configure()");
    if (s.is_prepared)
        return;
    const ITensor *w = tensors.get_const_tensor(ACL_SRC_1);
    ARM_COMPUTE_ERROR_ON_MSG(w == nullptr || w->buffer() == nullptr, "weights (ACL_SRC_1) are missing or have no memory");
    // the strides are those of the tensor in the pack, which may have been padded after configure()
    sync_conv_strides(nullptr, w->info(), nullptr, s.desc, s.handle, "CpuGemmConv2d::prepare");
    const int32_t *bias = nullptr;
    if (s.has_bias)
    {
        const ITensor *b = tensors.get_const_tensor(ACL_SRC_2);
        ARM_COMPUTE_ERROR_ON_MSG(b == nullptr || b->buffer() == nullptr, "biases (ACL_SRC_2) are missing or have no memory");
        bias = reinterpret_cast<const int32_t *>(first_element(b));
    }
    check_abi(mi355_conv_prepare(s.handle, first_element(w), bias, s.multipliers.empty() ? nullptr : s.multipliers.data(),
                                 s.shifts.empty() ? nullptr : s.shifts.data(), nullptr),
              "CpuGemmConv2d::prepare");
    w->mark_as_unused();
    s.is_prepared = true;
}

void CpuGemmConv2d::update_quantization_parameters(ITensorPack &tensors)
{
    Impl &s = *_impl;
    ARM_COMPUTE_ERROR_ON_MSG(s.handle == nullptr, "update_quantization_parameters() before configure()");
    const ITensor *src = tensors.get_const_tensor(ACL_SRC_0), *w = tensors.get_const_tensor(ACL_SRC_1);
    const ITensor *dst = tensors.get_const_tensor(ACL_DST);
    ARM_COMPUTE_ERROR_ON_MSG(src == nullptr || w == nullptr || dst == nullptr, "ACL_SRC_0 / ACL_SRC_1 / ACL_DST missing");
    refresh_conv_quant(src->info(), w->info(), dst->info(), s.act, s.desc, s.multipliers, s.shifts);
    check_abi(mi355_conv_update_quant(s.handle, s.desc.src_offset, s.desc.weights_offset, s.desc.pad_value, &s.desc.requant,
                                      s.multipliers.empty() ? nullptr : s.multipliers.data(),
                                      s.shifts.empty() ? nullptr : s.shifts.data(), nullptr),
              "CpuGemmConv2d::update_quantization_parameters");
}

void CpuGemmConv2d::run(ITensorPack &tensors)
{
    Impl &s = *_impl;
    ARM_COMPUTE_ERROR_ON_MSG(s.handle == nullptr, "CpuGemmConv2d::run() before configure()");
    const ITensor *src = tensors.get_const_tensor(ACL_SRC_0);
    ITensor       *dst = tensors.get_tensor(ACL_DST);
    ARM_COMPUTE_ERROR_ON_MSG(src == nullptr || dst == nullptr || src->buffer() == nullptr || dst->buffer() == nullptr,
                             "ACL_SRC_0 / ACL_DST missing or without memory");
    prepare(tensors);
    sync_conv_strides(src->info(), nullptr, dst->info(), s.desc, s.handle, "CpuGemmConv2d::run");
    check_abi(mi355_conv_run(s.handle, first_element(src), first_element(dst), nullptr), "CpuGemmConv2d::run");
}
} // namespace op
} // namespace experimental
} // namespace arm_compute
