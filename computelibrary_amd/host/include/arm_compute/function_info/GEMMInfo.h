// GEMMLowpOutputStageInfo and GEMMInfo. Mirrors arm_compute/function_info/GEMMInfo.h:40-400 of the reference: same field
// and accessor names, same defaults.
#ifndef ACL_MI355_FUNCTION_INFO_GEMMINFO_H
#define ACL_MI355_FUNCTION_INFO_GEMMINFO_H

#include "arm_compute/core/Types.h"

#include <limits>
#include <vector>

namespace arm_compute
{
enum class GEMMLowpOutputStageType
{
    NONE,
    QUANTIZE_DOWN,
    QUANTIZE_DOWN_FIXEDPOINT,
    QUANTIZE_DOWN_FLOAT
};

struct GEMMLowpOutputStageInfo
{
    GEMMLowpOutputStageType type{GEMMLowpOutputStageType::NONE};
    int32_t                 gemmlowp_offset{0};
    int32_t                 gemmlowp_multiplier{0};
    int32_t                 gemmlowp_shift{0};
    int32_t                 gemmlowp_min_bound{std::numeric_limits<int32_t>::lowest()};
    int32_t                 gemmlowp_max_bound{std::numeric_limits<int32_t>::max()};
    std::vector<int32_t>    gemmlowp_multipliers{};
    std::vector<int32_t>    gemmlowp_shifts{};
    float                   gemmlowp_real_multiplier{0};
    bool                    is_quantized_per_channel{false};
    DataType                output_data_type{DataType::UNKNOWN};
};

class GEMMInfo
{
public:
    GEMMInfo() noexcept = default;
    GEMMInfo(bool is_a_reshaped, bool is_b_reshaped, bool reshape_b_only_on_first_run, int depth_output_gemm3d = 0,
             bool reinterpret_input_as_3d = false, bool retain_internal_weights = false,
             GEMMLowpOutputStageInfo gemmlowp_output_stage = GEMMLowpOutputStageInfo(), bool fp_mixed_precision = false,
             bool fast_math = false, bool broadcast_bias = false,
             const ActivationLayerInfo &activation_info = ActivationLayerInfo(), bool fixed_format = false,
             WeightFormat weight_format = WeightFormat::UNSPECIFIED, bool pretranspose_B = false,
             bool accumulate = false) noexcept
        : _is_a_reshaped(is_a_reshaped), _is_b_reshaped(is_b_reshaped),
          _reshape_b_only_on_first_run(reshape_b_only_on_first_run), _depth_output_gemm3d(depth_output_gemm3d),
          _reinterpret_input_as_3d(reinterpret_input_as_3d), _retain_internal_weights(retain_internal_weights),
          _gemmlowp_output_stage(std::move(gemmlowp_output_stage)), _fast_math(fast_math),
          _fp_mixed_precision(fp_mixed_precision), _broadcast_bias(broadcast_bias), _pretranspose_A(false),
          _pretranspose_B(pretranspose_B), _activation_info(activation_info), _fixed_format(fixed_format),
          _weight_format(weight_format), _accumulate(accumulate)
    {
    }
    bool is_a_reshaped() const { return _is_a_reshaped; }
    bool is_b_reshaped() const { return _is_b_reshaped; }
    bool reshape_b_only_on_first_run() const { return _reshape_b_only_on_first_run; }
    int  depth_output_gemm3d() const { return _depth_output_gemm3d; }
    bool reinterpret_input_as_3d() const { return _reinterpret_input_as_3d; }
    bool retain_internal_weights() const { return _retain_internal_weights; }
    GEMMLowpOutputStageInfo gemmlowp_output_stage() const { return _gemmlowp_output_stage; }
    void set_gemmlowp_output_stage(GEMMLowpOutputStageInfo &output_stage) { _gemmlowp_output_stage = output_stage; }
    bool fp_mixed_precision() const { return _fp_mixed_precision; }
    bool fast_math() const { return _fast_math; }
    bool broadcast_bias() const { return _broadcast_bias; }
    bool pretranspose_A() const { return _pretranspose_A; }
    void set_pretranspose_A(bool flag) { _pretranspose_A = flag; }
    bool pretranspose_B() const { return _pretranspose_B; }
    void set_pretranspose_B(bool flag) { _pretranspose_B = flag; }
    ActivationLayerInfo activation_info() const { return _activation_info; }
    void set_activation_info(const ActivationLayerInfo &activation_info) { _activation_info = activation_info; }
    bool         fixed_format() const { return _fixed_format; }
    bool         accumulate() const { return _accumulate; }
    void         set_accumulate(bool value) { _accumulate = value; }
    WeightFormat weight_format() const { return _weight_format; }

private:
    bool                    _is_a_reshaped{false};
    bool                    _is_b_reshaped{false};
    bool                    _reshape_b_only_on_first_run{true};
    int                     _depth_output_gemm3d{0};
    bool                    _reinterpret_input_as_3d{false};
    bool                    _retain_internal_weights{false};
    GEMMLowpOutputStageInfo _gemmlowp_output_stage{};
    bool                    _fast_math{false};
    bool                    _fp_mixed_precision{false};
    bool                    _broadcast_bias{false};
    bool                    _pretranspose_A{false};
    bool                    _pretranspose_B{false};
    ActivationLayerInfo     _activation_info{};
    bool                    _fixed_format{false};
    WeightFormat            _weight_format{WeightFormat::UNSPECIFIED};
    bool                    _accumulate{false};
};
} // namespace arm_compute
#endif
