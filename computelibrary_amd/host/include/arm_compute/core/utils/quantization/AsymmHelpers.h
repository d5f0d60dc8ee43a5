// float scale -> (Q31 multiplier, shift) conversions used to build a fixed-point output stage.
// Mirrors src/core/utils/quantization/AsymmHelpers.cpp:43-152 of the reference (same names, same results).
#ifndef ACL_MI355_CORE_UTILS_QUANTIZATION_ASYMMHELPERS_H
#define ACL_MI355_CORE_UTILS_QUANTIZATION_ASYMMHELPERS_H

#include "arm_compute/core/Error.h"
#include "arm_compute/core/Types.h"
#include "arm_compute/function_info/GEMMInfo.h"

namespace arm_compute
{
namespace quantization
{
Status calculate_quantized_multiplier(float multiplier, int32_t *quant_multiplier, int32_t *shift,
                                      bool ignore_epsilon = false);
Status calculate_quantized_multiplier_less_than_one(float multiplier, int32_t *quant_multiplier, int32_t *right_shift,
                                                    bool ignore_epsilon = false);
Status calculate_quantized_multiplier_greater_than_one(float multiplier, int32_t *quantized_multiplier,
                                                       int32_t *left_shift);
// fills stage_info.gemmlowp_multipliers / gemmlowp_shifts (padded by 32 entries when per-channel) and the scalar pair
Status calculate_quantized_multipliers(const QuantizationInfo &iq_info, const QuantizationInfo &wq_info,
                                       const QuantizationInfo &oq_info, GEMMLowpOutputStageInfo &stage_info);
std::pair<int, int> get_min_max_values_from_quantized_data_type(DataType data_type);
} // namespace quantization
} // namespace arm_compute
#endif
