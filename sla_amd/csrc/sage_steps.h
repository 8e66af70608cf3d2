// What the linear branch's state build hands to the FP8 quantiser of v when both run in one call
// (sla_linear_state_quant_v_fwd): the largest |v| of every column per slice of the sequence.
#pragma once
#include "common.h"

namespace sla {

// v_scale = max over the `nparts` partial maxima / v_range, then v_fp8 = e4m3(v / v_scale): the second and third
// step of sage_quant_v (reference SageSLA/core.py:127-129), on `st`.  `part` is [BH][nparts][D] fp32.
int quant_v_from_partial_amax(const void* v, const RowLayout& lay, int dtype, int BH, int L, int D, const float* part,
                              int nparts, uint8_t* v_fp8, float* v_scale, float v_range, hipStream_t st);
int validate_v_range(float v_range);

}  // namespace sla
