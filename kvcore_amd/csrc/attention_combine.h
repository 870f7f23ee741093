// Joining the partial results of attention over parts of a row's keys; shared by the
// kernels for single tokens and for portions of prompts.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "device_utils.h"

namespace kvc {

constexpr int kMaxAttentionSplits = 64;

// An attention result on its way out: bfloat16, or (f32) the float32 value itself into the same
// place of a float32 array.
__device__ __forceinline__ void store_result(bf16_t* out, int64_t index, float value, int f32) {
  if (f32) reinterpret_cast<float*>(out)[index] = value;
  else out[index] = from_float<bf16_t>(value);
}

// out[row, :] = sum_s w_s * part_o[row, s, :] / sum_s w_s * l_s with w_s = exp2(m_s - max_s m_s),
// for part_o [rows, nsplit, d] float32 and part_ml [rows, nsplit, 2] = (m_s, l_s): the sums
// of a split are relative to its own m_s, which is in the exponent's units (base 2).
// out_f32: out receives float32 values instead of bfloat16.
int launch_attention_combine(bf16_t* out, const float* part_o, const float* part_ml, int64_t rows,
                             int d, int nsplit, int out_f32, hipStream_t stream);

}  // namespace kvc
