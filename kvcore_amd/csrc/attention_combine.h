// Joining the partial results of attention over parts of a row's keys; shared by the
// kernels for single tokens and for portions of prompts.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "device_utils.h"

namespace kvc {

constexpr int kMaxAttentionSplits = 64;

// out[row, :] = sum_s w_s * part_o[row, s, :] / sum_s w_s * l_s with w_s = exp2(m_s - max_s m_s),
// for part_o [rows, nsplit, d] float32 and part_ml [rows, nsplit, 2] = (m_s, l_s): the sums
// of a split are relative to its own m_s, which is in the exponent's units (base 2).
int launch_attention_combine(bf16_t* out, const float* part_o, const float* part_ml, int64_t rows,
                             int d, int nsplit, hipStream_t stream);

}  // namespace kvc
