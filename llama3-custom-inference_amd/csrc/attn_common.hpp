// Pieces shared by the attention kernels: constants and the parameter block.
#pragma once

#include "l3_device.hpp"
#include "l3_host.hpp"

namespace l3 {

constexpr float kMaskedScore = -1.0e30f;  // finite stand-in for -inf (differences stay defined)
constexpr int kAttnMaxRatio = 8;          // query heads per kv head the kernels are sized for

// Row of the partial buffers that belongs to (batch b, query head qh, split).
__device__ __forceinline__ int64_t attn_partial_row(const AttnParams& p, int b, int qh, int split) {
    return (int64_t(b) * p.QH + qh) * p.num_splits + split;
}

}  // namespace l3
