// Host-side declarations shared by the C-ABI layer and the kernel launchers.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/l3_kernels.h"

namespace l3 {

// How one decode-attention call is cut into workgroups.  The reference fixes 64 tokens per
// workgroup (custom_kernels.cu:243,251); here the cut depends on the problem and device.
struct AttnPlan {
    int num_splits;        // workgroups per (batch, kv head)
    int tokens_per_split;  // multiple of the workgroup tile, except that the last split is shorter
};

// Tokens one workgroup consumes per main-loop trip (4 waves x 8 KiB of K+V each).
constexpr int attn_block_tile_tokens(int HD) { return HD == 128 ? 64 : 128; }

// Pure integer logic (no HIP): the plan for `requested` splits (0 = automatic).
AttnPlan attn_make_plan(int B, int KVH, int S, int HD, int requested, int num_cus);

// Compute units of the current device, 256 when no device can be queried.
int current_device_cus();

struct AttnParams {
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    uint16_t* out;
    float* part_o;    // [B][QH][num_splits][HD] unnormalised partial outputs
    float2* part_ml;  // [B][QH][num_splits] (max in log2 units, sum of exp2)
    int B, QH, KVH, S;
    int num_splits, tokens_per_split;
    int64_t q_sb, q_sh;
    int64_t k_sb, k_sh, k_st;
    int64_t v_sb, v_sh, v_st;
    int64_t o_sb, o_sh;
    float scale_log2e;
};

// Launchers: return a hipError_t cast to int (0 = success).
int launch_attn_decode(const AttnParams& p, int HD, int R, hipStream_t stream);
int launch_rms_norm(const uint16_t* x, const uint16_t* w, uint16_t* y, int64_t rows, int C, float eps,
                    bool vec_ok, hipStream_t stream);
int launch_rot_embed(const uint16_t* x, const float* freq, uint16_t* y, int B, int T, int NH, int HD,
                     int64_t sb, int64_t st, int64_t sh, bool vec_ok, hipStream_t stream);

}  // namespace l3
