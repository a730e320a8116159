// Host-side declarations shared by the C-ABI layer and the kernel launchers.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/l3_kernels.h"

namespace l3 {

// How one decode-attention call is cut up.  The reference fixes 64 tokens per workgroup
// (custom_kernels.cu:243,251); here the cut depends on the problem and the device.
struct AttnPlan {
    int num_splits;        // token ranges per (batch, kv head); each yields one partial per query head
    int tokens_per_split;  // multiple of the kernel's tile, except that the last split is shorter
    bool coop;             // MFMA kernel only: whole workgroup on one (batch, kv head, split) -- short sequences
};

// The two split-KV kernels: FMA dot products on the vector ALUs, or MFMA tiles fed through LDS.
constexpr int kAttnImplFma = 0;
constexpr int kAttnImplMfma = 1;

constexpr int kMfmaWaves = 8;  // wavefronts per workgroup of the MFMA kernel

// K/V token strides (elements) must stay below this: the MFMA kernels address the rows of a tile
// (at most 64 tokens) with 32-bit byte offsets from the tile's first token.
constexpr int64_t kAttnMaxTokenStride = int64_t(1) << 24;

// Granularity of a split in tokens.  FMA kernel: one main-loop trip of its 4-wave workgroup
// (4 x 8 KiB of K+V).  MFMA kernel: one tile of a wavefront (16 KiB of K+V).
constexpr int attn_tile_tokens(int HD, int impl) {
    return impl == kAttnImplMfma ? (HD == 128 ? 32 : 64) : (HD == 128 ? 64 : 128);
}

// Adjacent kv heads that share a workgroup of the MFMA kernel (largest power of two <= 8 dividing KVH).
int attn_mfma_heads_per_wg(int KVH);

// Pure integer logic (no HIP): the plan for `requested` splits (0 = automatic).
// `form`: L3_ATTN_FLAG_FORM_* bits of the call (which form a requested count is run in);
// `merge_in_launch`: the call can merge inside the split launch where the grid allows it.
AttnPlan attn_make_plan(int B, int KVH, int S, int HD, int requested, int num_cus, int impl, int form = 0,
                        bool merge_in_launch = false);

// Compute units of the current device, 256 when no device can be queried.
int current_device_cus();

// What a wavefront needs before it can issue its first K/V load comes first, so that it sits in the
// first 64 bytes of the kernel arguments (one scalar-cache miss instead of three in a row).
struct AttnParams {
    int B, QH, KVH, S;
    int num_splits, tokens_per_split;
    const int* seqlen_dev;  // when set, the KV length is read from here (<= S, which then only bounds the plan)
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    int64_t k_sb, k_sh, k_st;
    int64_t v_sb, v_sh, v_st;
    int64_t q_sb, q_sh;
    float scale_log2e;
    uint16_t* out;
    float* part_o;    // [B][QH][num_splits][HD] unnormalised partial outputs; null = write `out` directly
    float2* part_ml;  // [B][QH][num_splits] (max in log2 units, sum of exp2)
    int64_t o_sb, o_sh;
    // Single-launch form of the MFMA kernel: arrival counters, one per (batch, kv head) at a stride of
    // kAttnArriveStride words, all zero between launches; null = partials only, a combine launch follows.
    unsigned* arrive;
};

// The counters sit a cache line apart (units on different XCDs never share a line); the last slot
// counts workgroups that found themselves on another XCD than their id implies (a diagnostic).
constexpr int kAttnArriveStride = 32;
constexpr int kAttnArriveSlots = int(L3_ATTN_COUNTER_BYTES / (kAttnArriveStride * sizeof(unsigned)));
constexpr int kAttnDiagSlot = kAttnArriveSlots - 1;

struct PrefillParams {
    const uint16_t* q;   // (B, QH, T, HD) with {batch, head, token} strides
    const uint16_t* k;   // (B, KVH, S, HD)
    const uint16_t* v;
    uint16_t* out;       // (B, QH, T, HD) with {batch, head, token} strides
    int B, QH, KVH, T, S;
    int64_t q_sb, q_sh, q_st;
    int64_t k_sb, k_sh, k_st;
    int64_t v_sb, v_sh, v_st;
    int64_t o_sb, o_sh, o_st;
    float scale_log2e;
    int snake;   // tiled form: ranks per round of the reversed-every-second-round order, 0 = plain (set by the launcher)
    int no_max_tiles;   // tiled form, head size 64: the tiles that take no maximum also for launches the device holds at once
    int auto_form;      // the form was the library's choice (it may then run one column block per wavefront)
};

struct LinearParams {
    const uint16_t* x;    // (M, K) activations, row stride x_stride
    const uint16_t* w0;   // (N, K) weights, row stride w_stride
    const uint16_t* w1;   // second weight matrix of the SwiGLU form (else null)
    const uint16_t* norm_w;  // (K) RMSNorm weight applied to x first (else null)
    const uint16_t* res;     // (M, N) residual added to the product, y's row stride (else null)
    float norm_eps;
    uint16_t* y;          // (M, N), row stride y_stride
    int M, N, K;
    int64_t x_stride, w_stride, y_stride;
    int sk;               // wavefronts that split K for one block of 16 weight rows (set by the launcher)
    // fused qkv projection of a decode step (rope_table != null): the N = (NH + 2 KVH) HD outputs of
    // activation row b are rotated at position *rope_pos and go to q_out / the KV cache instead of y
    const float* rope_table;   // (table_rows, HD) interleaved cos/sin
    const int* rope_pos;
    uint16_t* q_out;           // (M, NH, HD)
    uint16_t* cache_k;         // element strides c_sb (batch), c_st (token); (KVH, HD) contiguous
    uint16_t* cache_v;
    int NH, KVH, HD, cache_len, table_rows;
    int64_t c_sb, c_st;
};

// Launchers: return a hipError_t cast to int (0 = success).
int linear_skinny_plan(int N, int K, int waves_per_wg, int num_cus, int rows_per_wave, int kstep);
bool linear_skinny_can_stage(int M, int K);
int linear_splitk_plan(int N, int K, int num_cus);
int launch_add_rms_norm_partials(const uint16_t* x, const float* part, int ksplit, int64_t split_stride,
                                 const uint16_t* w, uint16_t* sum_out, uint16_t* y, int rows, int C, float eps,
                                 hipStream_t stream);
int launch_rot_embed_append_partials(const float* part, int ksplit, int64_t split_stride, const float* table,
                                     uint16_t* q_out, uint16_t* cache_k, uint16_t* cache_v, const int* pos_dev, int B,
                                     int NH, int KVH, int HD, int64_t c_sb, int64_t c_st, int cache_len,
                                     int table_rows, hipStream_t stream);
int linear_splitk_max_chunks(int N, int num_cus);
int launch_linear_splitk(const uint16_t* x, const uint16_t* w, float* part, int M, int N, int K, int64_t x_stride,
                         int64_t w_stride, int ksplit, int num_cus, hipStream_t stream);
int launch_linear_splitk_finish(const float* part, int ksplit, const uint16_t* res, uint16_t* y, int M, int N,
                                int64_t y_stride, hipStream_t stream);
int launch_linear_skinny(LinearParams p, bool swiglu, int num_cus, hipStream_t stream);
int launch_attn_prefill(const PrefillParams& p, int HD, hipStream_t stream);        // a wavefront per column group
// Workgroups of the tiled prefill kernel: 16-column blocks per wavefront, wavefronts per workgroup
// (small workgroups, several per compute unit).
constexpr int kPrefillColBlocks = 2;
constexpr int kPrefillTiledWaves = 4;
constexpr int prefill_tiled_positions_per_wg(int R) { return kPrefillTiledWaves * kPrefillColBlocks * (16 / R); }
int launch_attn_prefill_tiled(const PrefillParams& p, int HD, hipStream_t stream);  // K/V tiles shared by a workgroup
int launch_attn_splitkv_fma(const AttnParams& p, int HD, int R, hipStream_t stream);
int launch_attn_splitkv_mfma(const AttnParams& p, int HD, int R, bool coop, hipStream_t stream);
// producer_groups: head groups per batch entry of the streaming MFMA split kernel that wrote the partials (its
// grid's x extent), 0 when another kernel or a caller produced them
int launch_attn_combine(const AttnParams& p, int HD, int producer_groups, hipStream_t stream);
// True when every workgroup of a (batch, kv head) of the MFMA kernel's grid has the same linear id modulo 8
// (runs on one XCD) and the counters suffice: the condition for merging inside the split launch.
bool attn_mfma_can_merge_in_launch(int B, int KVH, bool coop, int num_splits);
// Writes the XCD each of `n` workgroups of a 1-D grid ran on to where[i * stride_words]; and a zero fill.
int launch_xcd_probe(unsigned* where, int n, int stride_words, hipStream_t stream);
int launch_fill_zero_u32(unsigned* dst, size_t n, hipStream_t stream);
int launch_hbm_read_stream(const void* src, size_t bytes, void* sink, int workgroups, hipStream_t stream);
int launch_hbm_rw_stream(const void* src, void* dst, size_t bytes, int workgroups, int block_kib, hipStream_t stream);
int launch_rms_norm(const uint16_t* x, const uint16_t* w, uint16_t* y, int64_t rows, int C, float eps,
                    bool vec_ok, hipStream_t stream);
int launch_add_rms_norm(const uint16_t* x, const uint16_t* res, const uint16_t* w, uint16_t* sum_out, uint16_t* y,
                        int64_t rows, int C, float eps, bool vec_ok, hipStream_t stream);
int launch_silu_mul_rows(const uint16_t* a, const uint16_t* b, uint16_t* y, int64_t rows, int64_t cols,
                         int64_t a_row_stride, int64_t b_row_stride, hipStream_t stream);
int launch_silu_mul(const uint16_t* a, const uint16_t* b, uint16_t* y, int64_t n, bool vec_ok, hipStream_t stream);
constexpr int kArgmaxChunk = 2048;  // logits one workgroup of the first argmax stage scans
int argmax_parts(int V);
int launch_argmax(const uint16_t* logits, int64_t row_stride, int rows, int V, float* part_val, int* part_idx,
                  int64_t* out, hipStream_t stream);
int launch_greedy_step(const uint16_t* logits, int64_t row_stride, int rows, int V, float* part_val, int* part_idx,
                       int64_t* tokens, const uint8_t* text_mask, int64_t total_len, int64_t* tok, int* pos,
                       int* kv_len, uint8_t* eos, const int64_t* stop, int n_stop, hipStream_t stream);
int launch_rot_embed(const uint16_t* x, const float* freq, uint16_t* y, int B, int T, int NH, int HD,
                     int64_t sb, int64_t st, int64_t sh, bool vec_ok, hipStream_t stream);
int launch_rot_embed_append(const uint16_t* qkv, const float* table, uint16_t* q_out, uint16_t* cache_k,
                            uint16_t* cache_v, const int* pos_dev, int B, int NH, int KVH, int HD, int64_t qkv_sb,
                            int64_t c_sb, int64_t c_st, int cache_len, int table_rows, hipStream_t stream);

}  // namespace l3
