/*
 * C ABI of libl3kernels.so: MI355X (gfx950) kernels for the custom-operator hot path of
 * llama3-custom-inference -- split-KV decode attention with its log-sum-exp combine,
 * fused RMSNorm and fused rotary embedding.
 *
 * The three compute entry points replace the three host launchers the reference binds
 * in custom_kernels/main.cpp:2-8.  Conventions shared by all of them:
 *   - every pointer is a device pointer to bfloat16 (uint16 bit patterns) unless stated;
 *   - strides are in ELEMENTS, as torch reports them; the innermost dimension must be
 *     contiguous (the reference assumes it: custom_kernels.cu:44,55,401);
 *   - the library never allocates, frees or retains device memory: outputs and the
 *     attention workspace are caller-owned;
 *   - work is enqueued on the caller's `stream` (a hipStream_t; NULL = the null stream)
 *     and the call returns without synchronising (the reference launches on the legacy
 *     stream, custom_kernels.cu:274-275,386,439);
 *   - the return value is L3_OK or a negative L3_ERR_* code; argument checks run before
 *     any HIP call, so they can be exercised on a machine without a GPU.  Nothing here
 *     calls exit() (the reference's unused cudaCheck would: custom_kernels.cu:224-229).
 */
#ifndef L3_KERNELS_H
#define L3_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    L3_OK = 0,
    L3_ERR_NULL_POINTER = -1,   /* a required pointer is NULL */
    L3_ERR_HEAD_SIZE = -2,      /* head size not 64 or 128 (custom_kernels.cu:317-319) */
    L3_ERR_HEAD_RATIO = -3,     /* QH/KVH not one of 1,2,3,4,8 (custom_kernels.cu:289-291,312-314) */
    L3_ERR_SHAPE = -4,          /* a dimension is <= 0, too large, or QH is not a multiple of KVH */
    L3_ERR_STRIDE = -5,         /* a stride is negative or not a multiple of what the loads need */
    L3_ERR_ALIGNMENT = -6,      /* a base pointer is not aligned for the vector loads */
    L3_ERR_WORKSPACE = -7,      /* workspace NULL or smaller than l3_attn_decode_workspace_bytes */
    L3_ERR_SPLITS = -8,         /* num_splits negative or above L3_ATTN_MAX_SPLITS */
    L3_ERR_HIP = -9,            /* the HIP runtime reported an error at launch */
    L3_ERR_FLAGS = -10,         /* bits set in `flags` that this version does not define */
    L3_ERR_SCRATCH = -11,       /* l3_attn_decode_static: the problem needs more than L3_ATTN_STATIC_SCRATCH_BYTES */
    L3_ERR_SCALE = -12          /* attention: the softmax scale is not a positive finite number */
};

#define L3_ATTN_MAX_SPLITS 512

/* Library version: major*10000 + minor*100 + patch. */
int l3_version(void);

/* Static, NUL-terminated description of an error code (never NULL). */
const char* l3_strerror(int code);

/*
 * Per-call options of the attention entry points: the `flags` argument, 0 = the library's own
 * choices.  The library keeps no option between calls (no setter, no environment variable), so
 * calls from different threads cannot change each other's plan or workspace size; pass the same
 * flags to l3_attn_choose_splits / l3_attn_decode_workspace_bytes as to the call they size.
 *   L3_ATTN_FLAG_KERNEL_FMA  decode: the split-KV kernel built on FMA dot products on the vector
 *                            ALUs instead of the default MFMA tiles fed through LDS.  Both compute
 *                            the same thing; the flag exists so that the comparison can be repeated
 *                            (the reference has one kernel and no counterpart of this choice).
 *   L3_ATTN_FLAG_PREFILL_*   prefill: force one form of l3_attn_prefill instead of the choice by
 *                            prompt length -- WAVE (every wavefront streams K/V on its own), TILED (a
 *                            workgroup shares K/V tiles; forced, it is the kernel with two column blocks
 *                            per wavefront, where the library's own choice runs one for launches that
 *                            would leave much of the device empty) or TILED_NO_MAX (the tiled kernels whose
 *                            loop takes no maximum, whatever the size of the launch; left to itself
 *                            the library uses them for prompts of 4096 tokens or more in launches of more
 *                            workgroups than the device holds at once).  Same results within the stated
 *                            tolerance; for tests and timing.
 *   L3_ATTN_FLAG_WS_COUNTERS decode: the workspace starts with L3_ATTN_COUNTER_BYTES of arrival counters
 *                            that l3_attn_workspace_init prepared (see there); the library may then merge
 *                            the split partials inside the split launch instead of launching a combine.
 *   L3_ATTN_FLAG_TWO_LAUNCHES decode: always split kernel + combine kernel, also where the counters would
 *                            allow a single launch (for comparisons; same results).
 *   L3_ATTN_FLAG_FORM_*      decode with an explicit num_splits: run that count as cooperative workgroups
 *                            (COOP: a workgroup per (batch, kv head, split)) or streamed (STREAM, the default
 *                            for an explicit count: a wavefront per (batch, kv head, split)).  The automatic
 *                            plan chooses the form itself.
 * Any other bit, or both bits of the FORM field at once, gives L3_ERR_FLAGS.
 */
#define L3_ATTN_FLAG_KERNEL_FMA 0x1
#define L3_ATTN_FLAG_WS_COUNTERS 0x2
#define L3_ATTN_FLAG_FORM_COOP 0x4
#define L3_ATTN_FLAG_FORM_STREAM 0x8
#define L3_ATTN_FLAG_FORM_MASK 0xc
#define L3_ATTN_FLAG_TWO_LAUNCHES 0x40
#define L3_ATTN_FLAG_PREFILL_WAVE 0x10
#define L3_ATTN_FLAG_PREFILL_TILED 0x20
#define L3_ATTN_FLAG_PREFILL_TILED_NO_MAX 0x30
#define L3_ATTN_FLAG_PREFILL_MASK 0x30

/*
 * Split count the attention kernel would pick for this problem on a device with
 * `num_cus` compute units (<= 0: ask the current HIP device, 256 if there is none).
 * Pure integer host logic.  Replaces the fixed rule n_step = ceil(S / 64) of
 * custom_kernels.cu:243,251; the count is chosen so that the workgroups fill the device (one
 * per compute unit, three quarters of them when there are many sequences, a single split
 * where that saves the combine) while every split keeps at least one full tile of tokens.
 * Returns a value in [1, L3_ATTN_MAX_SPLITS], or a negative error code.
 */
int l3_attn_choose_splits(int B, int KVH, int S, int HD, int num_cus, int flags);

/*
 * Bytes of workspace l3_attn_decode needs for `num_splits` (0 = the automatic choice for
 * the current device).  0 when the plan has a single split (the kernel then writes the
 * output directly).  Replaces the three per-call temporaries of custom_kernels.cu:269-271
 * (tmp_result, score_maxes, softmax_sums); partial outputs are kept in float32 here.
 */
size_t l3_attn_decode_workspace_bytes(int B, int QH, int KVH, int S, int HD, int num_splits, int flags);

/*
 * out[b, h, :] = softmax(scale * q[b, h, :] . k[b, h / (QH/KVH), :, :]^T) @ v[b, h / (QH/KVH), :, :]
 *
 * Replaces flash_attention_decode(query, keys, values), custom_kernels.cu:233-338
 * (main.cpp:2,6), i.e. the split-KV kernel :13-177 followed by the combine kernel
 * :179-223, for one query token per sequence.
 *   q, out : (B, QH, 1, HD) bf16; q_strides / out_strides = {batch, head} strides
 *   k, v   : (B, KVH, S, HD) bf16; k_strides / v_strides = {batch, head, token} strides.
 *            Token rows must start on 16-byte boundaries (base pointers 16-byte aligned,
 *            strides multiples of 8, token stride below 2^24 elements).  q and out need
 *            16-byte aligned rows as well.
 *   scale  : softmax scale, positive and finite (L3_ERR_SCALE otherwise); the reference uses
 *            1/sqrt(HD) (custom_kernels.cu:253)
 *   num_splits : 0 = automatic, otherwise 1..L3_ATTN_MAX_SPLITS (the kernel may use fewer
 *            when S is short); results do not depend on it beyond float32 rounding
 *   workspace : >= l3_attn_decode_workspace_bytes(...) bytes, 256-byte aligned; may be NULL
 *            when that size is 0.  Contents on entry are ignored (with L3_ATTN_FLAG_WS_COUNTERS: except
 *            the counters at its start, see l3_attn_workspace_init); calls that share a workspace
 *            must not overlap in time.
 * Supported: HD in {64, 128}, QH/KVH in {1, 2, 3, 4, 8}, S >= 1.
 */
int l3_attn_decode(const void* q, const void* k, const void* v, void* out,
                   void* workspace, size_t workspace_bytes,
                   int B, int QH, int KVH, int S, int HD,
                   const int64_t q_strides[2], const int64_t k_strides[3],
                   const int64_t v_strides[3], const int64_t out_strides[2],
                   float scale, int num_splits, int flags, void* stream);

/*
 * Single-launch decode attention: prepares a workspace whose first L3_ATTN_COUNTER_BYTES hold the arrival
 * counters with which the split kernel itself merges the partials of a (batch, kv head) -- the workgroup
 * that finishes a head last does it, out of the L2 of the XCD all workgroups of that head were placed on --
 * so that no combine kernel is launched (the reference always launches two kernels: custom_kernels.cu:274-275).
 *   l3_attn_workspace_init  zeroes the counters on `stream` and, on the first call per device, runs a probe
 *       launch that confirms the placement rule the scheme rests on (the workgroups of a grid go to the 8
 *       XCDs in turn, so workgroups whose ids agree modulo 8 share an XCD) and WAITS for it: call it at set-up, outside stream capture.  workspace: 256-byte aligned, at least
 *       L3_ATTN_COUNTER_BYTES.  Every later l3_attn_decode / l3_attn_decode_devlen call on that workspace must
 *       pass L3_ATTN_FLAG_WS_COUNTERS (sizes from l3_attn_decode_workspace_bytes with the same flag); the
 *       counters are zero again when a call's kernels have finished, nothing else may write them, and calls
 *       that share a workspace must not overlap in time.  Where the probe did not confirm the rule, or the
 *       grid of a call does not keep a head on one XCD (B x KVH not a multiple of 8, more than 32 splits,
 *       a plan of streaming workgroups, more than 1023 (batch, kv head) pairs), the call runs split kernel + combine as without the flag.
 *   l3_attn_merge_in_launch_available  1 when the probe has confirmed the rule on the current device.
 *   l3_attn_launches  kernels an l3_attn_decode call with these arguments launches on the current device
 *       right now: 1 (a single split, or the merge inside the split launch) or 2 (split kernel + combine).
 *   l3_attn_placement_errors  number of (batch, kv head) merges whose arrivals did not all come from the
 *       merging workgroup's XCD since the counters were prepared (every arrival carries its XCC_ID; always 0
 *       on a device that passed the probe; a diagnostic that synchronises): workspace = a prepared workspace, or NULL for l3_attn_decode_static's array.
 */
#define L3_ATTN_COUNTER_BYTES (128u << 10)
int l3_attn_workspace_init(void* workspace, size_t workspace_bytes, void* stream);
int l3_attn_merge_in_launch_available(void);
int l3_attn_launches(int B, int QH, int KVH, int S, int HD, int num_splits, int flags);
int64_t l3_attn_placement_errors(const void* workspace);

/*
 * l3_attn_decode for callers that cannot allocate device memory and have no workspace to pass
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the
 * float32 partials and the arrival counters live in a static device array of
 * L3_ATTN_STATIC_SCRATCH_BYTES inside the library instead of a caller's workspace, and the call
 * allocates and frees nothing.  It has no counterpart in the reference, whose launcher allocates
 * three temporaries per call (custom_kernels.cu:269-271).  Same arguments, kernels and results (bit
 * for bit) as l3_attn_decode with L3_ATTN_FLAG_WS_COUNTERS on a workspace prepared by
 * l3_attn_workspace_init (the flag is implied here).  A problem whose plan needs more scratch than
 * the array holds returns L3_ERR_SCRATCH (size it with l3_attn_decode_workspace_bytes and that flag;
 * every BASELINE shape needs under 5 MiB).  Every GPU the library runs on holds its own copy of the
 * array from the first call on that GPU until the process ends; on that first call the address is
 * looked up and the placement probe of l3_attn_workspace_init runs (and is waited for), so make one
 * call outside stream capture first.  All calls on one GPU share the array: calls that overlap in
 * time on the same GPU (different streams or threads) race.  The counters at its start are zero when
 * the library is loaded and every call leaves them at zero; the partial rows need no clearing --
 * every row a merge reads was written by the same call -- so the previous call's contents are
 * simply overwritten.
 */
#define L3_ATTN_STATIC_SCRATCH_BYTES (16u << 20)
int l3_attn_decode_static(const void* q, const void* k, const void* v, void* out,
                          int B, int QH, int KVH, int S, int HD,
                          const int64_t q_strides[2], const int64_t k_strides[3],
                          const int64_t v_strides[3], const int64_t out_strides[2],
                          float scale, int num_splits, int flags, void* stream);

/*
 * l3_attn_decode with the KV length read from device memory at run time (*kv_len_dev, clamped to
 * [1, max_S]: a length below 1 attends to token 0 alone), so that one recorded launch -- a HIP graph node -- serves every step of a decode loop
 * whose cache grows by a token per step.  `k`/`v` are views of the whole cache row range
 * [0, max_S) with the usual {batch, head, token} strides; the split plan and the workspace are
 * sized for max_S.  No counterpart in the reference, whose KV length is the tensor shape
 * (custom_kernels.cu:246) and therefore fixed per launch.
 */
int l3_attn_decode_devlen(const void* q, const void* k, const void* v, void* out,
                          void* workspace, size_t workspace_bytes,
                          int B, int QH, int KVH, int max_S, int HD,
                          const int64_t q_strides[2], const int64_t k_strides[3],
                          const int64_t v_strides[3], const int64_t out_strides[2],
                          float scale, int num_splits, int flags, const int32_t* kv_len_dev, void* stream);

/*
 * Causal GQA attention for T > 1 query tokens per sequence (prompt prefill):
 *   out[b, h, i, :] = softmax_j<=p(i)( scale * q[b, h, i, :] . k[b, h/(QH/KVH), j, :] ) @ v[...],
 *   p(i) = S - T + i
 * i.e. query i sits at absolute position S - T + i of a cache that holds S >= T tokens.  For
 * S == T this is scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True), which
 * the reference calls for this case (model.py:114-116) instead of a kernel of its own.
 *   q, out : (B, QH, T, HD) bf16 with {batch, head, token} strides
 *   k, v   : (B, KVH, S, HD) bf16 with {batch, head, token} strides
 * Same head sizes, ratios and alignment rules as l3_attn_decode; no workspace.
 */
int l3_attn_prefill(const void* q, const void* k, const void* v, void* out, int B, int QH, int KVH, int T, int S,
                    int HD, const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                    const int64_t out_strides[3], float scale, int flags, void* stream);

/*
 * The two stages of l3_attn_decode on their own, for callers that hold one sequence's KV
 * cache in several pieces (e.g. token ranges on different GPUs): every piece runs the split
 * stage on its range, the partials are concatenated along the split axis, and one combine
 * finishes the row.  Together they replace the reference's two kernels one to one
 * (custom_kernels.cu:13-177 and :179-223); the reference has no host entry that runs them
 * separately.
 *
 * l3_attn_split: same inputs as l3_attn_decode; ALWAYS writes partials, even for one split:
 *   part_o  : (B, QH, n, HD) float32, sum_j 2^(s_j - m) v_j over the split's tokens, where
 *             s_j = scale * log2(e) * q.k_j  (scores in log2 units) and m = max_j s_j
 *   part_ml : (B, QH, n, 2) float32, the pair (m, sum_j 2^(s_j - m))
 *   Returns n >= 1, the number of splits actually used (<= the requested count; the caller
 *   sizes both buffers for the requested count, or for l3_attn_choose_splits when 0), or a
 *   negative error code.
 * l3_attn_combine: out[b, h, :] = sum_i part_o_i 2^(m_i - M) / sum_i l_i 2^(m_i - M),
 *   M = max_i m_i, over i < n; out is (B, QH, 1, HD) bf16 with {batch, head} strides.
 *   1 <= n <= L3_ATTN_MAX_SPLITS.
 */
int l3_attn_split(const void* q, const void* k, const void* v, float* part_o, float* part_ml,
                  int B, int QH, int KVH, int S, int HD,
                  const int64_t q_strides[2], const int64_t k_strides[3], const int64_t v_strides[3],
                  float scale, int num_splits, int flags, void* stream);
int l3_attn_combine(const float* part_o, const float* part_ml, void* out, int B, int QH, int HD, int n,
                    const int64_t out_strides[2], void* stream);

/*
 * y[r, :] = bf16( x[r, :] * rsqrt(mean(x[r, :]^2) + eps) * w[:] ), float32 inside, one rounding.
 *
 * Replaces rms_norm(input, weight, eps), custom_kernels.cu:369-389 (kernel :340-367,
 * main.cpp:3,7).  x and y are `rows` contiguous rows of C bf16 values (the reference
 * indexes its (B, T, C) input as contiguous: custom_kernels.cu:355), w is C bf16 values.
 * Any C >= 1; rows of C % 8 == 0 with 16-byte aligned pointers take the vector path.
 */
int l3_rms_norm(const void* x, const void* w, void* y, int64_t rows, int C, float eps, void* stream);

/*
 * Residual addition fused with the RMSNorm that follows it in a transformer block
 * (model.py:147-148: x = x + attn(...), then ln_2(x); likewise before the next block's ln_1 and
 * before ln_f):
 *   sum_out[r, :] = bf16( x[r, :] + residual[r, :] )
 *   y[r, :]       = rms_norm(sum_out[r, :], w, eps)          (of the rounded sum)
 * so that (sum_out, y) carry the same bits as a bf16 tensor addition followed by l3_rms_norm.
 * Layout and fast-path rules as for l3_rms_norm; sum_out may alias x or residual, y must not.
 * One launch and one pass over the row instead of two launches and three passes.  The
 * reference has no counterpart (it adds with a separate torch kernel).
 */
int l3_add_rms_norm(const void* x, const void* residual, const void* w, void* sum_out, void* y, int64_t rows,
                    int C, float eps, void* stream);

/*
 * y[i] = bf16( bf16(silu(a[i])) * b[i] ) over n contiguous bf16 values: the SwiGLU elementwise
 * product of model.py:134, F.silu(c_fc2(x)) * c_fc(x), in one launch with the same two roundings
 * as the two torch kernels.  No counterpart among the reference's kernels.
 */
int l3_silu_mul(const void* a, const void* b, void* y, int64_t n, void* stream);

/*
 * l3_silu_mul on row-strided operands: y[r][j] = silu(a[r][j]) * b[r][j] for rows x cols elements,
 * a and b with the given row strides (elements), y dense.  For the two halves of one fused
 * gate|up projection (a = first half, b = second half, both strides 2 * cols).  cols and the
 * strides multiples of 8, pointers 16-byte aligned.
 */
int l3_silu_mul_rows(const void* a, const void* b, void* y, int64_t rows, int64_t cols, int64_t a_row_stride,
                     int64_t b_row_stride, void* stream);

/*
 * y[M, N] = x[M, K] . w[N, K]^T for the few activation rows of a decode step: bf16 in and out,
 * float32 accumulation, one rounding.  Stands where the reference calls nn.Linear with T == 1
 * (model.py:95 c_attn, :121 c_proj, :134 mlp c_proj, :225 lm_head); hipBLASLt treats these as
 * GEMMs, this entry point as a single pass over the weight matrix at HBM speed.
 * 1 <= M <= L3_LINEAR_MAX_ROWS (one 16-column block of the matrix instruction); N % 4 == 0; K % 32 == 0;
 * strides are row strides in elements (x_stride, w_stride >= K and multiples of 8; y_stride >= N and a
 * multiple of 4); x and w 16-byte aligned, y 8-byte aligned.  Needs no workspace.  For 17 .. 64 rows use
 * l3_linear_splitk (matrices of a few thousand rows) or a library GEMM (larger ones).
 */
#define L3_LINEAR_MAX_ROWS 16
int l3_linear_decode(const void* x, const void* w, void* y, int M, int N, int K, int64_t x_stride,
                     int64_t w_stride, int64_t y_stride, void* stream);

/*
 * y[M, N] = silu(x . w_gate^T) * (x . w_up^T) in one pass over both weight matrices: the
 * SwiGLU front half of model.py:134 (F.silu(c_fc2(x)) * c_fc(x)).  Both products and the silu
 * are rounded to bf16 before the multiplication, as the three separate torch operators do.
 * Same constraints as l3_linear_decode; w_gate and w_up share w_stride.
 */
int l3_linear_swiglu_decode(const void* x, const void* w_gate, const void* w_up, void* y, int M, int N, int K,
                            int64_t x_stride, int64_t w_stride, int64_t y_stride, void* stream);

/*
 * l3_linear_decode with what a transformer block does around its linears folded in; each of
 * norm_weight, w_up and residual may be NULL:
 *   h = norm_weight ? bf16(x * rsqrt(mean(x^2) + norm_eps) * norm_weight) : x     (model.py:70-72 in front of
 *                                                                                 c_attn / the MLP / lm_head)
 *   t = w_up ? bf16(silu(bf16(h.w^T))) * bf16(h.w_up^T) : h.w^T                   (model.py:134)
 *   y = residual ? bf16(residual + bf16(t)) : bf16(t)                             (model.py:147-148)
 * with the rounding points of the separate operators.  residual has y's shape and row stride and
 * may be y itself.  The input norm stages x in LDS and needs K % 512 == 0 and M * (K + 8) <= 24576
 * (L3_ERR_SHAPE otherwise); everything else as for l3_linear_decode.
 */
int l3_linear_decode_fused(const void* x, const void* norm_weight, float norm_eps, const void* w, const void* w_up,
                           const void* residual, void* y, int M, int N, int K, int64_t x_stride, int64_t w_stride,
                           int64_t y_stride, void* stream);

/*
 * The fused qkv projection of a decode step with what follows it folded in (model.py:95-106 for
 * one new token per sequence): qkv = [rms_norm(x, norm_weight)] . w_qkv^T with N = (NH + 2 KVH) HD
 * outputs in q | k | v order, rounded to bf16; the query and key heads are rotated with row *pos_dev
 * of freq_table ((table_rows, HD) float32, interleaved cos/sin); rotated keys and the values go
 * into cache_k / cache_v at token *pos_dev (element strides cache_strides = {batch, token},
 * (KVH, HD) contiguous), the rotated queries to q_out (B, NH, HD).  One launch where the separate
 * operators take l3_linear_decode_fused and l3_rot_embed_append, with the same bits.  Constraints
 * of both apply (B <= 16, K % 32 == 0, HD % 8 == 0, norm limits as above); an
 * out-of-range position writes nothing.
 */
int l3_linear_qkv_rope_append(const void* x, const void* norm_weight, float norm_eps, const void* w_qkv,
                              const float* freq_table, void* q_out, void* cache_k, void* cache_v,
                              const int32_t* pos_dev, int B, int NH, int KVH, int HD, int K, int64_t x_stride,
                              int64_t w_stride, const int64_t cache_strides[2], int cache_len, int table_rows,
                              void* stream);

/*
 * Split-K form of l3_linear_decode for 17 .. 64 activation rows (hipBLASLt's territory in the
 * reference: nn.Linear at batch 64, model.py:95,121,134).  Eight wavefronts of a workgroup share
 * the activations of one k range through LDS and take 128 weight rows (64, with the k range halved
 * among them, for small matrices); K is split `ksplit` ways across workgroups, each covering at
 * most 512 (1024) k, and split s writes its float32 partial products
 * to part[s][m][n] (M x N floats per split, contiguous).  The splits are NOT added up here: the
 * elementwise operator that follows the linear in a decode step does that on its way
 * (l3_add_rms_norm_partials, l3_rot_embed_append_partials), in split order, without atomics;
 * l3_linear_splitk_finish does it where there is no such operator.
 * l3_linear_splitk_plan returns the split count for a device with num_cus compute units (<= 0: the
 * current device); l3_linear_splitk_workspace_bytes the size of `part`.  1 <= M <=
 * L3_LINEAR_SPLITK_MAX_ROWS, N % 8 == 0, K % 128 == 0, ceil((K / 128) / ksplit) <= 4 (<= 8 for a matrix
 * with fewer than 32 rows per compute unit, which gets 64-row workgroups); strides and
 * alignment as for l3_linear_decode.  Meant for matrices of a few thousand rows, where the split
 * count fills the device; for a matrix whose rows alone do (a vocabulary projection), every split
 * costs M x N floats of traffic and a library GEMM is the better tool.
 */
#define L3_LINEAR_SPLITK_MAX_ROWS 64
int l3_linear_splitk_plan(int N, int K, int num_cus);
size_t l3_linear_splitk_workspace_bytes(int M, int N, int ksplit);
int l3_linear_splitk(const void* x, const void* w, void* part, size_t part_bytes, int M, int N, int K,
                     int64_t x_stride, int64_t w_stride, int ksplit, void* stream);

/*
 * y[m][n] = bf16(sum over the splits of part[s][m][n]), or bf16(residual + that) with the two
 * roundings of a separate addition when residual (same shape and row stride as y, may be y) is not
 * NULL: finishes l3_linear_splitk on its own.  N % 8 == 0, y_stride >= N and a multiple of 8,
 * pointers 16-byte aligned.
 */
int l3_linear_splitk_finish(const void* part, int ksplit, const void* residual, void* y, int M, int N,
                            int64_t y_stride, void* stream);

/*
 * l3_add_rms_norm whose residual operand is a split-K linear's partial products (`part`,
 * ksplit x rows x C floats): r = bf16(sum of the splits), sum_out = bf16(x + r),
 * y = rms_norm(sum_out): sum_out has the bits of the unsplit sequence given the same r; y agrees
 * with l3_rms_norm of it to one bf16 ulp (the squares are added in another order).  C % 8 == 0,
 * C <= 8192; all pointers 16-byte aligned.
 */
int l3_add_rms_norm_partials(const void* x, const void* part, int ksplit, const void* w, void* sum_out, void* y,
                             int rows, int C, float eps, void* stream);

/*
 * l3_rot_embed_append whose fused qkv projection is a split-K linear's partial products (`part`,
 * ksplit x B x (NH + 2 KVH) HD floats), added up and rounded to bf16 first.
 */
int l3_rot_embed_append_partials(const void* part, int ksplit, const float* freq_table, void* q_out, void* cache_k,
                                 void* cache_v, const int32_t* pos_dev, int B, int NH, int KVH, int HD,
                                 const int64_t cache_strides[2], int cache_len, int table_rows, void* stream);

/*
 * out[r] = index of the first maximum of the bf16 row logits[r*row_stride : r*row_stride + V]
 * (int64; a NaN counts as the maximum and the first one wins, as in torch.argmax): the greedy pick of model.py:371.  Two small
 * launches (per-chunk maxima into the caller's workspace of l3_argmax_workspace_bytes(rows, V)
 * bytes, then one merge per row).  rows <= 65535.  No counterpart among the reference's kernels.
 */
size_t l3_argmax_workspace_bytes(int rows, int V);
int l3_argmax(const void* logits, int64_t row_stride, int rows, int V, void* workspace, size_t workspace_bytes,
              int64_t* out, void* stream);

/*
 * One greedy decoding step's tail on the device: the argmax of every logits row, then the
 * bookkeeping of the reference's generate() loop (model.py:371-378) with next = *pos + 1
 * (clamped to total_len - 1):
 *   nxt = text_mask[b][next] ? tokens[b][next] : argmax(logits[b])
 *   tokens[b][next] = nxt;  tok[b] = nxt;  eos[b] |= !text_mask[b][next] && nxt in stop_tokens
 * and finally *pos += 1, *kv_len += 1.  tokens (rows, total_len) int64 and text_mask (rows,
 * total_len) one byte per element, both contiguous; tok (rows) int64; eos (rows) one byte per
 * element; pos, kv_len device int32.  Workspace as for l3_argmax.  With every operand in device
 * memory the step can be replayed from a HIP graph.
 */
int l3_greedy_step(const void* logits, int64_t row_stride, int rows, int V, void* workspace, size_t workspace_bytes,
                   int64_t* tokens, const uint8_t* text_mask, int64_t total_len, int64_t* tok, int32_t* pos,
                   int32_t* kv_len, uint8_t* eos, const int64_t* stop_tokens, int n_stop, void* stream);

/*
 * Rotary embedding on adjacent pairs:
 *   y[b,t,h,2i]   = bf16( x[b,t,h,2i] * freq[t,2i] - x[b,t,h,2i+1] * freq[t,2i+1] )
 *   y[b,t,h,2i+1] = bf16( x[b,t,h,2i] * freq[t,2i+1] + x[b,t,h,2i+1] * freq[t,2i] )
 *
 * Replaces rot_embed(input, freq), custom_kernels.cu:418-442 (kernel :391-416,
 * main.cpp:4,8).  x is (B, T, NH, HD) bf16 with x_strides = {batch, token, head} strides
 * (q and k arrive as views into the fused qkv projection: model.py:96-97); freq is a
 * contiguous (T, HD) float32 table of interleaved cos/sin (model.py:59-60); y is a
 * CONTIGUOUS (B, T, NH, HD) bf16 tensor, as the reference writes it
 * (custom_kernels.cu:414).  HD must be even; pairs must be 4-byte aligned.  16-byte
 * aligned rows with HD % 8 == 0 take the vector path.
 */
int l3_rot_embed(const void* x, const float* freq, void* y, int B, int T, int NH, int HD,
                 const int64_t x_strides[3], void* stream);

/*
 * Decode-step fusion of the two rot_embed calls and the two KV-cache slice assignments of
 * model.py:100-106 for ONE new token per sequence, with the position read from device memory
 * (*pos_dev) so that the launch can be replayed from a HIP graph:
 *   q_out[b, 0, h, :]            = rope(qkv[b, h*HD : (h+1)*HD], freq_table[pos])            h < NH
 *   cache_k[b, pos, h, :]        = rope(qkv[b, (NH+h)*HD : ...], freq_table[pos])            h < KVH
 *   cache_v[b, pos, h, :]        = qkv[b, (NH+KVH+h)*HD : ...]                               h < KVH
 * qkv is the fused projection output (B, 1, (NH+2*KVH)*HD) bf16 in the q|k|v order of
 * model.py:96 with `qkv_batch_stride` elements between rows; freq_table is the whole
 * (table_rows, HD) float32 cos/sin table; q_out is contiguous (B, 1, NH, HD); the caches are
 * (maxB, cache_len, KVH, HD) with cache_strides = {batch, token} strides.  HD % 8 == 0, 16-byte
 * aligned rows.  A position outside [0, min(cache_len, table_rows)) writes nothing.
 * The rotation arithmetic is that of l3_rot_embed.  No counterpart in the reference.
 */
int l3_rot_embed_append(const void* qkv, const float* freq_table, void* q_out, void* cache_k, void* cache_v,
                        const int32_t* pos_dev, int B, int NH, int KVH, int HD, int64_t qkv_batch_stride,
                        const int64_t cache_strides[2], int cache_len, int table_rows, void* stream);

/*
 * Measurement yardstick, not an operator: reads `bytes` (a multiple of 16, 16-byte aligned) of
 * device memory once with 16-byte loads from `workgroups` 512-thread workgroups (<= 0: four per
 * compute unit), all workgroups together sweeping the buffer front to back.  The loads are kept
 * alive by xor-ing what they return; the xor goes to `sink` (4 bytes, device memory) only when it
 * equals a constant that no realistic input produces, so the kernel writes nothing.  Timed by the
 * benchmark over buffers larger than the memory-side cache, it gives the read bandwidth this
 * device delivers to a pure stream: the ceiling every HBM-bound kernel here is read against.
 * No counterpart in the reference.
 */
int l3_hbm_read_stream(const void* src, size_t bytes, void* sink, int workgroups, void* stream);

/*
 * The second yardstick: the same sweep, but every 16 bytes read from `src` are written once to `dst`
 * (both 16-byte aligned, `bytes` a multiple of 16, no overlap): `bytes` read plus `bytes` written per
 * launch, which is the traffic of a row-wise operator such as the RMSNorm and the rotary embedding.
 * block_kib: what a workgroup moves per trip, 8, 16, 32 or 64 KiB (0 = 64); which is fastest depends on
 * how the buffer divides over the compute units, so the benchmark takes the best of the four.
 * No counterpart in the reference.
 */
int l3_hbm_rw_stream(const void* src, void* dst, size_t bytes, int workgroups, int block_kib, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* L3_KERNELS_H */
