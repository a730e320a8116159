// C ABI of libl3kernels.so: argument checks, split planning and dispatch.  Every check runs
// before the first HIP call so the error paths can be driven on a machine without a GPU.
// Takes the place of the host launchers flash_attention_decode / rms_norm / rot_embed
// (custom_kernels.cu:233-338, 369-389, 418-442) and of the pybind table in main.cpp:5-9.
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include <algorithm>

#include "l3_host.hpp"

namespace l3 {

namespace {

constexpr int kVersion = 100;  // 0.1.0
constexpr size_t kWorkspaceAlign = 256;

bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }
// The kernels track the maximum of the raw scores and scale it afterwards, which needs a positive scale.
bool scale_ok(float scale) { return scale > 0.0f && scale <= 3.0e38f; }

bool ratio_supported(int R) { return R == 1 || R == 2 || R == 3 || R == 4 || R == 8; }

int ceil_div(int a, int b) { return (a + b - 1) / b; }

size_t round_up(size_t n, size_t a) { return (n + a - 1) / a * a; }

int check_attn_shape(int B, int QH, int KVH, int S, int HD) {
    if (HD != 64 && HD != 128) return L3_ERR_HEAD_SIZE;
    if (B <= 0 || QH <= 0 || KVH <= 0 || S <= 0) return L3_ERR_SHAPE;
    if (QH % KVH != 0) return L3_ERR_SHAPE;
    if (!ratio_supported(QH / KVH)) return L3_ERR_HEAD_RATIO;
    // grid = B * KVH * splits workgroups and B * QH combine workgroups must fit 31 bits
    if (int64_t(B) * QH * L3_ATTN_MAX_SPLITS >= (int64_t(1) << 31)) return L3_ERR_SHAPE;
    return L3_OK;
}

// With `counters` the workspace starts with the arrival counters of the single-launch form.
size_t attn_workspace_bytes(int B, int QH, int HD, int num_splits, bool counters) {
    if (num_splits <= 1) return 0;
    const size_t rows = size_t(B) * size_t(QH) * size_t(num_splits);
    return (counters ? size_t(L3_ATTN_COUNTER_BYTES) : 0) + round_up(rows * HD * sizeof(float), kWorkspaceAlign) +
           round_up(rows * sizeof(float2), kWorkspaceAlign);
}

}  // namespace

// Scratch of l3_attn_decode_static: the float32 partials and their (max, sum) pairs live in this
// array instead of a caller's workspace.  Every device the library runs on holds its own copy at
// its own address for the life of the process; in host code the NAME is only a handle for
// hipGetSymbolAddress, never an address to hand to a kernel.
static __device__ __align__(256) unsigned char g_attn_static_scratch[L3_ATTN_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
std::atomic<void*> g_scratch_ptr[kMaxDevices];
// Per device: 0 = not probed yet, 1 = the workgroups of a grid go to the 8 XCDs in turn, so that workgroups
// whose ids agree modulo 8 share an XCD (the single-launch attention form may be used), -1 = they do not.
std::atomic<int> g_xcd_state[kMaxDevices];

int current_device_index() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return -1;
    }
    return dev;
}

// Launches a probe grid that records the XCD of each workgroup into `counters` (the counter region
// of a workspace, used as scratch), waits for it and compares with the rule.  Synchronises `st`.
int probe_xcd_mapping(int dev, unsigned* counters, hipStream_t st) {
    constexpr int kProbe = 256;
    static_assert(kProbe <= kAttnArriveSlots, "one counter slot per probe workgroup");
    if (launch_xcd_probe(counters, kProbe, kAttnArriveStride, st) != 0) return L3_ERR_HIP;
    static unsigned host[kProbe * kAttnArriveStride];
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (hipStreamSynchronize(st) != hipSuccess ||
        hipMemcpy(host, counters, sizeof(host), hipMemcpyDeviceToHost) != hipSuccess) {
        (void)hipGetLastError();
        return L3_ERR_HIP;
    }
    bool ok = true;
    // round robin from whichever XCD the dispatcher starts this grid on
    const unsigned first = host[0];
    ok = first < 8u;
    for (int i = 0; i < kProbe; ++i) ok = ok && host[i * kAttnArriveStride] == (first + unsigned(i)) % 8u;
    g_xcd_state[dev].store(ok ? 1 : -1, std::memory_order_release);
    return L3_OK;
}

// Device address of the current device's copy of the array, looked up once per device (null on failure).
void* static_scratch_ptr() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return nullptr;
    }
    void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (ptr) return ptr;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    ptr = g_scratch_ptr[dev].load(std::memory_order_relaxed);
    if (ptr) return ptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_attn_static_scratch)) != hipSuccess || !ptr) {
        (void)hipGetLastError();
        return nullptr;
    }
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    return ptr;
}

// The static array starts with its arrival counters, which the loader zeroed.  On the first call on a
// device (outside stream capture, as that call has to be anyway) the XCD rule is probed there and the
// words the probe used are cleared again.
void* static_scratch_ready() {
    void* ptr = static_scratch_ptr();
    const int dev = current_device_index();
    if (!ptr || dev < 0) return nullptr;
    if (g_xcd_state[dev].load(std::memory_order_acquire) == 0) {
        unsigned* counters = static_cast<unsigned*>(ptr);
        if (probe_xcd_mapping(dev, counters, nullptr) != L3_OK) return nullptr;
        if (launch_fill_zero_u32(counters, L3_ATTN_COUNTER_BYTES / sizeof(unsigned), nullptr) != 0 ||
            hipStreamSynchronize(nullptr) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
    }
    return ptr;
}
}  // namespace

int current_device_cus() {
    static std::once_flag once;
    static int cus = 256;
    std::call_once(once, [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) {
            cus = n;
        } else {
            (void)hipGetLastError();  // do not leave a sticky "no device" behind
        }
    });
    return cus;
}

namespace {
// The split-KV kernel a call's flags ask for (the library keeps no such choice between calls).
int attn_impl_of(int flags) { return (flags & L3_ATTN_FLAG_KERNEL_FMA) ? kAttnImplFma : kAttnImplMfma; }
bool attn_flags_ok(int flags) {
    constexpr int known = L3_ATTN_FLAG_KERNEL_FMA | L3_ATTN_FLAG_PREFILL_MASK | L3_ATTN_FLAG_WS_COUNTERS |
                          L3_ATTN_FLAG_TWO_LAUNCHES | L3_ATTN_FLAG_FORM_MASK;
    return (flags & ~known) == 0 && (flags & L3_ATTN_FLAG_FORM_MASK) != L3_ATTN_FLAG_FORM_MASK;
}
// Whether the plan may count on the merge inside the split launch (the MFMA kernel with a counter
// region in the workspace, not switched off for the call).
bool attn_merge_in_launch_wanted(int flags) {
    return (flags & L3_ATTN_FLAG_WS_COUNTERS) && !(flags & (L3_ATTN_FLAG_TWO_LAUNCHES | L3_ATTN_FLAG_KERNEL_FMA));
}
}  // namespace

AttnPlan attn_make_plan(int B, int KVH, int S, int HD, int requested, int num_cus, int impl, int form,
                        bool merge_in_launch) {
    const int tile = attn_tile_tokens(HD, impl);
    const int tiles = ceil_div(S, tile);
    AttnPlan plan;
    plan.coop = false;
    int splits;
    if (requested > 0) {
        splits = requested;
        // a requested count is streamed unless the call asks for cooperative workgroups
        plan.coop = impl == kAttnImplMfma && form == L3_ATTN_FLAG_FORM_COOP;
    } else if (impl == kAttnImplMfma) {
        // Short sequences are latency-bound.  With at most one tile per wavefront of a workgroup (or two,
        // when there are too many heads for each to get a second workgroup) and not already enough
        // heads to fill the device twice over, one cooperative workgroup per (batch, kv head) finishes
        // the row in a single launch.
        const int64_t units = int64_t(B) * KVH;
        if (units <= 2 * int64_t(num_cus)) {
            const int wgs = int(std::max<int64_t>(1, num_cus / units));   // workgroups a head can have, one per unit
            // (Head size 64 with at least four workgroups to spare per head: up to six tiles only; its wavefronts
            // work through half tiles one after the other, 4.1 us at 256 tokens but 5.6 / 6.0 us at 448 / 512,
            // where four splits and a combine take 5.4 us.)
            const int one_launch_tiles = (HD == 64 && wgs >= 4) ? 6 : kMfmaWaves;
            if (tiles <= one_launch_tiles || (tiles <= 2 * kMfmaWaves && wgs < 2)) {
                plan.coop = true;
                plan.num_splits = 1;
                plan.tokens_per_split = tiles * tile;
                return plan;
            }
            // Medium sequences over few heads: still cooperative workgroups (eight wavefronts on one
            // head's token range, merged through LDS into ONE partial row per workgroup), spread over
            // the units with at least two tiles each.  Against the streaming form this measured
            // 6.7 instead of 8.6 us at 1024 tokens and 11.5 instead of 12.4 us at 8192 (head size 128,
            // batch 1, 8 kv heads) and 13.6 instead of 14.2 us at 12288; from two tiles per wavefront on
            // (16384: 17.9 against 16.2 us) the streaming form's whole-row reads win (head size 64, whose
            // per-head rows are 128 bytes: from one tile per wavefront).
            // When the last workgroup of a head can merge inside the launch (merge_in_launch, and a grid that
            // keeps a head on one XCD), the cooperative form has no combine launch to pay for and stays ahead
            // much longer: up to four tiles per wavefront at head size 128 (32768 tokens over 8 kv heads:
            // 24.8 against 25.6 us; 65536: level, left to the streaming form), one at head size 64 (16384
            // tokens: 10.0 against 11.1 us; 32768: level), and with short sequences a tile per workgroup at
            // head size 64 (1024 tokens in 16 splits: 4.6 against 4.9 us in 8).
            // (Not at head size 64 with eight kv heads per streaming workgroup and fewer than four workgroups
            // per head: 16 sequences of 1024 tokens took 11.1 us in two cooperative splits against 10.2 us streamed.)
            const bool merges = merge_in_launch && attn_mfma_can_merge_in_launch(B, KVH, true, 2);
            const bool longer = merges && !(HD == 64 && wgs < 4 && KVH % kMfmaWaves == 0);
            const int64_t tiles_per_wg = longer ? (HD == 128 ? 4 * kMfmaWaves : kMfmaWaves)
                                                : (HD == 128 ? kMfmaWaves * 3 / 2 : kMfmaWaves / 2);
            const int64_t coop_tiles = tiles_per_wg * wgs;
            if (tiles <= coop_tiles) {
                int coop_splits = std::min(wgs, (merges && HD == 64) ? tiles : ceil_div(tiles, 2));
                if (coop_splits > L3_ATTN_MAX_SPLITS) coop_splits = L3_ATTN_MAX_SPLITS;
                const int tps = ceil_div(ceil_div(S, coop_splits), tile) * tile;
                plan.coop = true;
                plan.tokens_per_split = tps;
                plan.num_splits = ceil_div(S, tps);
                return plan;
            }
        }
        // Streaming form; a workgroup covers heads_per_wg kv heads x (8 / heads_per_wg) splits, so the
        // split count comes in groups.  Few (batch, head group) pairs: one 8-wave workgroup per compute
        // unit, never more (a workgroup or two beyond one per unit run as a second round).  From a
        // thirty-second of the units on, three quarters of the units already saturate HBM and every
        // further split only adds partials for the combine; and where a group is a single split (eight
        // kv heads per workgroup) it is kept alone, with no combine at all, while a workgroup's stream
        // stays short.
        const int hpw = attn_mfma_heads_per_wg(KVH);
        const int spg = kMfmaWaves / hpw;
        const int64_t wgs_per_split_group = int64_t(B) * (KVH / hpw);
        int64_t groups;
        if (wgs_per_split_group * 32 >= num_cus) {
            groups = (int64_t(num_cus) * 3 / 4) / wgs_per_split_group;
            if (groups < 1) groups = 1;
            // K + V bytes a workgroup streams when there is a single group
            const int64_t stream_bytes = int64_t(kMfmaWaves) * ((S + spg - 1) / spg) * HD * 4;
            const bool short_stream = stream_bytes <= (int64_t(3) << 20);
            if (short_stream && spg == 1 && wgs_per_split_group * 4 >= num_cus) {
                groups = 1;   // a quarter of the units busy, but no partials and no second launch
            } else if (groups == 1 && !short_stream && int64_t(num_cus) / wgs_per_split_group >= 2) {
                groups = 2;
            } else if (groups > 1) {
                // Splits are whole tiles: with few tiles the rounding can halve the workgroup count (16 tiles
                // over 12 groups become 8 groups of two).  Shorter splits then, down to one tile, until
                // three fifths of the units are busy (B 16 x 1024 tokens at head size 64: 11.0 -> 8.9 us).
                int64_t split_tiles = ceil_div(tiles, int(std::min<int64_t>(groups * spg, tiles)));
                while (split_tiles > 1 &&
                       ceil_div(ceil_div(tiles, int(split_tiles)), spg) * wgs_per_split_group * 5 < int64_t(num_cus) * 3) {
                    --split_tiles;
                }
                groups = ceil_div(ceil_div(tiles, int(split_tiles)), spg);
            }
        } else {
            // Few workgroups per split group (batch 1 of a long sequence): four fifths of the units, each
            // with a longer stream, beat one workgroup on every unit (16384 tokens at head size 128: 171
            // workgroups of three tiles per wavefront 16.0 us, 256 of two 16.9 us; 32768: 205 of five
            // 25.5 us, 256 of four 26.2 us) -- fewer starts and ends, fewer partials for the combine --
            // as long as the rounding to whole tiles leaves at least three fifths of the units busy.
            groups = (int64_t(num_cus) * 4 + 4) / 5 / wgs_per_split_group;
            if (groups < 1) groups = 1;
            int64_t split_tiles = ceil_div(tiles, int(std::min<int64_t>(groups * spg, tiles)));
            while (split_tiles > 1 &&
                   ceil_div(tiles, int(split_tiles)) / spg * wgs_per_split_group * 5 < int64_t(num_cus) * 3) {
                --split_tiles;
            }
            groups = ceil_div(ceil_div(tiles, int(split_tiles)), spg);
        }
        splits = int(groups * spg);
    } else {
        // Two 4-wave workgroups per compute unit; more splits than that only add partials.
        const int64_t units = int64_t(B) * KVH;
        splits = int((int64_t(num_cus) * 2 + units - 1) / units);
    }
    if (splits > tiles) splits = tiles;  // a split shorter than one tile leaves lanes idle
    if (splits > L3_ATTN_MAX_SPLITS) splits = L3_ATTN_MAX_SPLITS;
    if (splits < 1) splits = 1;
    const int tps = ceil_div(ceil_div(S, splits), tile) * tile;
    plan.tokens_per_split = tps;
    plan.num_splits = ceil_div(S, tps);  // every split is non-empty
    return plan;
}

}  // namespace l3

using namespace l3;

extern "C" {

int l3_version(void) { return kVersion; }

const char* l3_strerror(int code) {
    switch (code) {
        case L3_OK: return "success";
        case L3_ERR_NULL_POINTER: return "null pointer argument";
        case L3_ERR_HEAD_SIZE: return "Unsupported head size for splitkv kernel";
        case L3_ERR_HEAD_RATIO: return "Unsupported QKV head ratio for splitkv kernel";
        case L3_ERR_SHAPE: return "invalid shape";
        case L3_ERR_STRIDE: return "unsupported stride";
        case L3_ERR_ALIGNMENT: return "misaligned pointer";
        case L3_ERR_WORKSPACE: return "workspace missing or too small";
        case L3_ERR_SPLITS: return "num_splits out of range";
        case L3_ERR_HIP: return "HIP runtime error at kernel launch";
        case L3_ERR_FLAGS: return "unknown bits in flags";
        case L3_ERR_SCRATCH: return "problem needs more scratch than the static device buffer holds";
        case L3_ERR_SCALE: return "softmax scale must be positive and finite";
        default: return "unknown error code";
    }
}

int l3_attn_choose_splits(int B, int KVH, int S, int HD, int num_cus, int flags) {
    if (HD != 64 && HD != 128) return L3_ERR_HEAD_SIZE;
    if (B <= 0 || KVH <= 0 || S <= 0) return L3_ERR_SHAPE;
    if (!attn_flags_ok(flags)) return L3_ERR_FLAGS;
    if (num_cus <= 0) num_cus = current_device_cus();
    return attn_make_plan(B, KVH, S, HD, 0, num_cus, attn_impl_of(flags), flags & L3_ATTN_FLAG_FORM_MASK,
                          attn_merge_in_launch_wanted(flags)).num_splits;
}

size_t l3_attn_decode_workspace_bytes(int B, int QH, int KVH, int S, int HD, int num_splits, int flags) {
    if (check_attn_shape(B, QH, KVH, S, HD) != L3_OK) return 0;
    if (num_splits < 0 || num_splits > L3_ATTN_MAX_SPLITS || !attn_flags_ok(flags)) return 0;
    const int cus = (num_splits == 0) ? current_device_cus() : 0;
    const AttnPlan plan = attn_make_plan(B, KVH, S, HD, num_splits, cus, attn_impl_of(flags),
                                         flags & L3_ATTN_FLAG_FORM_MASK, attn_merge_in_launch_wanted(flags));
    return attn_workspace_bytes(B, QH, HD, plan.num_splits, (flags & L3_ATTN_FLAG_WS_COUNTERS) != 0);
}

namespace {

// Argument checks shared by l3_attn_decode and l3_attn_split (out may be absent for the latter).
int check_attn_args(const void* q, const void* k, const void* v, const void* out, int B, int QH, int KVH, int S,
                    int HD, const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                    const int64_t* out_strides, int num_splits, bool need_out) {
    if (!q || !k || !v || !q_strides || !k_strides || !v_strides) return L3_ERR_NULL_POINTER;
    if (need_out && (!out || !out_strides)) return L3_ERR_NULL_POINTER;
    if (int rc = check_attn_shape(B, QH, KVH, S, HD); rc != L3_OK) return rc;
    if (num_splits < 0 || num_splits > L3_ATTN_MAX_SPLITS) return L3_ERR_SPLITS;
    // 16-byte vector loads: every row must start on a 16-byte boundary.
    // (strides of size-1 dimensions are never used to form an address and are not checked)
    const int q_dims[2] = {B, QH};
    for (int i = 0; i < 2; ++i) {
        if (q_dims[i] == 1) continue;
        if (q_strides[i] < 0 || q_strides[i] % 8) return L3_ERR_STRIDE;
        if (need_out && (out_strides[i] < 0 || out_strides[i] % 8)) return L3_ERR_STRIDE;
    }
    const int kv_dims[3] = {B, KVH, S};
    for (int i = 0; i < 3; ++i) {
        if (kv_dims[i] == 1) continue;
        if (k_strides[i] < 0 || v_strides[i] < 0 || k_strides[i] % 8 || v_strides[i] % 8) return L3_ERR_STRIDE;
    }
    // a tile's rows are addressed with 32-bit byte offsets from the tile's first token
    if (S > 1 && (k_strides[2] >= kAttnMaxTokenStride || v_strides[2] >= kAttnMaxTokenStride)) return L3_ERR_STRIDE;
    if (!aligned(q, 16) || !aligned(k, 16) || !aligned(v, 16) || (need_out && !aligned(out, 16)))
        return L3_ERR_ALIGNMENT;
    return L3_OK;
}

void fill_attn_params(AttnParams& p, const void* q, const void* k, const void* v, void* out, int B, int QH,
                      int KVH, int S, const int64_t* q_strides, const int64_t* k_strides,
                      const int64_t* v_strides, const int64_t* out_strides, float scale, const AttnPlan& plan) {
    p.q = static_cast<const uint16_t*>(q);
    p.k = static_cast<const uint16_t*>(k);
    p.v = static_cast<const uint16_t*>(v);
    p.out = static_cast<uint16_t*>(out);
    p.part_o = nullptr;
    p.part_ml = nullptr;
    p.B = B; p.QH = QH; p.KVH = KVH; p.S = S;
    p.seqlen_dev = nullptr;
    p.num_splits = plan.num_splits;
    p.tokens_per_split = plan.tokens_per_split;
    p.q_sb = q_strides[0]; p.q_sh = q_strides[1];
    p.k_sb = k_strides[0]; p.k_sh = k_strides[1]; p.k_st = k_strides[2];
    p.v_sb = v_strides[0]; p.v_sh = v_strides[1]; p.v_st = v_strides[2];
    p.o_sb = out_strides ? out_strides[0] : 0;
    p.o_sh = out_strides ? out_strides[1] : 0;
    p.scale_log2e = scale * 1.4426950408889634f;
    p.arrive = nullptr;
}

int launch_split_stage(const AttnParams& p, int HD, int R, int impl, bool coop, hipStream_t st) {
    return (impl == kAttnImplMfma) ? launch_attn_splitkv_mfma(p, HD, R, coop, st)
                                   : launch_attn_splitkv_fma(p, HD, R, st);
}

}  // namespace

namespace {
int attn_decode_impl(const void* q, const void* k, const void* v, void* out, void* workspace,
                     size_t workspace_bytes, int B, int QH, int KVH, int S, int HD,
                     const int64_t q_strides[2], const int64_t k_strides[3], const int64_t v_strides[3],
                     const int64_t out_strides[2], float scale, int num_splits, int flags, const int* seqlen_dev,
                     void* stream, bool static_scratch = false) {
    if (int rc = check_attn_args(q, k, v, out, B, QH, KVH, S, HD, q_strides, k_strides, v_strides, out_strides,
                                 num_splits, true); rc != L3_OK)
        return rc;
    if (!attn_flags_ok(flags)) return L3_ERR_FLAGS;
    if (!scale_ok(scale)) return L3_ERR_SCALE;
    const int impl = attn_impl_of(flags);
    if (static_scratch) flags |= L3_ATTN_FLAG_WS_COUNTERS;   // the static array always starts with its counters
    const bool counters = (flags & L3_ATTN_FLAG_WS_COUNTERS) != 0;
    const int cus = (num_splits == 0) ? current_device_cus() : 0;
    const AttnPlan plan = attn_make_plan(B, KVH, S, HD, num_splits, cus, impl, flags & L3_ATTN_FLAG_FORM_MASK,
                                         attn_merge_in_launch_wanted(flags));
    const size_t need = attn_workspace_bytes(B, QH, HD, plan.num_splits, counters);
    if (static_scratch) {
        // the partials go to this device's copy of the static array; nothing is allocated
        if (need > L3_ATTN_STATIC_SCRATCH_BYTES) return L3_ERR_SCRATCH;
        if (need > 0) {
            workspace = static_scratch_ready();
            if (!workspace) return L3_ERR_HIP;
        }
    } else if (need > 0) {
        if (!workspace || workspace_bytes < need) return L3_ERR_WORKSPACE;
        if (!aligned(workspace, kWorkspaceAlign)) return L3_ERR_ALIGNMENT;
    }
    AttnParams p;
    fill_attn_params(p, q, k, v, out, B, QH, KVH, S, q_strides, k_strides, v_strides, out_strides, scale, plan);
    p.seqlen_dev = seqlen_dev;
    bool merge_in_launch = false;
    if (plan.num_splits > 1) {
        const size_t rows = size_t(B) * size_t(QH) * size_t(plan.num_splits);
        char* ws = static_cast<char*>(workspace) + (counters ? size_t(L3_ATTN_COUNTER_BYTES) : 0);
        p.part_o = reinterpret_cast<float*>(ws);
        p.part_ml = reinterpret_cast<float2*>(ws + round_up(rows * HD * sizeof(float), kWorkspaceAlign));
        // One launch instead of two: only with prepared counters, on a device whose workgroup placement has
        // been confirmed, and for a grid that keeps every (batch, kv head) on one XCD.
        if (attn_merge_in_launch_wanted(flags) && attn_mfma_can_merge_in_launch(B, KVH, plan.coop, plan.num_splits)) {
            const int dev = current_device_index();
            merge_in_launch = dev >= 0 && g_xcd_state[dev].load(std::memory_order_acquire) == 1;
        }
        if (merge_in_launch) p.arrive = static_cast<unsigned*>(workspace);
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    int err = launch_split_stage(p, HD, QH / KVH, impl, plan.coop, st);
    const int groups = (impl == kAttnImplMfma && !plan.coop && B <= 65535) ? KVH / attn_mfma_heads_per_wg(KVH) : 0;
    if (err == 0 && plan.num_splits > 1 && !merge_in_launch) err = launch_attn_combine(p, HD, groups, st);
    return err == 0 ? L3_OK : L3_ERR_HIP;
}
}  // namespace

int l3_attn_decode(const void* q, const void* k, const void* v, void* out, void* workspace,
                   size_t workspace_bytes, int B, int QH, int KVH, int S, int HD,
                   const int64_t q_strides[2], const int64_t k_strides[3], const int64_t v_strides[3],
                   const int64_t out_strides[2], float scale, int num_splits, int flags, void* stream) {
    return attn_decode_impl(q, k, v, out, workspace, workspace_bytes, B, QH, KVH, S, HD, q_strides, k_strides,
                            v_strides, out_strides, scale, num_splits, flags, nullptr, stream);
}

int l3_attn_decode_static(const void* q, const void* k, const void* v, void* out, int B, int QH, int KVH, int S,
                          int HD, const int64_t q_strides[2], const int64_t k_strides[3],
                          const int64_t v_strides[3], const int64_t out_strides[2], float scale, int num_splits,
                          int flags, void* stream) {
    return attn_decode_impl(q, k, v, out, nullptr, 0, B, QH, KVH, S, HD, q_strides, k_strides, v_strides,
                            out_strides, scale, num_splits, flags, nullptr, stream, true);
}

int l3_attn_workspace_init(void* workspace, size_t workspace_bytes, void* stream) {
    if (!workspace) return L3_ERR_NULL_POINTER;
    if (workspace_bytes < L3_ATTN_COUNTER_BYTES) return L3_ERR_WORKSPACE;
    if (!aligned(workspace, kWorkspaceAlign)) return L3_ERR_ALIGNMENT;
    const int dev = current_device_index();
    if (dev < 0) return L3_ERR_HIP;
    hipStream_t st = static_cast<hipStream_t>(stream);
    unsigned* counters = static_cast<unsigned*>(workspace);
    if (g_xcd_state[dev].load(std::memory_order_acquire) == 0) {
        if (int rc = probe_xcd_mapping(dev, counters, st); rc != L3_OK) return rc;
    }
    if (launch_fill_zero_u32(counters, L3_ATTN_COUNTER_BYTES / sizeof(unsigned), st) != 0) return L3_ERR_HIP;
    return L3_OK;
}

int l3_attn_merge_in_launch_available(void) {
    const int dev = current_device_index();
    return dev >= 0 && g_xcd_state[dev].load(std::memory_order_acquire) == 1;
}

int l3_attn_launches(int B, int QH, int KVH, int S, int HD, int num_splits, int flags) {
    if (int rc = check_attn_shape(B, QH, KVH, S, HD); rc != L3_OK) return rc;
    if (num_splits < 0 || num_splits > L3_ATTN_MAX_SPLITS) return L3_ERR_SPLITS;
    if (!attn_flags_ok(flags)) return L3_ERR_FLAGS;
    const int cus = (num_splits == 0) ? current_device_cus() : 0;
    const AttnPlan plan = attn_make_plan(B, KVH, S, HD, num_splits, cus, attn_impl_of(flags),
                                         flags & L3_ATTN_FLAG_FORM_MASK, attn_merge_in_launch_wanted(flags));
    if (plan.num_splits == 1) return 1;
    const bool merge = attn_merge_in_launch_wanted(flags) && l3_attn_merge_in_launch_available() &&
                       attn_mfma_can_merge_in_launch(B, KVH, plan.coop, plan.num_splits);
    return merge ? 1 : 2;
}

int64_t l3_attn_placement_errors(const void* workspace) {
    if (!workspace) workspace = static_scratch_ptr();
    if (!workspace) return L3_ERR_HIP;
    unsigned n = 0;
    const char* word = static_cast<const char*>(workspace) + size_t(kAttnDiagSlot) * kAttnArriveStride * sizeof(unsigned);
    if (hipMemcpy(&n, word, sizeof(n), hipMemcpyDeviceToHost) != hipSuccess) {
        (void)hipGetLastError();
        return L3_ERR_HIP;
    }
    return int64_t(n);
}

int l3_attn_decode_devlen(const void* q, const void* k, const void* v, void* out, void* workspace,
                          size_t workspace_bytes, int B, int QH, int KVH, int max_S, int HD,
                          const int64_t q_strides[2], const int64_t k_strides[3], const int64_t v_strides[3],
                          const int64_t out_strides[2], float scale, int num_splits, int flags,
                          const int32_t* kv_len_dev, void* stream) {
    if (!kv_len_dev) return L3_ERR_NULL_POINTER;
    if (!aligned(kv_len_dev, 4)) return L3_ERR_ALIGNMENT;
    return attn_decode_impl(q, k, v, out, workspace, workspace_bytes, B, QH, KVH, max_S, HD, q_strides, k_strides,
                            v_strides, out_strides, scale, num_splits, flags, kv_len_dev, stream);
}

int l3_attn_prefill(const void* q, const void* k, const void* v, void* out, int B, int QH, int KVH, int T, int S,
                    int HD, const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                    const int64_t out_strides[3], float scale, int flags, void* stream) {
    if (!q || !k || !v || !out || !q_strides || !k_strides || !v_strides || !out_strides)
        return L3_ERR_NULL_POINTER;
    if (int rc = check_attn_shape(B, QH, KVH, S, HD); rc != L3_OK) return rc;
    if (!attn_flags_ok(flags)) return L3_ERR_FLAGS;
    if (!scale_ok(scale)) return L3_ERR_SCALE;
    if (T <= 0 || T > S) return L3_ERR_SHAPE;
    if (int64_t(B) * KVH * ((int64_t(T) + 1) / 2 + kMfmaWaves) >= (int64_t(1) << 31)) return L3_ERR_SHAPE;  // grid
    const int q_dims[3] = {B, QH, T};
    const int kv_dims[3] = {B, KVH, S};
    for (int i = 0; i < 3; ++i) {
        if (q_dims[i] != 1 && (q_strides[i] < 0 || out_strides[i] < 0 || q_strides[i] % 8 || out_strides[i] % 8))
            return L3_ERR_STRIDE;
        if (kv_dims[i] != 1 && (k_strides[i] < 0 || v_strides[i] < 0 || k_strides[i] % 8 || v_strides[i] % 8))
            return L3_ERR_STRIDE;
    }
    if (S > 1 && (k_strides[2] >= kAttnMaxTokenStride || v_strides[2] >= kAttnMaxTokenStride)) return L3_ERR_STRIDE;
    if (!aligned(q, 16) || !aligned(k, 16) || !aligned(v, 16) || !aligned(out, 16)) return L3_ERR_ALIGNMENT;
    PrefillParams p;
    p.q = static_cast<const uint16_t*>(q);
    p.k = static_cast<const uint16_t*>(k);
    p.v = static_cast<const uint16_t*>(v);
    p.out = static_cast<uint16_t*>(out);
    p.B = B; p.QH = QH; p.KVH = KVH; p.T = T; p.S = S;
    p.q_sb = q_strides[0]; p.q_sh = q_strides[1]; p.q_st = q_strides[2];
    p.k_sb = k_strides[0]; p.k_sh = k_strides[1]; p.k_st = k_strides[2];
    p.v_sb = v_strides[0]; p.v_sh = v_strides[1]; p.v_st = v_strides[2];
    p.o_sb = out_strides[0]; p.o_sh = out_strides[1]; p.o_st = out_strides[2];
    p.scale_log2e = scale * 1.4426950408889634f;
    p.snake = 0;
    p.no_max_tiles = (flags & L3_ATTN_FLAG_PREFILL_MASK) == L3_ATTN_FLAG_PREFILL_TILED_NO_MAX;
    p.auto_form = (flags & L3_ATTN_FLAG_PREFILL_MASK) == 0;
    // Which form (graph-timed sweeps over B 1 ... 256, T 8 ... 8192, head ratios 1, 3, 4 and 8): a prompt
    // that does not exceed one workgroup of the tiled form's small variant (one column block per wavefront) per
    // kv head, with few enough wavefronts for the device to hold them all at once, runs as independent
    // wavefronts with no barrier (16 tokens at head size 128: 4.8 against 6.1 us); everything else shares K/V
    // tiles (32 tokens: 5.2 against 5.9 us at head size 128, 4.2 against 5.1 us at 64).
    int form = flags & L3_ATTN_FLAG_PREFILL_MASK;
    if (form == 0) {
        const int R = QH / KVH;
        const int64_t private_waves = int64_t(B) * KVH * ((int64_t(T) * R + 15) / 16);
        const bool tiny = T <= prefill_tiled_positions_per_wg(R) / 2 && private_waves <= 4 * int64_t(current_device_cus());
        form = tiny ? L3_ATTN_FLAG_PREFILL_WAVE : L3_ATTN_FLAG_PREFILL_TILED;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int rc = (form == L3_ATTN_FLAG_PREFILL_WAVE) ? launch_attn_prefill(p, HD, st) : launch_attn_prefill_tiled(p, HD, st);
    return rc == 0 ? L3_OK : L3_ERR_HIP;
}

int l3_attn_split(const void* q, const void* k, const void* v, float* part_o, float* part_ml,
                  int B, int QH, int KVH, int S, int HD,
                  const int64_t q_strides[2], const int64_t k_strides[3], const int64_t v_strides[3],
                  float scale, int num_splits, int flags, void* stream) {
    if (!part_o || !part_ml) return L3_ERR_NULL_POINTER;
    if (int rc = check_attn_args(q, k, v, nullptr, B, QH, KVH, S, HD, q_strides, k_strides, v_strides, nullptr,
                                 num_splits, false); rc != L3_OK)
        return rc;
    if (!aligned(part_o, 16) || !aligned(part_ml, 8)) return L3_ERR_ALIGNMENT;
    if (!attn_flags_ok(flags)) return L3_ERR_FLAGS;
    if (!scale_ok(scale)) return L3_ERR_SCALE;
    const int impl = attn_impl_of(flags);
    const int cus = (num_splits == 0) ? current_device_cus() : 0;
    const AttnPlan plan = attn_make_plan(B, KVH, S, HD, num_splits, cus, impl, flags & L3_ATTN_FLAG_FORM_MASK,
                                         attn_merge_in_launch_wanted(flags));
    AttnParams p;
    fill_attn_params(p, q, k, v, nullptr, B, QH, KVH, S, q_strides, k_strides, v_strides, nullptr, scale, plan);
    p.part_o = part_o;
    p.part_ml = reinterpret_cast<float2*>(part_ml);
    const int err = launch_split_stage(p, HD, QH / KVH, impl, plan.coop, static_cast<hipStream_t>(stream));
    return err == 0 ? plan.num_splits : L3_ERR_HIP;
}

int l3_attn_combine(const float* part_o, const float* part_ml, void* out, int B, int QH, int HD, int n,
                    const int64_t out_strides[2], void* stream) {
    if (!part_o || !part_ml || !out || !out_strides) return L3_ERR_NULL_POINTER;
    if (HD != 64 && HD != 128) return L3_ERR_HEAD_SIZE;
    if (B <= 0 || QH <= 0 || int64_t(B) * QH >= (int64_t(1) << 31)) return L3_ERR_SHAPE;
    if (n < 1 || n > L3_ATTN_MAX_SPLITS) return L3_ERR_SPLITS;
    const int dims[2] = {B, QH};
    for (int i = 0; i < 2; ++i) {
        if (dims[i] != 1 && (out_strides[i] < 0 || out_strides[i] % 8)) return L3_ERR_STRIDE;
    }
    if (!aligned(part_o, 16) || !aligned(part_ml, 8) || !aligned(out, 16)) return L3_ERR_ALIGNMENT;
    AttnParams p = {};
    p.out = static_cast<uint16_t*>(out);
    p.part_o = const_cast<float*>(part_o);
    p.part_ml = reinterpret_cast<float2*>(const_cast<float*>(part_ml));
    p.B = B; p.QH = QH;
    p.num_splits = n;
    p.o_sb = out_strides[0]; p.o_sh = out_strides[1];
    return launch_attn_combine(p, HD, 0, static_cast<hipStream_t>(stream)) == 0 ? L3_OK : L3_ERR_HIP;
}

int l3_rms_norm(const void* x, const void* w, void* y, int64_t rows, int C, float eps, void* stream) {
    if (!x || !w || !y) return L3_ERR_NULL_POINTER;
    if (rows <= 0 || C <= 0 || rows >= (int64_t(1) << 31)) return L3_ERR_SHAPE;
    if (!aligned(x, 2) || !aligned(w, 2) || !aligned(y, 2)) return L3_ERR_ALIGNMENT;
    const bool vec_ok = (C % 8 == 0) && aligned(x, 16) && aligned(w, 16) && aligned(y, 16);
    return launch_rms_norm(static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(w),
                           static_cast<uint16_t*>(y), rows, C, eps, vec_ok,
                           static_cast<hipStream_t>(stream)) == 0 ? L3_OK : L3_ERR_HIP;
}

int l3_add_rms_norm(const void* x, const void* residual, const void* w, void* sum_out, void* y, int64_t rows,
                    int C, float eps, void* stream) {
    if (!x || !residual || !w || !sum_out || !y) return L3_ERR_NULL_POINTER;
    if (rows <= 0 || C <= 0 || rows >= (int64_t(1) << 31)) return L3_ERR_SHAPE;
    if (!aligned(x, 2) || !aligned(residual, 2) || !aligned(w, 2) || !aligned(sum_out, 2) || !aligned(y, 2))
        return L3_ERR_ALIGNMENT;
    const bool vec_ok = (C % 8 == 0) && aligned(x, 16) && aligned(residual, 16) && aligned(w, 16) &&
                        aligned(sum_out, 16) && aligned(y, 16);
    return launch_add_rms_norm(static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(residual),
                               static_cast<const uint16_t*>(w), static_cast<uint16_t*>(sum_out),
                               static_cast<uint16_t*>(y), rows, C, eps, vec_ok,
                               static_cast<hipStream_t>(stream)) == 0 ? L3_OK : L3_ERR_HIP;
}

int l3_silu_mul(const void* a, const void* b, void* y, int64_t n, void* stream) {
    if (!a || !b || !y) return L3_ERR_NULL_POINTER;
    if (n <= 0 || n >= (int64_t(1) << 38)) return L3_ERR_SHAPE;
    if (!aligned(a, 2) || !aligned(b, 2) || !aligned(y, 2)) return L3_ERR_ALIGNMENT;
    const bool vec_ok = (n % 8 == 0) && aligned(a, 16) && aligned(b, 16) && aligned(y, 16);
    return launch_silu_mul(static_cast<const uint16_t*>(a), static_cast<const uint16_t*>(b),
                           static_cast<uint16_t*>(y), n, vec_ok, static_cast<hipStream_t>(stream)) == 0
               ? L3_OK : L3_ERR_HIP;
}

namespace {

struct QkvTarget {
    const float* table;
    const int* pos;
    uint16_t *q_out, *cache_k, *cache_v;
    int NH, KVH, HD, cache_len, table_rows;
    int64_t c_sb, c_st;
};

int linear_decode_impl(const void* x, const void* norm_w, float norm_eps, const void* w0, const void* w1,
                       const void* res, void* y, int M, int N, int K, int64_t x_stride, int64_t w_stride,
                       int64_t y_stride, bool swiglu, void* stream, const QkvTarget* qkv = nullptr) {
    if (!x || !w0 || (!y && !qkv) || (swiglu && !w1)) return L3_ERR_NULL_POINTER;
    if (M <= 0 || M > L3_LINEAR_MAX_ROWS || N <= 0 || K <= 0 || N % 4 != 0 || K % 32 != 0) return L3_ERR_SHAPE;
    if (N > (1 << 24) || K > (1 << 24)) return L3_ERR_SHAPE;
    if (norm_w && !linear_skinny_can_stage(M, K)) return L3_ERR_SHAPE;
    if (x_stride < K || w_stride < K || y_stride < N || x_stride % 8 || w_stride % 8 || y_stride % 4)
        return L3_ERR_STRIDE;
    if (!aligned(x, 16) || !aligned(w0, 16) || (swiglu && !aligned(w1, 16)) || (y && !aligned(y, 8)) ||
        (norm_w && !aligned(norm_w, 16)) || (res && !aligned(res, 8)))
        return L3_ERR_ALIGNMENT;
    LinearParams p;
    p.x = static_cast<const uint16_t*>(x);
    p.w0 = static_cast<const uint16_t*>(w0);
    p.w1 = static_cast<const uint16_t*>(w1);
    p.norm_w = static_cast<const uint16_t*>(norm_w);
    p.res = static_cast<const uint16_t*>(res);
    p.norm_eps = norm_eps;
    p.y = static_cast<uint16_t*>(y);
    p.M = M; p.N = N; p.K = K;
    p.x_stride = x_stride; p.w_stride = w_stride; p.y_stride = y_stride;
    p.sk = 1;
    if (qkv) {
        p.rope_table = qkv->table; p.rope_pos = qkv->pos; p.q_out = qkv->q_out;
        p.cache_k = qkv->cache_k; p.cache_v = qkv->cache_v;
        p.NH = qkv->NH; p.KVH = qkv->KVH; p.HD = qkv->HD; p.cache_len = qkv->cache_len; p.table_rows = qkv->table_rows;
        p.c_sb = qkv->c_sb; p.c_st = qkv->c_st;
    } else {
        p.rope_table = nullptr; p.rope_pos = nullptr; p.q_out = p.cache_k = p.cache_v = nullptr;
        p.NH = p.KVH = p.HD = p.cache_len = p.table_rows = 0;
        p.c_sb = p.c_st = 0;
    }
    return launch_linear_skinny(p, swiglu, current_device_cus(), static_cast<hipStream_t>(stream)) == 0 ? L3_OK
                                                                                                        : L3_ERR_HIP;
}

}  // namespace

int l3_linear_decode(const void* x, const void* w, void* y, int M, int N, int K, int64_t x_stride, int64_t w_stride,
                     int64_t y_stride, void* stream) {
    return linear_decode_impl(x, nullptr, 0.f, w, nullptr, nullptr, y, M, N, K, x_stride, w_stride, y_stride, false,
                              stream);
}

int l3_linear_swiglu_decode(const void* x, const void* w_gate, const void* w_up, void* y, int M, int N, int K,
                            int64_t x_stride, int64_t w_stride, int64_t y_stride, void* stream) {
    return linear_decode_impl(x, nullptr, 0.f, w_gate, w_up, nullptr, y, M, N, K, x_stride, w_stride, y_stride, true,
                              stream);
}

int l3_linear_decode_fused(const void* x, const void* norm_weight, float norm_eps, const void* w, const void* w_up,
                           const void* residual, void* y, int M, int N, int K, int64_t x_stride, int64_t w_stride,
                           int64_t y_stride, void* stream) {
    return linear_decode_impl(x, norm_weight, norm_eps, w, w_up, residual, y, M, N, K, x_stride, w_stride, y_stride,
                              w_up != nullptr, stream);
}

int l3_linear_qkv_rope_append(const void* x, const void* norm_weight, float norm_eps, const void* w_qkv,
                              const float* freq_table, void* q_out, void* cache_k, void* cache_v,
                              const int32_t* pos_dev, int B, int NH, int KVH, int HD, int K, int64_t x_stride,
                              int64_t w_stride, const int64_t cache_strides[2], int cache_len, int table_rows,
                              void* stream) {
    if (!freq_table || !q_out || !cache_k || !cache_v || !pos_dev || !cache_strides) return L3_ERR_NULL_POINTER;
    if (NH <= 0 || KVH <= 0 || HD <= 0 || HD % 8 != 0 || cache_len <= 0 || table_rows <= 0) return L3_ERR_SHAPE;
    if (int64_t(NH + 2 * KVH) * HD > (1 << 24)) return L3_ERR_SHAPE;
    if (cache_strides[0] < 0 || cache_strides[1] < 0 || cache_strides[1] % 8 || (B > 1 && cache_strides[0] % 8))
        return L3_ERR_STRIDE;
    if (!aligned(q_out, 16) || !aligned(cache_k, 16) || !aligned(cache_v, 16) || !aligned(freq_table, 16) ||
        !aligned(pos_dev, 4))
        return L3_ERR_ALIGNMENT;
    QkvTarget t;
    t.table = freq_table; t.pos = pos_dev;
    t.q_out = static_cast<uint16_t*>(q_out);
    t.cache_k = static_cast<uint16_t*>(cache_k);
    t.cache_v = static_cast<uint16_t*>(cache_v);
    t.NH = NH; t.KVH = KVH; t.HD = HD; t.cache_len = cache_len; t.table_rows = table_rows;
    t.c_sb = cache_strides[0]; t.c_st = cache_strides[1];
    const int N = (NH + 2 * KVH) * HD;
    return linear_decode_impl(x, norm_weight, norm_eps, w_qkv, nullptr, nullptr, nullptr, B, N, K, x_stride, w_stride,
                              N, false, stream, &t);
}

int l3_silu_mul_rows(const void* a, const void* b, void* y, int64_t rows, int64_t cols, int64_t a_row_stride,
                     int64_t b_row_stride, void* stream) {
    if (!a || !b || !y) return L3_ERR_NULL_POINTER;
    if (rows <= 0 || cols <= 0 || cols % 8 != 0 || rows * cols >= (int64_t(1) << 38)) return L3_ERR_SHAPE;
    if (a_row_stride < cols || b_row_stride < cols || a_row_stride % 8 || b_row_stride % 8) return L3_ERR_STRIDE;
    if (!aligned(a, 16) || !aligned(b, 16) || !aligned(y, 16)) return L3_ERR_ALIGNMENT;
    return launch_silu_mul_rows(static_cast<const uint16_t*>(a), static_cast<const uint16_t*>(b),
                                static_cast<uint16_t*>(y), rows, cols, a_row_stride, b_row_stride,
                                static_cast<hipStream_t>(stream)) == 0 ? L3_OK : L3_ERR_HIP;
}

int l3_linear_splitk_plan(int N, int K, int num_cus) {
    if (N <= 0 || K <= 0 || K % 128 != 0) return L3_ERR_SHAPE;
    if (num_cus <= 0) num_cus = current_device_cus();
    return linear_splitk_plan(N, K, num_cus);
}

size_t l3_linear_splitk_workspace_bytes(int M, int N, int ksplit) {
    if (M <= 0 || N <= 0 || ksplit <= 0) return 0;
    return size_t(ksplit) * size_t(M) * size_t(N) * sizeof(float);
}

int l3_linear_splitk(const void* x, const void* w, void* part, size_t part_bytes, int M, int N, int K,
                     int64_t x_stride, int64_t w_stride, int ksplit, void* stream) {
    if (!x || !w || !part) return L3_ERR_NULL_POINTER;
    if (M <= 0 || M > L3_LINEAR_SPLITK_MAX_ROWS || N <= 0 || K <= 0 || N % 8 != 0 || K % 128 != 0) return L3_ERR_SHAPE;
    if (N > (1 << 24) || K > (1 << 24)) return L3_ERR_SHAPE;
    if (ksplit <= 0 || ksplit > K / 128 ||
        (K / 128 + ksplit - 1) / ksplit > linear_splitk_max_chunks(N, current_device_cus()))
        return L3_ERR_SPLITS;
    if (x_stride < K || w_stride < K || x_stride % 8 || w_stride % 8) return L3_ERR_STRIDE;
    if (!aligned(x, 16) || !aligned(w, 16) || !aligned(part, 16)) return L3_ERR_ALIGNMENT;
    if (part_bytes < l3_linear_splitk_workspace_bytes(M, N, ksplit)) return L3_ERR_WORKSPACE;
    return launch_linear_splitk(static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(w),
                                static_cast<float*>(part), M, N, K, x_stride, w_stride, ksplit, current_device_cus(),
                                static_cast<hipStream_t>(stream)) == 0 ? L3_OK : L3_ERR_HIP;
}

int l3_linear_splitk_finish(const void* part, int ksplit, const void* residual, void* y, int M, int N,
                            int64_t y_stride, void* stream) {
    if (!part || !y) return L3_ERR_NULL_POINTER;
    if (M <= 0 || M > L3_LINEAR_SPLITK_MAX_ROWS || N <= 0 || N % 8 != 0 || N > (1 << 24)) return L3_ERR_SHAPE;
    if (ksplit <= 0 || ksplit > L3_ATTN_MAX_SPLITS) return L3_ERR_SPLITS;
    if (y_stride < N || y_stride % 8) return L3_ERR_STRIDE;
    if (!aligned(part, 16) || !aligned(y, 16) || (residual && !aligned(residual, 16))) return L3_ERR_ALIGNMENT;
    return launch_linear_splitk_finish(static_cast<const float*>(part), ksplit, static_cast<const uint16_t*>(residual),
                                       static_cast<uint16_t*>(y), M, N, y_stride,
                                       static_cast<hipStream_t>(stream)) == 0 ? L3_OK : L3_ERR_HIP;
}

int l3_add_rms_norm_partials(const void* x, const void* part, int ksplit, const void* w, void* sum_out, void* y,
                             int rows, int C, float eps, void* stream) {
    if (!x || !part || !w || !sum_out || !y) return L3_ERR_NULL_POINTER;
    if (rows <= 0 || rows > 65535 || C <= 0 || C % 8 != 0 || C > 8192) return L3_ERR_SHAPE;
    if (ksplit <= 0 || ksplit > L3_ATTN_MAX_SPLITS) return L3_ERR_SPLITS;
    if (!aligned(x, 16) || !aligned(part, 16) || !aligned(w, 16) || !aligned(sum_out, 16) || !aligned(y, 16))
        return L3_ERR_ALIGNMENT;
    return launch_add_rms_norm_partials(static_cast<const uint16_t*>(x), static_cast<const float*>(part), ksplit,
                                        int64_t(rows) * C, static_cast<const uint16_t*>(w),
                                        static_cast<uint16_t*>(sum_out), static_cast<uint16_t*>(y), rows, C, eps,
                                        static_cast<hipStream_t>(stream)) == 0 ? L3_OK : L3_ERR_HIP;
}

int l3_rot_embed_append_partials(const void* part, int ksplit, const float* freq_table, void* q_out, void* cache_k,
                                 void* cache_v, const int32_t* pos_dev, int B, int NH, int KVH, int HD,
                                 const int64_t cache_strides[2], int cache_len, int table_rows, void* stream) {
    if (!part || !freq_table || !q_out || !cache_k || !cache_v || !pos_dev || !cache_strides)
        return L3_ERR_NULL_POINTER;
    if (B <= 0 || NH <= 0 || KVH <= 0 || HD <= 0 || HD % 8 != 0 || cache_len <= 0 || table_rows <= 0)
        return L3_ERR_SHAPE;
    if (int64_t(B) * (NH + 2 * KVH) * (HD / 8) >= (int64_t(1) << 31)) return L3_ERR_SHAPE;
    if (ksplit <= 0 || ksplit > L3_ATTN_MAX_SPLITS) return L3_ERR_SPLITS;
    if (cache_strides[0] < 0 || cache_strides[1] < 0 || cache_strides[1] % 8 || (B > 1 && cache_strides[0] % 8))
        return L3_ERR_STRIDE;
    if (!aligned(part, 16) || !aligned(q_out, 16) || !aligned(cache_k, 16) || !aligned(cache_v, 16) ||
        !aligned(freq_table, 16) || !aligned(pos_dev, 4))
        return L3_ERR_ALIGNMENT;
    return launch_rot_embed_append_partials(static_cast<const float*>(part), ksplit,
                                            int64_t(B) * (NH + 2 * KVH) * HD, freq_table,
                                            static_cast<uint16_t*>(q_out), static_cast<uint16_t*>(cache_k),
                                            static_cast<uint16_t*>(cache_v), pos_dev, B, NH, KVH, HD, cache_strides[0],
                                            cache_strides[1], cache_len, table_rows,
                                            static_cast<hipStream_t>(stream)) == 0 ? L3_OK : L3_ERR_HIP;
}

size_t l3_argmax_workspace_bytes(int rows, int V) {
    if (rows <= 0 || V <= 0) return 0;
    return size_t(rows) * size_t(argmax_parts(V)) * (sizeof(float) + sizeof(int));
}

int l3_argmax(const void* logits, int64_t row_stride, int rows, int V, void* workspace, size_t workspace_bytes,
              int64_t* out, void* stream) {
    if (!logits || !out || !workspace) return L3_ERR_NULL_POINTER;
    if (rows <= 0 || V <= 0 || rows > 65535) return L3_ERR_SHAPE;
    if (row_stride < V) return L3_ERR_STRIDE;
    if (!aligned(logits, 2) || !aligned(out, 8) || !aligned(workspace, 8)) return L3_ERR_ALIGNMENT;
    if (workspace_bytes < l3_argmax_workspace_bytes(rows, V)) return L3_ERR_WORKSPACE;
    const size_t parts = size_t(rows) * size_t(argmax_parts(V));
    float* pv = static_cast<float*>(workspace);
    int* pi = reinterpret_cast<int*>(pv + parts);
    return launch_argmax(static_cast<const uint16_t*>(logits), row_stride, rows, V, pv, pi, out,
                         static_cast<hipStream_t>(stream)) == 0 ? L3_OK : L3_ERR_HIP;
}

int l3_greedy_step(const void* logits, int64_t row_stride, int rows, int V, void* workspace, size_t workspace_bytes,
                   int64_t* tokens, const uint8_t* text_mask, int64_t total_len, int64_t* tok, int32_t* pos,
                   int32_t* kv_len, uint8_t* eos, const int64_t* stop_tokens, int n_stop, void* stream) {
    if (!logits || !workspace || !tokens || !text_mask || !tok || !pos || !kv_len || !eos || (n_stop > 0 && !stop_tokens))
        return L3_ERR_NULL_POINTER;
    if (rows <= 0 || V <= 0 || rows > 65535 || total_len <= 0 || n_stop < 0) return L3_ERR_SHAPE;
    if (row_stride < V) return L3_ERR_STRIDE;
    if (!aligned(logits, 2) || !aligned(workspace, 8) || !aligned(tokens, 8) || !aligned(tok, 8) || !aligned(pos, 4) ||
        !aligned(kv_len, 4) || (stop_tokens && !aligned(stop_tokens, 8)))
        return L3_ERR_ALIGNMENT;
    if (workspace_bytes < l3_argmax_workspace_bytes(rows, V)) return L3_ERR_WORKSPACE;
    const size_t parts = size_t(rows) * size_t(argmax_parts(V));
    float* pv = static_cast<float*>(workspace);
    int* pi = reinterpret_cast<int*>(pv + parts);
    return launch_greedy_step(static_cast<const uint16_t*>(logits), row_stride, rows, V, pv, pi, tokens, text_mask,
                              total_len, tok, pos, kv_len, eos, stop_tokens, n_stop,
                              static_cast<hipStream_t>(stream)) == 0 ? L3_OK : L3_ERR_HIP;
}

int l3_rot_embed(const void* x, const float* freq, void* y, int B, int T, int NH, int HD,
                 const int64_t x_strides[3], void* stream) {
    if (!x || !freq || !y || !x_strides) return L3_ERR_NULL_POINTER;
    if (B <= 0 || T <= 0 || NH <= 0 || HD <= 0 || (HD % 2) != 0) return L3_ERR_SHAPE;
    if (int64_t(B) * T * NH * (HD / 2) >= (int64_t(1) << 38)) return L3_ERR_SHAPE;  // grid size
    const int x_dims[3] = {B, T, NH};
    bool strides8 = true;
    for (int i = 0; i < 3; ++i) {
        if (x_dims[i] == 1) continue;
        if (x_strides[i] < 0 || x_strides[i] % 2) return L3_ERR_STRIDE;
        strides8 = strides8 && (x_strides[i] % 8 == 0);
    }
    if (!aligned(x, 4) || !aligned(y, 4) || !aligned(freq, 8)) return L3_ERR_ALIGNMENT;
    const bool vec_ok = (HD % 8 == 0) && aligned(x, 16) && aligned(y, 16) && aligned(freq, 16) && strides8;
    return launch_rot_embed(static_cast<const uint16_t*>(x), freq, static_cast<uint16_t*>(y), B, T, NH, HD,
                            x_strides[0], x_strides[1], x_strides[2], vec_ok,
                            static_cast<hipStream_t>(stream)) == 0 ? L3_OK : L3_ERR_HIP;
}

int l3_rot_embed_append(const void* qkv, const float* freq_table, void* q_out, void* cache_k, void* cache_v,
                        const int32_t* pos_dev, int B, int NH, int KVH, int HD, int64_t qkv_batch_stride,
                        const int64_t cache_strides[2], int cache_len, int table_rows, void* stream) {
    if (!qkv || !freq_table || !q_out || !cache_k || !cache_v || !pos_dev || !cache_strides)
        return L3_ERR_NULL_POINTER;
    if (B <= 0 || NH <= 0 || KVH <= 0 || HD <= 0 || HD % 8 != 0 || cache_len <= 0 || table_rows <= 0)
        return L3_ERR_SHAPE;
    if (int64_t(B) * (NH + 2 * KVH) * (HD / 8) >= (int64_t(1) << 31)) return L3_ERR_SHAPE;
    if (qkv_batch_stride < 0 || (B > 1 && qkv_batch_stride % 8)) return L3_ERR_STRIDE;
    if (cache_strides[0] < 0 || cache_strides[1] < 0 || cache_strides[1] % 8 || (B > 1 && cache_strides[0] % 8))
        return L3_ERR_STRIDE;
    if (!aligned(qkv, 16) || !aligned(q_out, 16) || !aligned(cache_k, 16) || !aligned(cache_v, 16) ||
        !aligned(freq_table, 16) || !aligned(pos_dev, 4))
        return L3_ERR_ALIGNMENT;
    return launch_rot_embed_append(static_cast<const uint16_t*>(qkv), freq_table, static_cast<uint16_t*>(q_out),
                                   static_cast<uint16_t*>(cache_k), static_cast<uint16_t*>(cache_v), pos_dev, B, NH,
                                   KVH, HD, qkv_batch_stride, cache_strides[0], cache_strides[1], cache_len,
                                   table_rows, static_cast<hipStream_t>(stream)) == 0 ? L3_OK : L3_ERR_HIP;
}

int l3_hbm_read_stream(const void* src, size_t bytes, void* sink, int workgroups, void* stream) {
    if (!src || !sink) return L3_ERR_NULL_POINTER;
    if (bytes == 0 || bytes % 16 != 0) return L3_ERR_SHAPE;
    if (!aligned(src, 16) || !aligned(sink, 4)) return L3_ERR_ALIGNMENT;
    if (workgroups <= 0) workgroups = 4 * current_device_cus();
    if (workgroups > (1 << 20)) return L3_ERR_SHAPE;
    return launch_hbm_read_stream(src, bytes, sink, workgroups, static_cast<hipStream_t>(stream)) == 0 ? L3_OK
                                                                                                       : L3_ERR_HIP;
}

int l3_hbm_rw_stream(const void* src, void* dst, size_t bytes, int workgroups, int block_kib, void* stream) {
    if (!src || !dst) return L3_ERR_NULL_POINTER;
    if (bytes == 0 || bytes % 16 != 0) return L3_ERR_SHAPE;
    if (!aligned(src, 16) || !aligned(dst, 16)) return L3_ERR_ALIGNMENT;
    if (block_kib == 0) block_kib = 64;
    if (block_kib != 8 && block_kib != 16 && block_kib != 32 && block_kib != 64) return L3_ERR_SHAPE;
    if (workgroups <= 0) workgroups = 4 * current_device_cus();
    if (workgroups > (1 << 20)) return L3_ERR_SHAPE;
    return launch_hbm_rw_stream(src, dst, bytes, workgroups, block_kib, static_cast<hipStream_t>(stream)) == 0 ? L3_OK
                                                                                                               : L3_ERR_HIP;
}

}  // extern "C"
