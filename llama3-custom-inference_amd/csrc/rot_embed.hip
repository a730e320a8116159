// Fused rotary embedding for gfx950.  Takes the place of custom_rot_embed_kernel
// (custom_kernels.cu:391-416): same arithmetic (float32 complex multiply of adjacent
// pairs by the (cos, sin) table row of the token, one rounding), same strided-input /
// contiguous-output contract, but each lane moves 16 bytes (four pairs) instead of 4 and
// the grid is a flat range over 16-byte items rather than one 32/64-thread block per
// (batch, token, head).
#include "l3_device.hpp"
#include "l3_host.hpp"

namespace l3 {

namespace {

constexpr int kRopeThreads = 256;

// One 16-byte item (8 values = 4 pairs) per thread.  VPR = HD / 8 items per (b, t, h) row.
__global__ void __launch_bounds__(kRopeThreads)
rot_embed_vec_kernel(const uint16_t* __restrict__ x, const float* __restrict__ freq, uint16_t* __restrict__ y,
                     int64_t total_items, int T, int NH, int HD, int64_t sb, int64_t st, int64_t sh) {
    const int64_t item = int64_t(blockIdx.x) * kRopeThreads + threadIdx.x;
    if (item >= total_items) return;
    const int vpr = HD / 8;
    const int c = int(item % vpr);
    int64_t r = item / vpr;
    const int h = int(r % NH);
    r /= NH;
    const int t = int(r % T);
    const int64_t b = r / T;

    const uint4 xv = load16(x + b * sb + t * st + h * sh + c * 8);
    const float4* fp = reinterpret_cast<const float4*>(freq + int64_t(t) * HD + c * 8);
    const float4 f0 = fp[0];
    const float4 f1 = fp[1];
    uint4 o;
    o.x = rotate_pair(xv.x, f0.x, f0.y);
    o.y = rotate_pair(xv.y, f0.z, f0.w);
    o.z = rotate_pair(xv.z, f1.x, f1.y);
    o.w = rotate_pair(xv.w, f1.z, f1.w);
    store16(y + item * 8, o);
}

// The same work with the index arithmetic taken out of the lanes: blockIdx.y is the batch row,
// blockIdx.x a block of `rpw` tokens, and a thread's place in the workgroup gives (token, head
// group, 16-byte chunk) -- by shifts when the counts are powers of two (POW2).  A thread rotates
// chunk c of HG consecutive heads of its token with one read of the table row (the flat kernel
// above spends most of its instructions on 64-bit divisions).  Needs vpr * NH / HG <= 256 threads
// per token and B <= 65535.
template <int HG, bool POW2>
__global__ void __launch_bounds__(kRopeThreads)
rot_embed_rows_kernel(const uint16_t* __restrict__ x, const float* __restrict__ freq, uint16_t* __restrict__ y, int T,
                      int NH, int HD, int64_t sb, int64_t st, int64_t sh, int tpr, int vpr, int rpw, int tpr_shift,
                      int vpr_shift) {
    const int tid = threadIdx.x;
    int rl, hq, c;
    if constexpr (POW2) {
        rl = tid >> tpr_shift;
        const int j = tid & (tpr - 1);
        hq = j >> vpr_shift;
        c = j & (vpr - 1);
    } else {
        rl = tid / tpr;
        const int j = tid - rl * tpr;
        hq = j / vpr;
        c = j - hq * vpr;
    }
    const int t = int(blockIdx.x) * rpw + rl;
    if (rl >= rpw || t >= T) return;
    const int64_t b = blockIdx.y;
    const float4* fp = reinterpret_cast<const float4*>(freq + int64_t(t) * HD + c * 8);
    const uint16_t* xp = x + b * sb + t * st + int64_t(hq * HG) * sh + c * 8;
    uint4 xv[HG];
#pragma unroll
    for (int i = 0; i < HG; ++i) xv[i] = load16_stream(xp + i * sh);
    const float4 f0 = fp[0];
    const float4 f1 = fp[1];
    uint16_t* yp = y + ((b * T + t) * NH + hq * HG) * HD + c * 8;
#pragma unroll
    for (int i = 0; i < HG; ++i) {
        uint4 o;
        o.x = rotate_pair(xv[i].x, f0.x, f0.y);
        o.y = rotate_pair(xv[i].y, f0.z, f0.w);
        o.z = rotate_pair(xv[i].z, f1.x, f1.y);
        o.w = rotate_pair(xv[i].w, f1.z, f1.w);
        store16(yp + i * HD, o);
    }
}

// Fallback: one pair per thread with 4-byte accesses (any even HD, 4-byte aligned rows).
__global__ void __launch_bounds__(kRopeThreads)
rot_embed_pair_kernel(const uint16_t* __restrict__ x, const float* __restrict__ freq, uint16_t* __restrict__ y,
                      int64_t total_pairs, int T, int NH, int HD, int64_t sb, int64_t st, int64_t sh) {
    const int64_t item = int64_t(blockIdx.x) * kRopeThreads + threadIdx.x;
    if (item >= total_pairs) return;
    const int ppr = HD / 2;
    const int c = int(item % ppr);
    int64_t r = item / ppr;
    const int h = int(r % NH);
    r /= NH;
    const int t = int(r % T);
    const int64_t b = r / T;
    const uint32_t xw = *reinterpret_cast<const uint32_t*>(x + b * sb + t * st + h * sh + c * 2);
    const float2 f = *reinterpret_cast<const float2*>(freq + int64_t(t) * HD + c * 2);
    *reinterpret_cast<uint32_t*>(y + item * 2) = rotate_pair(xw, f.x, f.y);
}

// Decode step (one new token per sequence): rotate the query and key heads of the fused qkv
// projection at the position held in device memory, write the rotated keys and the values
// straight into the KV cache row of that position, and return the rotated queries.  One launch
// in place of two rot_embed calls plus the two cache slice assignments of model.py:100-106;
// because the position is read on the device the launch can be replayed from a HIP graph.
// One 16-byte item per thread over (batch, q|k|v head slot, chunk).
// PART: the fused projection comes as the float32 partial products of a split-K linear
// (part[s][b][:], `ksplit` splits `split_stride` elements apart) and is added up here first.
template <bool PART>
__global__ void __launch_bounds__(kRopeThreads)
rot_embed_append_kernel(const uint16_t* __restrict__ qkv, const float* __restrict__ part, int ksplit,
                        int64_t split_stride, const float* __restrict__ table, uint16_t* __restrict__ q_out,
                        uint16_t* __restrict__ cache_k, uint16_t* __restrict__ cache_v,
                        const int* __restrict__ pos_dev, int total_items, int NH, int KVH, int HD, int64_t qkv_sb,
                        int64_t c_sb, int64_t c_st, int cache_len, int table_rows) {
    const int item = blockIdx.x * kRopeThreads + threadIdx.x;
    if (item >= total_items) return;
    const int vpr = HD / 8;
    const int slots = NH + 2 * KVH;
    const int c = item % vpr;
    const int slot = (item / vpr) % slots;
    const int b = item / (vpr * slots);
    // the projection does not depend on the position: its loads go out before the position is waited for
    uint4 xv;
    if constexpr (PART) {
        xv = sum_splits_bf16x8(part + b * qkv_sb + slot * HD + c * 8, ksplit, split_stride);
    } else {
        xv = load16(qkv + b * qkv_sb + slot * HD + c * 8);
    }
    const int pos = *pos_dev;
    if (pos < 0 || pos >= cache_len || pos >= table_rows) return;  // never write outside the cache
    if (slot >= NH + KVH) {  // value head: plain copy into the cache
        store16(cache_v + b * c_sb + pos * c_st + (slot - NH - KVH) * HD + c * 8, xv);
        return;
    }
    const float4* fp = reinterpret_cast<const float4*>(table + int64_t(pos) * HD + c * 8);
    const float4 f0 = fp[0];
    const float4 f1 = fp[1];
    uint4 o;
    o.x = rotate_pair(xv.x, f0.x, f0.y);
    o.y = rotate_pair(xv.y, f0.z, f0.w);
    o.z = rotate_pair(xv.z, f1.x, f1.y);
    o.w = rotate_pair(xv.w, f1.z, f1.w);
    if (slot < NH) {
        store16(q_out + (int64_t(b) * NH + slot) * HD + c * 8, o);
    } else {
        store16(cache_k + b * c_sb + pos * c_st + (slot - NH) * HD + c * 8, o);
    }
}

}  // namespace

int launch_rot_embed_append(const uint16_t* qkv, const float* table, uint16_t* q_out, uint16_t* cache_k,
                            uint16_t* cache_v, const int* pos_dev, int B, int NH, int KVH, int HD, int64_t qkv_sb,
                            int64_t c_sb, int64_t c_st, int cache_len, int table_rows, hipStream_t stream) {
    const int items = B * (NH + 2 * KVH) * (HD / 8);
    const unsigned blocks = unsigned((items + kRopeThreads - 1) / kRopeThreads);
    hipLaunchKernelGGL(rot_embed_append_kernel<false>, dim3(blocks), dim3(kRopeThreads), 0, stream, qkv, nullptr, 1,
                       int64_t(0), table, q_out, cache_k, cache_v, pos_dev, items, NH, KVH, HD, qkv_sb, c_sb, c_st,
                       cache_len, table_rows);
    return int(hipGetLastError());
}

int launch_rot_embed_append_partials(const float* part, int ksplit, int64_t split_stride, const float* table,
                                     uint16_t* q_out, uint16_t* cache_k, uint16_t* cache_v, const int* pos_dev, int B,
                                     int NH, int KVH, int HD, int64_t c_sb, int64_t c_st, int cache_len,
                                     int table_rows, hipStream_t stream) {
    const int items = B * (NH + 2 * KVH) * (HD / 8);
    const unsigned blocks = unsigned((items + kRopeThreads - 1) / kRopeThreads);
    hipLaunchKernelGGL(rot_embed_append_kernel<true>, dim3(blocks), dim3(kRopeThreads), 0, stream, nullptr, part,
                       ksplit, split_stride, table, q_out, cache_k, cache_v, pos_dev, items, NH, KVH, HD,
                       int64_t(NH + 2 * KVH) * HD, c_sb, c_st, cache_len, table_rows);
    return int(hipGetLastError());
}

int launch_rot_embed(const uint16_t* x, const float* freq, uint16_t* y, int B, int T, int NH, int HD,
                     int64_t sb, int64_t st, int64_t sh, bool vec_ok, hipStream_t stream) {
    const int64_t rows = int64_t(B) * T * NH;
    const int vpr = HD / 8;
    const int hg = (NH % 4 == 0) ? 4 : (NH % 2 == 0) ? 2 : 1;
    const int tpr = vec_ok ? vpr * (NH / hg) : 0;
    if (vec_ok && tpr <= kRopeThreads && B <= 65535) {
        const int rpw = kRopeThreads / tpr;
        const bool pow2 = (tpr & (tpr - 1)) == 0 && (vpr & (vpr - 1)) == 0;
        const int tpr_shift = pow2 ? __builtin_ctz(unsigned(tpr)) : 0;
        const int vpr_shift = pow2 ? __builtin_ctz(unsigned(vpr)) : 0;
        const dim3 grid(unsigned((T + rpw - 1) / rpw), unsigned(B));
        const dim3 block(kRopeThreads);
#define L3_ROPE_ROWS(HG, POW2)                                                                                       \
    hipLaunchKernelGGL((rot_embed_rows_kernel<HG, POW2>), grid, block, 0, stream, x, freq, y, T, NH, HD, sb, st, sh, \
                       tpr, vpr, rpw, tpr_shift, vpr_shift)
        if (hg == 4) {
            if (pow2) L3_ROPE_ROWS(4, true); else L3_ROPE_ROWS(4, false);
        } else if (hg == 2) {
            if (pow2) L3_ROPE_ROWS(2, true); else L3_ROPE_ROWS(2, false);
        } else {
            if (pow2) L3_ROPE_ROWS(1, true); else L3_ROPE_ROWS(1, false);
        }
#undef L3_ROPE_ROWS
    } else if (vec_ok) {
        const int64_t items = rows * (HD / 8);
        const unsigned blocks = unsigned((items + kRopeThreads - 1) / kRopeThreads);
        hipLaunchKernelGGL(rot_embed_vec_kernel, dim3(blocks), dim3(kRopeThreads), 0, stream, x, freq, y, items, T,
                           NH, HD, sb, st, sh);
    } else {
        const int64_t items = rows * (HD / 2);
        const unsigned blocks = unsigned((items + kRopeThreads - 1) / kRopeThreads);
        hipLaunchKernelGGL(rot_embed_pair_kernel, dim3(blocks), dim3(kRopeThreads), 0, stream, x, freq, y, items, T,
                           NH, HD, sb, st, sh);
    }
    return int(hipGetLastError());
}

}  // namespace l3
