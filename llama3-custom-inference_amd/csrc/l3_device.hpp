// Device-side helpers shared by the gfx950 kernels: bf16 <-> f32 on raw bit patterns and
// wave64 cross-lane reductions built on DPP.  These take the place of the reference's
// dtype_bfloat16.cuh:47-54 (casts) and reduce_kernels.cuh:8-64 (32-lane shuffle
// butterflies plus a shared-memory stage), re-thought for 64-wide wavefronts.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace l3 {

constexpr int kWaveSize = 64;

// ---------------------------------------------------------------- bf16 bit patterns
// A 32-bit word holds two bf16 values: element 2i in the low half, 2i+1 in the high half.
__device__ __forceinline__ float bf16lo_to_f32(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16hi_to_f32(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float(uint32_t(h) << 16); }

// Round-to-nearest-even f32 -> bf16 bit pattern (NaN stays a quiet NaN).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    uint32_t r = u + 0x7fffu + ((u >> 16) & 1u);
    r = (f != f) ? 0x7fc00000u : r;
    return r >> 16;
}
// Two f32 -> packed bf16x2 with the gfx950 v_cvt_pk_bf16_f32 (round-to-nearest-even).
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// Unpack the 8 bf16 values of a 16-byte vector into f32.
__device__ __forceinline__ void unpack8(const uint4& v, float (&f)[8]) {
    f[0] = bf16lo_to_f32(v.x); f[1] = bf16hi_to_f32(v.x);
    f[2] = bf16lo_to_f32(v.y); f[3] = bf16hi_to_f32(v.y);
    f[4] = bf16lo_to_f32(v.z); f[5] = bf16hi_to_f32(v.z);
    f[6] = bf16lo_to_f32(v.w); f[7] = bf16hi_to_f32(v.w);
}

// ------------------------------------------------------------------ DPP cross-lane
// dpp_ctrl encodings (GCN3+/CDNA): quad_perm = perm bits, 0x140 row_mirror,
// 0x141 row_half_mirror.  All lanes read a valid source for these patterns.
constexpr int kDppQuadXor1 = 0xB1;        // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;        // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;  // lane i <-> 7-i within each 8 lanes
constexpr int kDppRowMirror = 0x140;      // lane i <-> 15-i within each 16 lanes

template <int CTRL>
__device__ __forceinline__ float dpp_move(float x) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, true));
}

// Sum over aligned groups of N consecutive lanes (N in {4, 8, 16}); every lane of a
// group ends with the same bits (each step adds the two halves commutatively).
template <int N>
__device__ __forceinline__ float group_sum(float x) {
    static_assert(N == 4 || N == 8 || N == 16, "group size");
    x += dpp_move<kDppQuadXor1>(x);
    x += dpp_move<kDppQuadXor2>(x);
    if constexpr (N >= 8) x += dpp_move<kDppRowHalfMirror>(x);
    if constexpr (N >= 16) x += dpp_move<kDppRowMirror>(x);
    return x;
}

template <int N>
__device__ __forceinline__ float group_max(float x) {
    static_assert(N == 4 || N == 8 || N == 16, "group size");
    x = fmaxf(x, dpp_move<kDppQuadXor1>(x));
    x = fmaxf(x, dpp_move<kDppQuadXor2>(x));
    if constexpr (N >= 8) x = fmaxf(x, dpp_move<kDppRowHalfMirror>(x));
    if constexpr (N >= 16) x = fmaxf(x, dpp_move<kDppRowMirror>(x));
    return x;
}

// Whole-wavefront sum / max, result uniform across the 64 lanes: DPP inside each row of
// 16 lanes, then the four row results are read back through scalar lane reads.
__device__ __forceinline__ float wave_sum(float x) {
    x = group_sum<16>(x);
    int xi = __builtin_bit_cast(int, x);
    float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 0));
    float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 16));
    float c = __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 32));
    float d = __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 48));
    return (a + b) + (c + d);
}

__device__ __forceinline__ float wave_max(float x) {
    x = group_max<16>(x);
    int xi = __builtin_bit_cast(int, x);
    float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 0));
    float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 16));
    float c = __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 32));
    float d = __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 48));
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
}

// 2^x through the hardware v_exp_f32 (inputs here are <= 0 or small; no denormal fix-up).
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Sum over the K splits of a split-K linear (float32 partial products part[s][...], element
// stride split_stride between splits) for 8 consecutive outputs, in split order, rounded to bf16
// once: what the unsplit linear would have written.
__device__ __forceinline__ uint4 sum_splits_bf16x8(const float* p, int ksplit, int64_t split_stride) {
    float4 a = *reinterpret_cast<const float4*>(p);
    float4 b = *reinterpret_cast<const float4*>(p + 4);
    int s = 1;
    // four splits per round: their loads are independent and go out together, the additions keep
    // the split order
    for (; s + 4 <= ksplit; s += 4) {
        float4 c[4], d[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            c[i] = *reinterpret_cast<const float4*>(p + (s + i) * split_stride);
            d[i] = *reinterpret_cast<const float4*>(p + (s + i) * split_stride + 4);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            a.x += c[i].x; a.y += c[i].y; a.z += c[i].z; a.w += c[i].w;
            b.x += d[i].x; b.y += d[i].y; b.z += d[i].z; b.w += d[i].w;
        }
    }
    for (; s < ksplit; ++s) {
        const float4 c = *reinterpret_cast<const float4*>(p + s * split_stride);
        const float4 d = *reinterpret_cast<const float4*>(p + s * split_stride + 4);
        a.x += c.x; a.y += c.y; a.z += c.z; a.w += c.w;
        b.x += d.x; b.y += d.y; b.z += d.z; b.w += d.w;
    }
    uint4 o;
    o.x = pack_bf16x2(a.x, a.y);
    o.y = pack_bf16x2(a.z, a.w);
    o.z = pack_bf16x2(b.x, b.y);
    o.w = pack_bf16x2(b.z, b.w);
    return o;
}

// Rotation of one adjacent bf16 pair (packed in a word) by (cos, sin): the rotary embedding of
// custom_kernels.cu:400-414, float32 arithmetic, one rounding.
__device__ __forceinline__ uint32_t rotate_pair(uint32_t xw, float c, float s) {
    const float x0 = bf16lo_to_f32(xw);
    const float x1 = bf16hi_to_f32(xw);
    // x0*c - x1*s can cancel; a plain float32 evaluation then carries the rounding error of
    // the larger product into a much smaller result and can miss the exact answer by more
    // than one bf16 ulp.  The second product's rounding error is recovered exactly with an
    // fma (e = x1*s - p) so that the error stays relative to the result itself.
    const float p0 = x1 * s;
    const float e0 = fmaf(x1, s, -p0);
    const float y0 = fmaf(x0, c, -p0) - e0;
    const float p1 = x1 * c;
    const float e1 = fmaf(x1, c, -p1);
    const float y1 = fmaf(x0, s, p1) + e1;
    return pack_bf16x2(y0, y1);
}

// bf16(silu(a)) as a float: torch's F.silu(a) * b materialises silu's bf16 result before the
// multiplication (model.py:134), and so does every kernel here that fuses the product.
__device__ __forceinline__ float silu_rounded(float a) {
    const float s = a / (1.0f + expf(-a));
    return __uint_as_float(f32_to_bf16_bits(s) << 16);
}

// 16-byte global load / store on element pointers.
__device__ __forceinline__ uint4 load16(const uint16_t* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ __forceinline__ void store16(uint16_t* p, const uint4& v) { *reinterpret_cast<uint4*>(p) = v; }

// Loads of data that the whole grid touches once (K/V of a decode step, weights, the input of a
// row-wise operator): non-temporal, which the caches treat as a stream instead of keeping the lines.
// A pure read stream measured 6.4 TB/s this way against 5.8 TB/s with plain loads on the same
// buffers.  Stores stay plain: a non-temporal store of an operator's output cost the kernel that
// reads it next more (32 MB: 11.5 us instead of 8.4 us) than it saved the writer.
// (-DL3_STREAM_LOADS=0 turns these back into plain loads, for repeating the comparison.)
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
#ifndef L3_STREAM_LOADS
#define L3_STREAM_LOADS 1
#endif
__device__ __forceinline__ uint4 load16_stream(const uint16_t* p) {
#if L3_STREAM_LOADS
    const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
#else
    return load16(p);
#endif
}

}  // namespace l3
