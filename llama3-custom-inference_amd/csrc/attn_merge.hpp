// Log-sum-exp merge of split-KV partials by one wavefront, and the pieces of the single-launch
// form of decode attention in which the workgroup that finishes a head last merges it.
//
//   out = sum_i o_i 2^(m_i - M) / sum_i l_i 2^(m_i - M),   M = max_i m_i
//
// What custom_flash_attention_combine_kernel (custom_kernels.cu:179-223) is meant to do; see
// attn_combine.hip for how the reference's version differs.
//
// Merging inside the split kernel rests on two properties of this device.  (1) The workgroups of
// a grid (x fastest, then y, then z) go to the 8 XCDs in turn, so workgroups whose linear ids
// agree modulo 8 run on the same XCD, and the compute units of one XCD share one L2: a store that
// has been acknowledged (s_waitcnt vmcnt(0)) has reached that L2, an atomic without device scope
// executes there, and a load that misses the vector L1 (sc0) goes through it and so observes the
// store.  (The hardware counters show such rows coming back through the fabric rather than out of
// the L2's data array -- a line stored to without having been read is not kept -- which costs
// latency, not correctness: both accesses pass the same L2 channel in order.)
// So workgroups whose linear ids agree modulo 8 can hand data to each other with no cache
// write-back or invalidate, which on this part cost tens of microseconds.  (2) A counter that
// receives exactly n arrivals per launch lets the last arriver know itself and reset it, so the
// counters are zero between launches without a clearing kernel.
// The host only chooses this form when every workgroup of a (batch, kv head) has the same id
// modulo 8 and after a probe launch has confirmed (1) on the device; the arrivals carry their
// XCC_ID, and a head whose arrivals came from more than one XCD is counted in a diagnostic word.
#pragma once

#include "attn_common.hpp"

namespace l3 {

constexpr int kCombineRows = 32;   // splits a wavefront merges per pass (their loads are all in flight at once)

typedef float f32x4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2v __attribute__((ext_vector_type(2)));

// XCD this wavefront runs on (hardware register XCC_ID, bits 3:0).
__device__ __forceinline__ unsigned xcc_id() { return __builtin_amdgcn_s_getreg((3 << 11) | 20) & 0xfu; }

__device__ __forceinline__ unsigned linear_workgroup_id() {
    return blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
}

// One more arrival at a counter that gets `n` of them per launch.  An arrival adds 1 to the low half of
// the word and the arriver's XCD to the high half; the last one (true) sets the word back to zero --
// nothing else touches it before the next launch -- and reports through *same_xcd whether all n
// arrived from the XCD it runs on itself.  Executes in the L2 of the caller's XCD (no device scope).
__device__ __forceinline__ bool arrive_is_last(unsigned* counter, int n, bool* same_xcd) {
    const unsigned me = xcc_id();
    const unsigned old = __hip_atomic_fetch_add(counter, 1u | (me << 16), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    const bool last = (old & 0xffffu) == unsigned(n - 1);
    if (last) {
        __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        *same_xcd = (old >> 16) == me * unsigned(n - 1);
    }
    return last;
}

// All of this wavefront's earlier stores are in the L2 when this returns.
__device__ __forceinline__ void wait_stores_in_l2() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Loads of partials another compute unit wrote during this launch: buffer loads with sc0, which
// miss the vector L1 and read the XCD's L2.  `base` and `limit_bytes` are wave-uniform; offsets are
// bytes; a 16-byte load that reaches past `limit_bytes` touches no memory and returns zeros.
struct L2Reader {
    __amdgpu_buffer_rsrc_t rsrc;
    const char* base;
    __device__ __forceinline__ L2Reader(const void* b, uint32_t limit_bytes)
        : rsrc(__builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(b), 0, int(limit_bytes), 0x00020000)),
          base(static_cast<const char*>(b)) {}
    __device__ __forceinline__ f32x4v load16(uint32_t lane_off, uint32_t uniform_off) const {
        return __builtin_bit_cast(f32x4v, __builtin_amdgcn_raw_buffer_load_b128(rsrc, int(lane_off), int(uniform_off), 1));
    }
    // (an 8-byte load with the same policy: what a workgroup-scope atomic load compiles to on this target;
    // the caller keeps the offset inside the buffer)
    __device__ __forceinline__ float2 load8(uint32_t byte_off) const {
        const uint64_t bits = __hip_atomic_load(reinterpret_cast<const uint64_t*>(base + byte_off), __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_WORKGROUP);
        return make_float2(__builtin_bit_cast(float, uint32_t(bits)), __builtin_bit_cast(float, uint32_t(bits >> 32)));
    }
};
// Ordinary loads (a kernel of its own reads what an earlier kernel wrote): a 16-byte load past
// `limit_bytes` is moved back onto the last 16 bytes inside (its row has weight zero).
struct PlainReader {
    const char* base;
    uint32_t last;
    __device__ __forceinline__ PlainReader(const void* b, uint32_t limit_bytes)
        : base(static_cast<const char*>(b)), last(limit_bytes - 16u) {}
    __device__ __forceinline__ f32x4v load16(uint32_t lane_off, uint32_t uniform_off) const {
        return *reinterpret_cast<const f32x4v*>(base + min(lane_off + uniform_off, last));
    }
    __device__ __forceinline__ float2 load8(uint32_t byte_off) const {
        return *reinterpret_cast<const float2*>(base + byte_off);
    }
};

// Cross-lane sums and maxima on the vector ALU alone (no trip through the LDS crossbar, no scalar
// read-back): rotations inside the rows of 16 lanes (DPP), then the two cross-row swaps.
template <int CTRL>
__device__ __forceinline__ float dpp_rot(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, true));
}
template <bool MAX>
__device__ __forceinline__ float lane_op(float a, float b) { return MAX ? fmaxf(a, b) : a + b; }
template <bool MAX>
__device__ __forceinline__ float across_rows16(float x) {   // with lane ^ 16
    const uint32_t xi = __builtin_bit_cast(uint32_t, x);
    const auto r = __builtin_amdgcn_permlane16_swap(xi, xi, false, false);
    return lane_op<MAX>(__builtin_bit_cast(float, uint32_t(r[0])), __builtin_bit_cast(float, uint32_t(r[1])));
}
template <bool MAX>
__device__ __forceinline__ float across_halves32(float x) {   // with lane ^ 32
    const uint32_t xi = __builtin_bit_cast(uint32_t, x);
    const auto r = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
    return lane_op<MAX>(__builtin_bit_cast(float, uint32_t(r[0])), __builtin_bit_cast(float, uint32_t(r[1])));
}
// Over the lanes that agree in lane % TPR (TPR a power of two <= 32), result in every one of them.
template <int TPR, bool MAX>
__device__ __forceinline__ float coset_reduce(float x) {
    static_assert(TPR >= 1 && TPR <= 32 && (TPR & (TPR - 1)) == 0, "lanes per row");
    if constexpr (TPR <= 1) x = lane_op<MAX>(x, dpp_rot<0x121>(x));   // row_ror:1
    if constexpr (TPR <= 2) x = lane_op<MAX>(x, dpp_rot<0x122>(x));   // row_ror:2
    if constexpr (TPR <= 4) x = lane_op<MAX>(x, dpp_rot<0x124>(x));   // row_ror:4
    if constexpr (TPR <= 8) x = lane_op<MAX>(x, dpp_rot<0x128>(x));   // row_ror:8
    if constexpr (TPR <= 16) x = across_rows16<MAX>(x);
    return across_halves32<MAX>(x);
}
// Over aligned segments of G consecutive lanes (G = 16, 32 or 64), result in every lane of the segment.
template <int G, bool MAX>
__device__ __forceinline__ float segment_reduce(float x) {
    static_assert(G == 16 || G == 32 || G == 64, "segment size");
    x = lane_op<MAX>(x, dpp_rot<0x121>(x));
    x = lane_op<MAX>(x, dpp_rot<0x122>(x));
    x = lane_op<MAX>(x, dpp_rot<0x124>(x));
    x = lane_op<MAX>(x, dpp_rot<0x128>(x));
    if constexpr (G >= 32) x = across_rows16<MAX>(x);
    if constexpr (G >= 64) x = across_halves32<MAX>(x);
    return x;
}

// One wavefront merges the n >= 1 partial rows po[i][HD] with statistics ml[i] = (max in log2
// units, sum) of one (batch, query head) pair and writes the bf16 output row -- or, with CG > 1,
// column group cg of it (HD / CG columns), so that CG wavefronts share a pair and each pulls
// 1 / CG of the bytes.
// A wavefront-wide memory instruction costs the compute unit 16 cycles whatever its width, and the
// last arriver of a head has nothing to overlap them with, so the merge is built from as few as
// possible, all requested in one round trip before any weight is known and with nothing but a
// constant between one request and the next: ONE load of statistics (lane l < 32 holds split l of
// the pass) and 16-byte loads of the rows, whose lanes past the last split read zeros.  Weights
// are formed in the statistics lanes and handed to the lanes that hold the rows through the LDS
// crossbar; lanes that hold the same columns meet in coset_reduce.  More than 32 splits take
// further passes with a running maximum.  All arguments are wave-uniform.
template <int HD, typename Reader, int CG = 1>
__device__ __forceinline__ void merge_pair_rows(const float* __restrict__ po, const float2* __restrict__ ml, int n,
                                                uint16_t* __restrict__ out_row, int cg = 0) {
    constexpr int NR = kCombineRows;
    constexpr int RQ = HD / 4;              // 16-byte pieces of a whole partial row
    constexpr int TPR = RQ / CG;            // lanes covering this wavefront's columns of a row
    constexpr int RPL = kWaveSize / TPR;    // rows per wavefront-wide load
    constexpr int NLD = NR / RPL;           // row loads per pass
    static_assert(TPR >= 1 && kWaveSize % TPR == 0 && NR % RPL == 0 && NLD >= 1, "rows must divide over the lanes");
    const int lane = threadIdx.x & (kWaveSize - 1);
    const int dq = cg * TPR + lane % TPR;
    const int sub = lane / TPR;
    const Reader rows(po, uint32_t(n) * uint32_t(HD * 4)), stats(ml, uint32_t(n) * 8u);
    const uint32_t lane_off = uint32_t(sub * RQ + dq) * 16u;

    float m_w = kMaskedScore, l_w = 0.f;    // running statistics (the same in every lane)
    f32x4v acc = {0.f, 0.f, 0.f, 0.f};
    for (int r0 = 0; r0 < n; r0 += NR) {
        // (unconditional, from a clamped index: a load inside a divergent branch would be waited for there)
        float2 st = stats.load8(uint32_t(min(r0 + lane, n - 1)) * 8u);
        if (lane >= NR || r0 + lane >= n) st = make_float2(kMaskedScore, 0.f);
        f32x4v x[NLD];
#pragma unroll
        for (int u = 0; u < NLD; ++u) {
            x[u] = f32x4v{0.f, 0.f, 0.f, 0.f};
            // wavefront-uniform: nothing is requested past the last split
            if (r0 + u * RPL < n) x[u] = rows.load16(lane_off, uint32_t(r0 + u * RPL) * uint32_t(HD * 4));
        }
        const float m_new = fmaxf(m_w, segment_reduce<kWaveSize, true>(st.x));
        const float alpha = fast_exp2(m_w - m_new);
        const float wgt = fast_exp2(st.x - m_new);   // absent splits: 2^(-1e30 - m) = 0
        l_w = fmaf(l_w, alpha, segment_reduce<kWaveSize, false>(st.y * wgt));
        m_w = m_new;
        if (r0 > 0) acc *= alpha;
#pragma unroll
        for (int u = 0; u < NLD; ++u) {
            const float w = __shfl(wgt, u * RPL + sub, kWaveSize);
            acc.x = fmaf(w, x[u].x, acc.x);
            acc.y = fmaf(w, x[u].y, acc.y);
            acc.z = fmaf(w, x[u].z, acc.z);
            acc.w = fmaf(w, x[u].w, acc.w);
        }
    }
    const float inv = 1.0f / l_w;
    const float o0 = coset_reduce<TPR, false>(acc.x) * inv;
    const float o1 = coset_reduce<TPR, false>(acc.y) * inv;
    const float o2 = coset_reduce<TPR, false>(acc.z) * inv;
    const float o3 = coset_reduce<TPR, false>(acc.w) * inv;
    if (lane < TPR) {
        uint2 packed;
        packed.x = pack_bf16x2(o0, o1);
        packed.y = pack_bf16x2(o2, o3);
        *reinterpret_cast<uint2*>(out_row + dq * 4) = packed;
    }
}

}  // namespace l3
