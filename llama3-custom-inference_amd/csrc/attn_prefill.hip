// Causal GQA attention for T > 1 query tokens (prompt prefill) on the gfx950 matrix cores.
//
// The reference sends this case to PyTorch's fused attention (model.py:114-116:
// scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)); this kernel routes it
// through the same tile loop as the decode kernel (attn_mfma_core.hpp) instead.  The 16 columns
// of the MFMA tiles are (query position, query head) pairs: 16 / R consecutive positions of the
// R query heads that share a kv head.  A wavefront owns one such column group, streams the kv
// head's tokens from 0 up to its last position, and masks per column what lies after the
// column's own position; it needs no split and no combine.  Eight consecutive column groups of a
// (batch, kv head) share a workgroup, so their K/V tiles mostly hit in cache.
//
// Query i of T sits at absolute position S - T + i (the KV cache already holds S >= T tokens,
// the last T of which belong to the queries) and attends to tokens 0 .. S - T + i.  For S == T
// -- the only case the reference produces -- this is PyTorch's is_causal mask.
#include "attn_mfma_core.hpp"

namespace l3 {

namespace {

template <int HD>
__global__ void __launch_bounds__(kMfmaWaves * kWaveSize, 2)
attn_prefill_mfma_kernel(const PrefillParams p) {
    using T = MfmaTile<HD>;
    constexpr int WT = T::WT, KC = T::KC, NB = T::NB, SLAB = T::SLAB;
    __shared__ __align__(16) unsigned char s_slab[kMfmaWaves][SLAB];

    const int lane = threadIdx.x & (kWaveSize - 1);
    const int wave = wave_uniform(int(threadIdx.x) / kWaveSize);
    const int fn = lane & 15;   // column of the MFMA tiles
    const int fg = lane >> 4;   // k group

    const int R = p.QH / p.KVH;
    const int ppw = 16 / R;                          // query positions per wavefront
    const int groups = (p.T + ppw - 1) / ppw;        // column groups per (batch, kv head)
    const int wgs_per_head = (groups + kMfmaWaves - 1) / kMfmaWaves;
    int bid = blockIdx.x;
    const int wg = bid % wgs_per_head;
    bid /= wgs_per_head;
    const int kvh = bid % p.KVH;
    const int b = bid / p.KVH;
    const int group = wg * kMfmaWaves + wave;
    if (group >= groups) return;  // whole wavefront; the kernel has no barrier

    // this lane's column: query index qi (of T) and head; columns past the data stay empty
    const int qi = group * ppw + fn / R;
    const int qh = kvh * R + fn % R;
    const bool col_valid = (fn < ppw * R) && (qi < p.T);
    const int first_pos = p.S - p.T + group * ppw;            // absolute position of the group's first query
    const int t_end = min(p.S, first_pos + ppw);              // tokens any column of the group may see
    const int col_limit = col_valid ? (p.S - p.T + qi + 1) : 0;
    const int col_limit_min = first_pos + 1;

    bf16x8_t qfrag[KC];
#pragma unroll
    for (int m = 0; m < KC; ++m) {
        uint4 qv = make_uint4(0u, 0u, 0u, 0u);
        if (col_valid) qv = load16(p.q + b * p.q_sb + int64_t(qh) * p.q_sh + int64_t(qi) * p.q_st + (m * 4 + fg) * 8);
        qfrag[m] = __builtin_bit_cast(bf16x8_t, qv);
    }

    const int64_t k_head = b * p.k_sb + kvh * p.k_sh;   // token 0 of this kv head, in elements
    const int64_t v_head = b * p.v_sb + kvh * p.v_sh;

    f32x4_t O[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) O[nb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = kMaskedScore;
    float l_part = 0.f;
    mfma_tile_loop<HD>(p.k, p.v, k_head, v_head, p.k_st, p.v_st, s_slab[wave], qfrag, 0, t_end, WT, col_limit, col_limit_min,
                       p.scale_log2e, O, m_run, l_part);

    l_part += __shfl_xor(l_part, 16, kWaveSize);
    l_part += __shfl_xor(l_part, 32, kWaveSize);
    if (col_valid) {
        const float inv = 1.0f / l_part;
        uint16_t* orow = p.out + b * p.o_sb + int64_t(qh) * p.o_sh + int64_t(qi) * p.o_st + fg * 4;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            uint2 w;
            w.x = pack_bf16x2(O[nb][0] * inv, O[nb][1] * inv);
            w.y = pack_bf16x2(O[nb][2] * inv, O[nb][3] * inv);
            *reinterpret_cast<uint2*>(orow + nb * 16) = w;
        }
    }
}

}  // namespace

int launch_attn_prefill(const PrefillParams& p, int HD, hipStream_t stream) {
    const int R = p.QH / p.KVH;
    const int ppw = 16 / R;
    const int groups = (p.T + ppw - 1) / ppw;
    const int wgs_per_head = (groups + kMfmaWaves - 1) / kMfmaWaves;
    const dim3 grid(unsigned(p.B) * unsigned(p.KVH) * unsigned(wgs_per_head));
    const dim3 block(kMfmaWaves * kWaveSize);
    if (HD == 64) {
        hipLaunchKernelGGL((attn_prefill_mfma_kernel<64>), grid, block, 0, stream, p);
    } else {
        hipLaunchKernelGGL((attn_prefill_mfma_kernel<128>), grid, block, 0, stream, p);
    }
    return int(hipGetLastError());
}

}  // namespace l3
