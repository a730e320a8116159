// Log-sum-exp combine of the split-KV partials:
//   out = sum_i o_i 2^(m_i - M) / sum_i l_i 2^(m_i - M),   M = max_i m_i
// over the splits i of one (batch, query head).  Takes the place of
// custom_flash_attention_combine_kernel (custom_kernels.cu:179-223), which is meant to do
// this but reads split 0's (max, sum) for every split (:184,201,209) and so returns the plain
// mean of the per-split outputs; here every split contributes its own statistics.
//
// More than 32 splits: one workgroup of eight wavefronts per (batch, query head), or four of them
// (one per quarter of the head dimension) when there are few heads with many splits each; up to 32
// splits: a single wavefront per pair (attn_combine_rows_kernel below).  The kernel is short and
// latency-bound, so it is built around a single round trip to memory: a wavefront issues the
// loads of its (max, sum) pairs AND of its partial rows back to back, before it knows any
// weight, and only then reduces.  Each wavefront merges up to 32 splits per pass with its own
// local maximum; the eight local results are merged through LDS.
#include "attn_merge.hpp"

namespace l3 {

namespace {

constexpr int kCombineWaves = 8;

// CG = column groups: with few (batch, query head) pairs the head dimension is dealt to CG
// workgroups (blockIdx.y), each merging HD / CG columns of every split, so that more than
// B * QH compute units pull the partial rows.
template <int HD, int CG>
__global__ void __launch_bounds__(kCombineWaves * kWaveSize)
attn_combine_kernel(const float* __restrict__ part_o, const float2* __restrict__ part_ml,
                    uint16_t* __restrict__ out, int QH, int n_rows, int64_t o_sb, int64_t o_sh,
                    const int* __restrict__ seqlen_dev, int tokens_per_split) {
    constexpr int TPR = HD / CG / 4;        // lanes covering this workgroup's part of a partial row with float4 loads
    constexpr int RQ = HD / 4;              // float4 per whole partial row
    constexpr int RPL = kWaveSize / TPR;    // rows per wavefront-wide load (2 to 16)
    constexpr int NLD = kCombineRows / RPL; // row loads per pass

    __shared__ float s_m[kCombineWaves];
    __shared__ float s_l[kCombineWaves];
    __shared__ float4 s_acc[kCombineWaves][TPR];

    const int lane = threadIdx.x & (kWaveSize - 1);
    const int wave = threadIdx.x / kWaveSize;
    const int bq = blockIdx.x;
    // rows are laid out for n_rows splits; with a device-side KV length only the first n hold data
    int n = n_rows;
    if (seqlen_dev) n = min(n_rows, max(1, (*seqlen_dev + tokens_per_split - 1) / tokens_per_split));
    const float2* ml = part_ml + int64_t(bq) * n_rows;
    const float4* po = reinterpret_cast<const float4*>(part_o + int64_t(bq) * n_rows * HD);
    const int dq = int(blockIdx.y) * TPR + lane % TPR;
    const int sub = lane / TPR;

    float m_w = kMaskedScore, l_w = 0.f;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    // splits are dealt to the wavefronts in blocks of kCombineRows
    for (int r0 = wave * kCombineRows; r0 < n; r0 += kCombineWaves * kCombineRows) {
        // all loads of the pass first: statistics (lane j < 32 holds split r0 + j) and rows
        float2 st = make_float2(kMaskedScore, 0.f);
        if (lane < kCombineRows && r0 + lane < n) st = ml[r0 + lane];
        float4 x[NLD];
#pragma unroll
        for (int u = 0; u < NLD; ++u) {
            const int r = min(r0 + u * RPL + sub, n - 1);  // rows past the end get weight 0 below
            x[u] = po[int64_t(r) * RQ + dq];
        }
        const float m_new = fmaxf(m_w, wave_max(st.x));
        const float alpha = fast_exp2(m_w - m_new);
        const float wgt = fast_exp2(st.x - m_new);  // absent splits: 2^(-1e30 - m) = 0
        l_w = fmaf(l_w, alpha, wave_sum(st.y * wgt));
        acc.x *= alpha; acc.y *= alpha; acc.z *= alpha; acc.w *= alpha;
        m_w = m_new;
#pragma unroll
        for (int u = 0; u < NLD; ++u) {
            const float w = __shfl(wgt, u * RPL + sub, kWaveSize);
            acc.x = fmaf(w, x[u].x, acc.x);
            acc.y = fmaf(w, x[u].y, acc.y);
            acc.z = fmaf(w, x[u].z, acc.z);
            acc.w = fmaf(w, x[u].w, acc.w);
        }
    }
#pragma unroll
    for (int off = TPR; off < kWaveSize; off <<= 1) {
        acc.x += __shfl_xor(acc.x, off, kWaveSize);
        acc.y += __shfl_xor(acc.y, off, kWaveSize);
        acc.z += __shfl_xor(acc.z, off, kWaveSize);
        acc.w += __shfl_xor(acc.w, off, kWaveSize);
    }
    if (lane < TPR) s_acc[wave][lane] = acc;
    if (lane == 0) {
        s_m[wave] = m_w;
        s_l[wave] = l_w;
    }
    __syncthreads();

    if (threadIdx.x < TPR) {
        float M = s_m[0];
#pragma unroll
        for (int w = 1; w < kCombineWaves; ++w) M = fmaxf(M, s_m[w]);
        float L = 0.f;
        float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int w = 0; w < kCombineWaves; ++w) {
            const float e = fast_exp2(s_m[w] - M);  // idle wavefronts: 0
            const float4 a = s_acc[w][threadIdx.x];
            L = fmaf(s_l[w], e, L);
            t.x = fmaf(a.x, e, t.x);
            t.y = fmaf(a.y, e, t.y);
            t.z = fmaf(a.z, e, t.z);
            t.w = fmaf(a.w, e, t.w);
        }
        const float inv = 1.0f / L;
        uint2 packed;
        packed.x = pack_bf16x2(t.x * inv, t.y * inv);
        packed.y = pack_bf16x2(t.z * inv, t.w * inv);
        const int b = bq / QH;
        const int qh = bq % QH;
        *reinterpret_cast<uint2*>(out + b * o_sb + int64_t(qh) * o_sh + (int(blockIdx.y) * TPR + threadIdx.x) * 4) =
            packed;
    }
}

// At most 32 splits per (batch, query head) pair: one WAVEFRONT per pair, four pairs per workgroup, no
// LDS and no barrier -- with many pairs the eight-wavefront form above would launch thousands of
// workgroups that each merge two or three rows, with few it waits at its barrier for nothing.  The merge itself
// (merge_pair_rows) is shared with the split kernel's single-launch form, so both give the same bits.
template <int HD>
__global__ void __launch_bounds__(4 * kWaveSize)
attn_combine_rows_kernel(const float* __restrict__ part_o, const float2* __restrict__ part_ml,
                         uint16_t* __restrict__ out, int QH, int n_rows, int64_t total_pairs, int64_t o_sb,
                         int64_t o_sh, const int* __restrict__ seqlen_dev, int tokens_per_split, int producer_groups) {
    const int wave = threadIdx.x / kWaveSize;
    // A workgroup takes four consecutive pairs.  Workgroups go to the eight XCDs in turn (id % 8), each with an L2
    // of its own, and so did the streaming split kernel's: its workgroup (head group g of G, batch b, split group z)
    // has id g + G (b + B z), so with G B a multiple of 8 every partial row of a (batch, head group) was written
    // through ONE XCD's L2.  producer_groups = G then deals the pairs so that they are merged on that XCD
    // (B 16 x 4096 tokens: combine 2.55 -> 2.31 us); 0 = plain order.
    int64_t unit = blockIdx.x;
    if (producer_groups > 0) {
        const int U = QH / producer_groups / 4;        // workgroups per (batch, head group)
        const int x = int(blockIdx.x) % 8;
        const int64_t y = int64_t(blockIdx.x) / 8;
        const int64_t i = x + 8 * (y / U);             // (batch, head group) in the split kernel's launch order
        unit = (i / producer_groups) * (QH / 4) + (i % producer_groups) * U + y % U;
    }
    const int64_t bq = unit * 4 + wave;
    if (bq >= total_pairs) return;   // whole wavefront; the kernel has no barrier
    int n = n_rows;
    if (seqlen_dev) n = min(n_rows, max(1, (*seqlen_dev + tokens_per_split - 1) / tokens_per_split));
    const int64_t b = bq / QH;
    const int qh = int(bq % QH);
    merge_pair_rows<HD, PlainReader>(part_o + bq * n_rows * HD, part_ml + bq * n_rows, n,
                                     out + b * o_sb + int64_t(qh) * o_sh);
}

}  // namespace

int launch_attn_combine(const AttnParams& p, int HD, int producer_groups, hipStream_t stream) {
    const int64_t pairs = int64_t(p.B) * p.QH;
    // At most 32 splits: a wavefront per (batch, head) pair, whatever the number of pairs (32 pairs of 8 ... 32
    // splits: 0.6-0.7 us less per call than a workgroup per pair, which waits at a barrier for seven
    // wavefronts that have nothing to merge).
    if (p.num_splits <= kCombineRows) {
        const dim3 rgrid{unsigned((pairs + 3) / 4)};
        const dim3 rblock{4 * kWaveSize};
        // the XCD-local order needs whole groups of four pairs per head group and as many units on every XCD
        const int G = producer_groups;
        const int xg = (G > 0 && p.QH % (4 * G) == 0 && (int64_t(G) * p.B) % 8 == 0) ? G : 0;
        if (HD == 64) {
            hipLaunchKernelGGL((attn_combine_rows_kernel<64>), rgrid, rblock, 0, stream, p.part_o, p.part_ml, p.out,
                               p.QH, p.num_splits, pairs, p.o_sb, p.o_sh, p.seqlen_dev, p.tokens_per_split, xg);
        } else {
            hipLaunchKernelGGL((attn_combine_rows_kernel<128>), rgrid, rblock, 0, stream, p.part_o, p.part_ml, p.out,
                               p.QH, p.num_splits, pairs, p.o_sb, p.o_sh, p.seqlen_dev, p.tokens_per_split, xg);
        }
        return int(hipGetLastError());
    }
    const bool few = int64_t(p.B) * p.QH <= 64 && p.num_splits > kCombineRows;   // few heads, many rows each
    const dim3 grid(unsigned(p.B) * unsigned(p.QH), few ? 4u : 1u);
    const dim3 block(kCombineWaves * kWaveSize);
    if (HD == 64 && few) {
        hipLaunchKernelGGL((attn_combine_kernel<64, 4>), grid, block, 0, stream, p.part_o, p.part_ml, p.out, p.QH,
                           p.num_splits, p.o_sb, p.o_sh, p.seqlen_dev, p.tokens_per_split);
    } else if (HD == 64) {
        hipLaunchKernelGGL((attn_combine_kernel<64, 1>), grid, block, 0, stream, p.part_o, p.part_ml, p.out, p.QH,
                           p.num_splits, p.o_sb, p.o_sh, p.seqlen_dev, p.tokens_per_split);
    } else if (few) {
        hipLaunchKernelGGL((attn_combine_kernel<128, 4>), grid, block, 0, stream, p.part_o, p.part_ml, p.out, p.QH,
                           p.num_splits, p.o_sb, p.o_sh, p.seqlen_dev, p.tokens_per_split);
    } else {
        hipLaunchKernelGGL((attn_combine_kernel<128, 1>), grid, block, 0, stream, p.part_o, p.part_ml, p.out, p.QH,
                           p.num_splits, p.o_sb, p.o_sh, p.seqlen_dev, p.tokens_per_split);
    }
    return int(hipGetLastError());
}

}  // namespace l3
