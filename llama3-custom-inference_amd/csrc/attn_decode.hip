// Split-KV decode attention for gfx950 (wave64) with FMA dot products on the vector ALUs.
// This is the comparison kernel: the MFMA kernel (attn_mfma.hip) is the default because it
// measured faster; this one stays selectable so that the comparison can be repeated.
//
// Takes the place of custom_flash_attention_splitkv_kernel (custom_kernels.cu:13-177).
// What differs from it, by design:
//   * one workgroup (4 wavefronts) owns a (batch, kv head, token range) whose length the
//     host picks from the problem and the device, not a fixed 64 tokens;
//   * inside a workgroup every wavefront streams its own tiles with 16-byte loads, each
//     load covering whole token rows (HD/8 lanes per row), double-buffered in registers;
//   * the R query heads that share the kv head are scored against every K row while it is
//     in registers, so each K/V byte leaves HBM once per GQA group;
//   * each group of HD/8 lanes keeps a private online softmax (running max, sum and
//     output slice); the groups, then the wavefronts, are merged once at the end;
//   * partials handed to the combine are float32 and unnormalised (the reference rounds
//     them to bf16, custom_kernels.cu:163).
#include "attn_common.hpp"

namespace l3 {

namespace {

constexpr int kAttnWaves = 4;
constexpr int kAttnUnroll = 4;            // 16-byte loads of K (and of V) in flight per lane and tile

// LDS hand-over between the wavefronts of a workgroup: per wave and query head of the group,
// the running maximum (log2 units), the sum of exp2 and the unnormalised output row.
template <int HD, int R>
struct AttnMergeBuffers {
    float m[kAttnWaves][R];
    float l[kAttnWaves][R];
    alignas(16) float o[kAttnWaves][R][HD];
};

template <int HD, int R>
__global__ void __launch_bounds__(kAttnWaves * kWaveSize)
attn_splitkv_fma_kernel(const AttnParams p) {
    constexpr int U = kAttnUnroll;
    constexpr int LPR = HD / 8;          // lanes covering one token row
    constexpr int G = kWaveSize / LPR;   // token rows per wavefront-wide load
    constexpr int WT = U * G;            // tokens per wavefront tile
    constexpr int STEP = kAttnWaves * WT;
    static_assert(STEP == attn_tile_tokens(HD, kAttnImplFma), "host plan and kernel tile disagree");

    const int lane = threadIdx.x & (kWaveSize - 1);
    const int wave = threadIdx.x / kWaveSize;
    const int g = lane / LPR;
    const int c = lane % LPR;

    int bid = blockIdx.x;
    const int kvh = bid % p.KVH;
    bid /= p.KVH;
    const int b = bid % p.B;
    const int split = bid / p.B;
    const int t_begin = split * p.tokens_per_split;
    const int S = p.seqlen_dev ? max(1, min(*p.seqlen_dev, p.S)) : p.S;  // wave-uniform; a length below 1 counts as 1
    if (t_begin >= S) return;  // whole workgroup: split beyond a device-side KV length, the combine skips it
    const int t_end = min(S, t_begin + p.tokens_per_split);

    // Query slices for the R heads of this group, pre-multiplied by scale*log2(e).
    float qf[R][8];
#pragma unroll
    for (int h = 0; h < R; ++h) {
        const uint4 qv = load16(p.q + b * p.q_sb + int64_t(kvh * R + h) * p.q_sh + c * 8);
        unpack8(qv, qf[h]);
#pragma unroll
        for (int i = 0; i < 8; ++i) qf[h][i] *= p.scale_log2e;
    }

    const uint16_t* kbase = p.k + b * p.k_sb + kvh * p.k_sh + c * 8;
    const uint16_t* vbase = p.v + b * p.v_sb + kvh * p.v_sh + c * 8;

    float m[R], l[R], acc[R][8];
#pragma unroll
    for (int h = 0; h < R; ++h) {
        m[h] = kMaskedScore;
        l[h] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[h][i] = 0.f;
    }

    // Rows past the end of the split are clamped to its last row (a valid address) and
    // masked out of the softmax below.
    auto issue = [&](uint4 (&kr)[U], uint4 (&vr)[U], int tbase) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int tok = min(tbase + u * G + g, t_end - 1);
            kr[u] = load16_stream(kbase + int64_t(tok) * p.k_st);   // K/V are read once: a stream
            vr[u] = load16_stream(vbase + int64_t(tok) * p.v_st);
        }
    };

    auto consume = [&](const uint4 (&kr)[U], const uint4 (&vr)[U], int tbase) {
        float s[U][R];
        bool valid[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float kf[8];
            unpack8(kr[u], kf);
            valid[u] = (tbase + u * G + g) < t_end;
#pragma unroll
            for (int h = 0; h < R; ++h) {
                float d = 0.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) d = fmaf(qf[h][i], kf[i], d);
                d = group_sum<LPR>(d);
                s[u][h] = valid[u] ? d : kMaskedScore;
            }
        }
#pragma unroll
        for (int h = 0; h < R; ++h) {
            float mx = m[h];
#pragma unroll
            for (int u = 0; u < U; ++u) mx = fmaxf(mx, s[u][h]);
            const float alpha = fast_exp2(m[h] - mx);
            m[h] = mx;
            float psum = 0.f;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const float pu = valid[u] ? fast_exp2(s[u][h] - mx) : 0.f;
                s[u][h] = pu;
                psum += pu;
            }
            l[h] = fmaf(l[h], alpha, psum);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[h][i] *= alpha;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float vf[8];
            unpack8(vr[u], vf);
#pragma unroll
            for (int h = 0; h < R; ++h) {
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[h][i] = fmaf(s[u][h], vf[i], acc[h][i]);
            }
        }
    };

    // Register double buffer: the loads of the next tile are in flight while this one is consumed.
    {
        uint4 ka[U], va[U], kb[U], vb[U];
        int t0 = t_begin + wave * WT;
        issue(ka, va, t0);
        while (true) {
            issue(kb, vb, t0 + STEP);
            consume(ka, va, t0);
            t0 += STEP;
            if (t0 >= t_end) break;
            issue(ka, va, t0 + STEP);
            consume(kb, vb, t0);
            t0 += STEP;
            if (t0 >= t_end) break;
        }
    }

    // ---- merge the G lane groups of this wavefront (cross-row moves go through ds_bpermute)
#pragma unroll
    for (int h = 0; h < R; ++h) {
        float mw = m[h];
#pragma unroll
        for (int off = LPR; off < kWaveSize; off <<= 1) mw = fmaxf(mw, __shfl_xor(mw, off, kWaveSize));
        const float a = fast_exp2(m[h] - mw);
        m[h] = mw;
        l[h] *= a;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[h][i] *= a;
#pragma unroll
        for (int off = LPR; off < kWaveSize; off <<= 1) {
            l[h] += __shfl_xor(l[h], off, kWaveSize);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[h][i] += __shfl_xor(acc[h][i], off, kWaveSize);
        }
    }

    // ---- merge the wavefronts through LDS
    __shared__ AttnMergeBuffers<HD, R> s_merge;
    if (g == 0) {
#pragma unroll
        for (int h = 0; h < R; ++h) {
            float4* dst = reinterpret_cast<float4*>(&s_merge.o[wave][h][c * 8]);
            dst[0] = make_float4(acc[h][0], acc[h][1], acc[h][2], acc[h][3]);
            dst[1] = make_float4(acc[h][4], acc[h][5], acc[h][6], acc[h][7]);
        }
        if (c == 0) {
#pragma unroll
            for (int h = 0; h < R; ++h) {
                s_merge.m[wave][h] = m[h];
                s_merge.l[wave][h] = l[h];
            }
        }
    }
    __syncthreads();

    // Single split: the normalised bf16 output row; otherwise the unnormalised float32 partial
    // and its (max, sum) for the combine kernel.
    for (int idx = threadIdx.x; idx < R * HD; idx += kAttnWaves * kWaveSize) {
        const int h = idx / HD;
        const int d = idx % HD;
        float M = s_merge.m[0][h];
#pragma unroll
        for (int w = 1; w < kAttnWaves; ++w) M = fmaxf(M, s_merge.m[w][h]);
        float L = 0.f, o = 0.f;
#pragma unroll
        for (int w = 0; w < kAttnWaves; ++w) {
            const float e = fast_exp2(s_merge.m[w][h] - M);
            L = fmaf(s_merge.l[w][h], e, L);
            o = fmaf(s_merge.o[w][h][d], e, o);
        }
        const int qh = kvh * R + h;
        if (p.part_o == nullptr) {  // single split: the final output row
            p.out[b * p.o_sb + int64_t(qh) * p.o_sh + d] = uint16_t(f32_to_bf16_bits(o / L));
        } else {
            const int64_t row = attn_partial_row(p, b, qh, split);
            p.part_o[row * HD + d] = o;
            if (d == 0) p.part_ml[row] = make_float2(M, L);
        }
    }
}

template <int HD, int R>
int launch_split(const AttnParams& p, hipStream_t stream) {
    const dim3 grid(unsigned(p.B) * unsigned(p.KVH) * unsigned(p.num_splits));
    hipLaunchKernelGGL((attn_splitkv_fma_kernel<HD, R>), grid, dim3(kAttnWaves * kWaveSize), 0, stream, p);
    return int(hipGetLastError());
}

template <int HD>
int launch_for_ratio(const AttnParams& p, int R, hipStream_t stream) {
    switch (R) {
        case 1: return launch_split<HD, 1>(p, stream);
        case 2: return launch_split<HD, 2>(p, stream);
        case 3: return launch_split<HD, 3>(p, stream);
        case 4: return launch_split<HD, 4>(p, stream);
        case 8: return launch_split<HD, 8>(p, stream);
        default: return int(hipErrorInvalidValue);
    }
}

}  // namespace

int launch_attn_splitkv_fma(const AttnParams& p, int HD, int R, hipStream_t stream) {
    return (HD == 64) ? launch_for_ratio<64>(p, R, stream) : launch_for_ratio<128>(p, R, stream);
}

}  // namespace l3
