// Split-KV decode attention on the gfx950 matrix cores (the default kernel).
//
// Replaces custom_flash_attention_splitkv_kernel (custom_kernels.cu:13-177).  The tile loop (MFMA
// products, LDS slab, online softmax) is in attn_mfma_core.hpp; here are the two ways work is
// laid over wavefronts.
//
// Streaming form: the unit of work is one wavefront -- a (batch, kv head, token range) it streams
// alone, start to finish, so the kernel has no workgroup barrier at all.  A workgroup is eight
// such wavefronts laid side by side over the kv heads of one token range: in the token-major KV
// cache (model.py:89) the eight 256-byte head slices of a token are contiguous, so together the
// wavefronts read whole 2 KiB token rows, which measured ~8 % more HBM bandwidth than giving each
// head its own workgroup.  With fewer than eight kv heads the remaining wavefronts take further
// token ranges of the same heads.
//
// The 16 columns of the MFMA tiles carry the R <= 8 query heads of the GQA group (columns R..15
// are zero padding; the matrix cores have room to spare on a memory-bound kernel), so each K/V
// byte is fetched once per group.
#include "attn_merge.hpp"
#include "attn_mfma_core.hpp"

namespace l3 {

namespace {

// COOP = false: the streaming form described above (a wavefront per head and token range).
// COOP = true: the short-sequence form.  All eight wavefronts of a workgroup work on ONE
// (batch, kv head, token range), taking its tiles in turn, and merge their softmax states
// through LDS at the end; with a single split per head the workgroup writes the final output and
// no combine kernel runs.  It trades the contiguous-row access of the streaming form for eight
// times the parallelism per head, which is what a latency-bound call (a few tiles per head) needs.
// LOADS = 4 (head size 64, cooperative form, at most 512 tokens): half-size tiles of 32 tokens, so
// that a short sequence still gives every wavefront a tile, and slabs small enough for two
// workgroups per CU.
template <int HD, bool COOP, int LOADS = 8>
__global__ void __launch_bounds__(kMfmaWaves * kWaveSize, 2)
attn_splitkv_mfma_kernel(const int R, const int hpw_log2, const AttnParams p) {
    using T = MfmaTile<HD, LOADS>;
    constexpr int WT = T::WT, KC = T::KC, NB = T::NB, SLAB = T::SLAB;
    constexpr int STEP = COOP ? kMfmaWaves * WT : WT;  // token stride between a wavefront's tiles
    static_assert(LOADS != 8 || WT == attn_tile_tokens(HD, kAttnImplMfma), "host plan and kernel tile disagree");
    static_assert(LOADS == 8 || COOP, "the split plan counts full tiles");

    __shared__ __align__(16) unsigned char s_slab[kMfmaWaves][SLAB];

    const int lane = threadIdx.x & (kWaveSize - 1);
    const int wave = wave_uniform(int(threadIdx.x) / kWaveSize);   // scalar: everything derived from it is wave-uniform
    const int fn = lane & 15;        // role in an MFMA operand: row/column index ...
    const int fg = lane >> 4;        // ... and k group

    // Grid: x = kv head (COOP) or group of 2^hpw_log2 adjacent kv heads, y = batch, z = split (COOP)
    // or group of splits -- no division on the way to the first load.
    const int b = blockIdx.y;
    int kvh, split;
    if constexpr (COOP) {
        kvh = blockIdx.x;
        split = blockIdx.z;
    } else {
        // the eight wavefronts -> 2^hpw_log2 heads x (8 >> hpw_log2) consecutive splits
        kvh = (int(blockIdx.x) << hpw_log2) + (wave & ((1 << hpw_log2) - 1));
        split = (int(blockIdx.z) << (3 - hpw_log2)) + (wave >> hpw_log2);
    }
    const int t_begin = split * p.tokens_per_split;
    const int S = p.seqlen_dev ? max(1, min(*p.seqlen_dev, p.S)) : p.S;  // wave-uniform; a length below 1 counts as 1
    // Single-launch form (cooperative workgroups with p.arrive set): the workgroup that finishes a (batch,
    // kv head) last merges its partials, and every split of the plan is counted as an arrival -- also one
    // that a device-side KV length leaves without tokens (it streams and writes nothing, the merge skips its row).
    const bool merge_here = COOP && p.arrive != nullptr;
    // A split past the plan (last workgroup of the streaming form: whole wavefront, no barrier follows)
    // or, with a combine launch to follow, past a device-side KV length (whole workgroup when COOP).
    if (split >= p.num_splits || (!merge_here && t_begin >= S)) return;
    const bool has_tokens = t_begin < S;
    const int t_end = min(S, t_begin + p.tokens_per_split);
    const float c = p.scale_log2e;

    // B operand of the first product: lane (head fn, k group fg) holds q[head][(m*4+fg)*8 .. +8].
    bf16x8_t qfrag[KC];
#pragma unroll
    for (int m = 0; m < KC; ++m) {
        uint4 qv = make_uint4(0u, 0u, 0u, 0u);
        if (fn < R) qv = load16(p.q + b * p.q_sb + int64_t(kvh * R + fn) * p.q_sh + (m * 4 + fg) * 8);
        qfrag[m] = __builtin_bit_cast(bf16x8_t, qv);
    }

    const int64_t k_head = b * p.k_sb + kvh * p.k_sh;   // token 0 of this kv head, in elements
    const int64_t v_head = b * p.v_sb + kvh * p.v_sh;

    f32x4_t O[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) O[nb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = kMaskedScore;  // running maximum of the raw scores (common to the four k groups of a head)
    float l_part = 0.f;          // this lane's share of the softmax denominator
    // Cooperative workgroups take their tiles in an order rotated by the split index: the splits of a head
    // start a power of two apart (1 MiB at 16384 tokens in 32 splits), and 32 workgroups that walk such
    // ranges in step keep hitting the same memory channels (16384 tokens: 16.3 -> 14.9 us at head size 128,
    // 12.2 -> 10.0 us at 64).  The streaming form, whose split counts are not powers of two, gains nothing.
    mfma_tile_loop<HD, LOADS, true, COOP>(p.k, p.v, k_head, v_head, p.k_st, p.v_st, s_slab[wave], qfrag,
                                          t_begin + (COOP ? wave * WT : 0), t_end, STEP, t_end, t_end, c, O, m_run, l_part,
                                          t_begin, split);

    // ---- this wavefront's result.  O[nb][r] is dim 16*nb + 4*fg + r of head fn; the softmax
    //      denominator is still spread over the four k groups.
    l_part += __shfl_xor(l_part, 16, kWaveSize);
    l_part += __shfl_xor(l_part, 32, kWaveSize);
    const float m_log2 = (m_run == kMaskedScore) ? kMaskedScore : m_run * c;  // a COOP wave may have had no tile

    if constexpr (COOP) {
        // merge the eight wavefronts through LDS, then write like the streaming form
        __shared__ float s_m[kMfmaWaves][kAttnMaxRatio];
        __shared__ float s_l[kMfmaWaves][kAttnMaxRatio];
        __shared__ __align__(16) float s_o[kMfmaWaves][kAttnMaxRatio][HD];
        __shared__ int s_last;
        if (fn < R) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                *reinterpret_cast<float4*>(&s_o[wave][fn][nb * 16 + fg * 4]) =
                    make_float4(O[nb][0], O[nb][1], O[nb][2], O[nb][3]);
            }
            if (fg == 0) {
                s_m[wave][fn] = m_log2;
                s_l[wave][fn] = l_part;
            }
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < R * (HD / 2); idx += kMfmaWaves * kWaveSize) {
            const int h = idx / (HD / 2);
            const int d = (idx % (HD / 2)) * 2;
            float M = s_m[0][h];
#pragma unroll
            for (int w = 1; w < kMfmaWaves; ++w) M = fmaxf(M, s_m[w][h]);
            float L = 0.f, o0 = 0.f, o1 = 0.f;
#pragma unroll
            for (int w = 0; w < kMfmaWaves; ++w) {
                const float e = fast_exp2(s_m[w][h] - M);  // wavefronts without a tile: 0
                L = fmaf(s_l[w][h], e, L);
                o0 = fmaf(s_o[w][h][d], e, o0);
                o1 = fmaf(s_o[w][h][d + 1], e, o1);
            }
            const int qh = kvh * R + h;
            if (p.part_o == nullptr) {
                const float inv = 1.0f / L;
                *reinterpret_cast<uint32_t*>(p.out + b * p.o_sb + int64_t(qh) * p.o_sh + d) =
                    pack_bf16x2(o0 * inv, o1 * inv);
            } else if (has_tokens) {
                const int64_t row = attn_partial_row(p, b, qh, split);
                *reinterpret_cast<float2*>(p.part_o + row * HD + d) = make_float2(o0, o1);
                if (d == 0) p.part_ml[row] = make_float2(M, L);
            }
        }
        if (merge_here) {
            // the workgroup that arrives last at its (batch, kv head) merges the head's partial rows out of
            // the XCD's L2: the eight wavefronts share the R query heads, 8 / R column groups per head
            wait_stores_in_l2();
            __syncthreads();
            if (threadIdx.x == 0) {
                bool same_xcd = true;
                s_last = arrive_is_last(p.arrive + (int64_t(b) * p.KVH + kvh) * kAttnArriveStride, p.num_splits, &same_xcd);
                if (!same_xcd) atomicAdd(p.arrive + kAttnDiagSlot * kAttnArriveStride, 1u);
            }
            __syncthreads();
            if (s_last) {
                const int n = min(p.num_splits, (S + p.tokens_per_split - 1) / p.tokens_per_split);
                auto merge = [&](auto cgs) {
                    constexpr int CG = decltype(cgs)::value;
                    const int qh = kvh * R + wave / CG;
                    const int64_t row0 = attn_partial_row(p, b, qh, 0);
                    merge_pair_rows<HD, L2Reader, CG>(p.part_o + row0 * HD, p.part_ml + row0, n,
                                                      p.out + b * p.o_sb + int64_t(qh) * p.o_sh, wave % CG);
                };
                if (R == 8) merge(std::integral_constant<int, 1>{});
                else if (R == 4) merge(std::integral_constant<int, 2>{});
                else if (R == 2) merge(std::integral_constant<int, 4>{});
                else if (R == 1) merge(std::integral_constant<int, 8>{});
                else if (wave < R) merge(std::integral_constant<int, 1>{});   // R = 3
            }
        }
    } else if (fn < R) {
        const int qh = kvh * R + fn;
        if (p.part_o == nullptr) {  // single split: the final output row
            const float inv = 1.0f / l_part;
            uint16_t* orow = p.out + b * p.o_sb + int64_t(qh) * p.o_sh + fg * 4;
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                uint2 w;
                w.x = pack_bf16x2(O[nb][0] * inv, O[nb][1] * inv);
                w.y = pack_bf16x2(O[nb][2] * inv, O[nb][3] * inv);
                *reinterpret_cast<uint2*>(orow + nb * 16) = w;
            }
        } else {
            // unnormalised float32 partial and its (max in log2 units, sum) for the combine
            const int64_t row = attn_partial_row(p, b, qh, split);
            float* prow = p.part_o + row * HD + fg * 4;
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                *reinterpret_cast<float4*>(prow + nb * 16) = make_float4(O[nb][0], O[nb][1], O[nb][2], O[nb][3]);
            }
            if (fg == 0) p.part_ml[row] = make_float2(m_log2, l_part);
        }
    }
}

// Workgroup i of a 1-D grid reports the XCD it runs on.
__global__ void xcd_probe_kernel(unsigned* where, int stride_words) {
    if (threadIdx.x == 0) where[int64_t(blockIdx.x) * stride_words] = xcc_id();
}

__global__ void fill_zero_u32_kernel(unsigned* dst, size_t n) {
    const size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = 0u;
}

}  // namespace

int launch_xcd_probe(unsigned* where, int n, int stride_words, hipStream_t stream) {
    hipLaunchKernelGGL(xcd_probe_kernel, dim3(unsigned(n)), dim3(kWaveSize), 0, stream, where, stride_words);
    return int(hipGetLastError());
}

int launch_fill_zero_u32(unsigned* dst, size_t n, hipStream_t stream) {
    hipLaunchKernelGGL(fill_zero_u32_kernel, dim3(unsigned((n + 255) / 256)), dim3(256), 0, stream, dst, n);
    return int(hipGetLastError());
}

bool attn_mfma_can_merge_in_launch(int B, int KVH, bool coop, int num_splits) {
    // Cooperative form only: a workgroup per (batch, kv head, split) with linear id kvh + KVH (b + B split),
    // and a last arriver that merges in one pass.  (In the streaming form the arrivals would be single
    // wavefronts; built and measured on 16 sequences of 4096 tokens, a lone wavefront merging its head's four
    // query heads took longer than the combine launch it saved: 25.0 against 24.5 us.)
    if (!coop || num_splits < 2 || num_splits > kCombineRows) return false;
    if (B > 65535 || int64_t(B) * KVH > kAttnDiagSlot) return false;   // one launch, one counter per (batch, kv head)
    return (int64_t(KVH) * B) % 8 == 0;
}

int attn_mfma_heads_per_wg(int KVH) {
    for (int h = kMfmaWaves; h > 1; h /= 2) {
        if (KVH % h == 0) return h;
    }
    return 1;
}

int launch_attn_splitkv_mfma(const AttnParams& params, int HD, int R, bool coop, hipStream_t stream) {
    if (R < 1 || R > kAttnMaxRatio) return int(hipErrorInvalidValue);
    const dim3 block(kMfmaWaves * kWaveSize);
    const int hpw = attn_mfma_heads_per_wg(params.KVH);
    int hpw_log2 = 0;
    while ((1 << hpw_log2) < hpw) ++hpw_log2;
    const int spw = kMfmaWaves / hpw;
    // The batch index is the grid's y dimension (at most 65535): larger batches go out in slices, each
    // with its pointers moved to the slice's first sequence.
    constexpr int kMaxGridY = 65535;
    for (int b0 = 0; b0 < params.B; b0 += kMaxGridY) {
        AttnParams p = params;
        p.B = (params.B - b0 < kMaxGridY) ? params.B - b0 : kMaxGridY;
        p.q += b0 * p.q_sb;
        p.k += b0 * p.k_sb;
        p.v += b0 * p.v_sb;
        if (p.out) p.out += b0 * p.o_sb;
        if (p.part_o) {
            const int64_t row0 = int64_t(b0) * p.QH * p.num_splits;
            p.part_o += row0 * HD;
            p.part_ml += row0;
        }
        if (coop) {
            const dim3 grid(unsigned(p.KVH), unsigned(p.B), unsigned(p.num_splits));
            if (HD == 64 && p.tokens_per_split <= 2 * kMfmaWaves * 32) {
                hipLaunchKernelGGL((attn_splitkv_mfma_kernel<64, true, 4>), grid, block, 0, stream, R, 0, p);
            } else if (HD == 64) {
                hipLaunchKernelGGL((attn_splitkv_mfma_kernel<64, true>), grid, block, 0, stream, R, 0, p);
            } else {
                hipLaunchKernelGGL((attn_splitkv_mfma_kernel<128, true>), grid, block, 0, stream, R, 0, p);
            }
        } else {
            const dim3 grid(unsigned(p.KVH / hpw), unsigned(p.B), unsigned((p.num_splits + spw - 1) / spw));
            if (HD == 64) {
                hipLaunchKernelGGL((attn_splitkv_mfma_kernel<64, false>), grid, block, 0, stream, R, hpw_log2, p);
            } else {
                hipLaunchKernelGGL((attn_splitkv_mfma_kernel<128, false>), grid, block, 0, stream, R, hpw_log2, p);
            }
        }
        if (const hipError_t e = hipGetLastError(); e != hipSuccess) return int(e);
    }
    return 0;
}

}  // namespace l3
