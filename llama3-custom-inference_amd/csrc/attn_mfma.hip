// Split-KV decode attention on the gfx950 matrix cores (the default kernel).
//
// Replaces custom_flash_attention_splitkv_kernel (custom_kernels.cu:13-177).  The unit of
// work is one wavefront: a (batch, kv head, token range) triple it streams alone, start to
// finish, so the kernel has no workgroup barrier at all.  A workgroup is eight such
// wavefronts laid side by side over the kv heads of one token range: in the token-major KV
// cache (model.py:89) the eight 256-byte head slices of a token are contiguous, so together
// the wavefronts read whole 2 KiB token rows, which measured ~8 % more HBM bandwidth than
// giving each head its own workgroup.  With fewer than eight kv heads the remaining
// wavefronts take further token ranges of the same heads.
//
// The two products run as v_mfma_f32_16x16x32_bf16 tiles:
//
//   S[16 tokens x 16 heads]  = K[16 x 32 dims]        . Q^T[32 dims x 16 heads]   (per 32-dim chunk)
//   O^T[16 dims x 16 heads] += V^T[16 dims x 32 tok.] . P[32 tokens x 16 heads]  (per 16-dim block)
//
// The head axis carries the R <= 8 query heads of the GQA group (columns R..15 are zero
// padding; the matrix cores have room to spare on a memory-bound kernel), so each K/V byte
// is fetched once per group.  A wavefront loads its tile with 16-byte global loads that each
// cover whole head rows, writes it to its private LDS slab and reads it back in the operand
// layouts: ds_read_b128 for K (lane = token row, 8 consecutive dims), ds_read_b64_tr_b16 for
// V, whose transpose turns token-major rows into "8 tokens of one dim" per lane.  The slab
// rows are padded (16 bytes for K, 32 for V) to keep both read patterns off the same banks.
// The S accumulator layout (lane = head column, 4 token rows) is exactly the B-operand layout
// of the second product, so P never moves between lanes.  LDS executes one wavefront's
// accesses in order, which is all the synchronisation the slab needs.
#include "attn_common.hpp"

namespace l3 {

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(8))) short s16x8_t;

#define L3_LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))

// Keeps the compiler from moving LDS accesses across a phase boundary of the slab (the
// hardware already executes one wavefront's LDS accesses in order).
__device__ __forceinline__ void lds_phase_fence() { asm volatile("" ::: "memory"); }

// COOP = false: the streaming form described above (a wavefront per head and token range).
// COOP = true: the short-sequence form.  All eight wavefronts of a workgroup work on ONE
// (batch, kv head, token range), taking its tiles in turn, and merge their softmax states
// through LDS at the end; with a single split per head the workgroup writes the final output and
// no combine kernel runs.  It trades the contiguous-row access of the streaming form for eight
// times the parallelism per head, which is what a latency-bound call (a few tiles per head) needs.
template <int HD, bool COOP>
__global__ void __launch_bounds__(kMfmaWaves * kWaveSize, 2)
attn_splitkv_mfma_kernel(const AttnParams p, const int R, const int heads_per_wg) {
    constexpr int LPR = HD / 8;            // lanes per token row in a global load
    constexpr int G = kWaveSize / LPR;     // token rows per wavefront-wide load
    constexpr int U = 8;                   // loads of K (and of V) per tile and lane
    constexpr int WT = U * G;              // tokens per wavefront tile: 32 (HD 128) or 64 (HD 64)
    constexpr int NG = WT / 16;            // 16-token groups per tile (rows of one S tile)
    constexpr int KC = HD / 32;            // 32-dim chunks of the head dimension
    constexpr int NB = HD / 16;            // 16-dim blocks of the output
    constexpr int KS = WT / 32;            // 32-token steps of the second product
    constexpr int KPITCH = HD * 2 + 16;    // slab row pitch while it holds K
    constexpr int VPITCH = HD * 2 + 32;    // slab row pitch while it holds V
    constexpr int SLAB = WT * VPITCH;
    constexpr int STEP = COOP ? kMfmaWaves * WT : WT;  // token stride between a wavefront's tiles
    static_assert(WT == attn_tile_tokens(HD, kAttnImplMfma), "host plan and kernel tile disagree");

    __shared__ __align__(16) unsigned char s_slab[kMfmaWaves][SLAB];

    const int lane = threadIdx.x & (kWaveSize - 1);
    const int wave = threadIdx.x / kWaveSize;
    const int ld_row = lane / LPR;   // role in a global load: token row within the load ...
    const int ld_c = lane % LPR;     // ... and 16-byte chunk of that row
    const int fn = lane & 15;        // role in an MFMA operand: row/column index ...
    const int fg = lane >> 4;        // ... and k group

    int b, kvh, split;
    if constexpr (COOP) {
        // workgroup -> (batch, kv head, split), kv head fastest
        int bid = blockIdx.x;
        kvh = bid % p.KVH;
        bid /= p.KVH;
        b = bid % p.B;
        split = bid / p.B;
    } else {
        // workgroup -> (batch, group of heads_per_wg adjacent kv heads, group of splits); its eight
        // wavefronts -> heads_per_wg heads x (8 / heads_per_wg) consecutive splits
        const int head_groups = p.KVH / heads_per_wg;
        const int splits_per_wg = kMfmaWaves / heads_per_wg;
        int bid = blockIdx.x;
        const int hg = bid % head_groups;
        bid /= head_groups;
        b = bid % p.B;
        const int sg = bid / p.B;
        kvh = hg * heads_per_wg + wave % heads_per_wg;
        split = sg * splits_per_wg + wave / heads_per_wg;
        if (split >= p.num_splits) return;  // whole wavefront; no barrier follows
    }
    const int t_begin = split * p.tokens_per_split;
    const int S = p.seqlen_dev ? min(*p.seqlen_dev, p.S) : p.S;  // wave-uniform
    if (t_begin >= S) return;  // split beyond a device-side KV length (whole workgroup when COOP): the combine skips it
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

    const uint16_t* kbase = p.k + b * p.k_sb + kvh * p.k_sh + ld_c * 8;
    const uint16_t* vbase = p.v + b * p.v_sb + kvh * p.v_sh + ld_c * 8;

    unsigned char* slab = s_slab[wave];
    unsigned char* wr_k = slab + ld_row * KPITCH + ld_c * 16;
    unsigned char* wr_v = slab + ld_row * VPITCH + ld_c * 16;
    const unsigned char* rd_k = slab + fn * KPITCH + fg * 16;
    // transpose read: the 16 lanes of k group fg present a 4-token x 16-dim patch, row-major
    const unsigned char* rd_v = slab + (4 * fg + (fn >> 2)) * VPITCH + (fn & 3) * 8;

    f32x4_t O[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) O[nb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = kMaskedScore;  // running maximum of the raw scores (common to the four k groups of a head)
    float l_part = 0.f;          // this lane's share of the softmax denominator

    uint4 kr[U], vr[U];
    auto issue_k = [&](int tbase) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int tok = min(tbase + u * G + ld_row, t_end - 1);  // clamped rows are masked below
            kr[u] = load16(kbase + int64_t(tok) * p.k_st);
        }
    };
    auto issue_v = [&](int tbase) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int tok = min(tbase + u * G + ld_row, t_end - 1);
            vr[u] = load16(vbase + int64_t(tok) * p.v_st);
        }
    };

    int t0 = t_begin + (COOP ? wave * WT : 0);
    issue_k(t0);
    issue_v(t0);
    for (; t0 < t_end; t0 += STEP) {
        const int tn = t0 + STEP;

        // ---- K tile -> slab; its registers are free again, so the next K tile starts loading
#pragma unroll
        for (int u = 0; u < U; ++u) *reinterpret_cast<uint4*>(wr_k + u * G * KPITCH) = kr[u];
        lds_phase_fence();
        if (tn < t_end) issue_k(tn);

        // ---- S = K Q^T
        f32x4_t S[NG];
#pragma unroll
        for (int tg = 0; tg < NG; ++tg) {
            S[tg] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int m = 0; m < KC; ++m) {
                const uint4 a = *reinterpret_cast<const uint4*>(rd_k + tg * 16 * KPITCH + m * 64);
                S[tg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), qfrag[m], S[tg],
                                                                0, 0, 0);
            }
        }
        lds_phase_fence();

        // S[tg][j] is token t0 + tg*16 + 4*fg + j against head fn.  Mask the ragged tail.
        if (t0 + WT > t_end) {
#pragma unroll
            for (int tg = 0; tg < NG; ++tg) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (t0 + tg * 16 + 4 * fg + j >= t_end) S[tg][j] = kMaskedScore;
                }
            }
        }

        // ---- online softmax; the maximum is shared by the four k groups of a head column
        float mloc = S[0][0];
#pragma unroll
        for (int tg = 0; tg < NG; ++tg) {
#pragma unroll
            for (int j = 0; j < 4; ++j) mloc = fmaxf(mloc, S[tg][j]);
        }
        mloc = fmaxf(mloc, __shfl_xor(mloc, 16, kWaveSize));
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32, kWaveSize));
        if (__builtin_amdgcn_ballot_w64(mloc > m_run) != 0) {  // wave-uniform: rescale only when some maximum moved
            const float m_new = fmaxf(m_run, mloc);
            const float alpha = fast_exp2((m_run - m_new) * c);
            l_part *= alpha;
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) O[nb] *= alpha;
            m_run = m_new;
        }
        const float mc = m_run * c;
        float psum = 0.f;
#pragma unroll
        for (int tg = 0; tg < NG; ++tg) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float pj = fast_exp2(fmaf(S[tg][j], c, -mc));  // masked scores give exactly 0
                S[tg][j] = pj;
                psum += pj;
            }
        }
        l_part += psum;

        // ---- V tile -> the same slab (all K reads were issued before these writes)
#pragma unroll
        for (int u = 0; u < U; ++u) *reinterpret_cast<uint4*>(wr_v + u * G * VPITCH) = vr[u];
        lds_phase_fence();
        if (tn < t_end) issue_v(tn);

        // ---- O^T += V^T P.  k slot (fg, i) of a 32-token step is token 4*fg + i of its first
        //      16-token group for i < 4 and of its second group for i >= 4, on both operands.
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            uint4 pw;
            pw.x = pack_bf16x2(S[2 * ks][0], S[2 * ks][1]);
            pw.y = pack_bf16x2(S[2 * ks][2], S[2 * ks][3]);
            pw.z = pack_bf16x2(S[2 * ks + 1][0], S[2 * ks + 1][1]);
            pw.w = pack_bf16x2(S[2 * ks + 1][2], S[2 * ks + 1][3]);
            const bf16x8_t pfrag = __builtin_bit_cast(bf16x8_t, pw);
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    L3_LDS_PTR(s16x4_t, rd_v + (2 * ks) * 16 * VPITCH + nb * 32));
                const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    L3_LDS_PTR(s16x4_t, rd_v + (2 * ks + 1) * 16 * VPITCH + nb * 32));
                const s16x8_t vv = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                O[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vv), pfrag, O[nb],
                                                                0, 0, 0);
            }
        }
        lds_phase_fence();
    }

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
            } else {
                const int64_t row = attn_partial_row(p, b, qh, split);
                *reinterpret_cast<float2*>(p.part_o + row * HD + d) = make_float2(o0, o1);
                if (d == 0) p.part_ml[row] = make_float2(M, L);
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

}  // namespace

int attn_mfma_heads_per_wg(int KVH) {
    for (int h = kMfmaWaves; h > 1; h /= 2) {
        if (KVH % h == 0) return h;
    }
    return 1;
}

int launch_attn_splitkv_mfma(const AttnParams& p, int HD, int R, bool coop, hipStream_t stream) {
    if (R < 1 || R > kAttnMaxRatio) return int(hipErrorInvalidValue);
    const dim3 block(kMfmaWaves * kWaveSize);
    if (coop) {
        const dim3 grid(unsigned(p.B) * unsigned(p.KVH) * unsigned(p.num_splits));
        if (HD == 64) {
            hipLaunchKernelGGL((attn_splitkv_mfma_kernel<64, true>), grid, block, 0, stream, p, R, 1);
        } else {
            hipLaunchKernelGGL((attn_splitkv_mfma_kernel<128, true>), grid, block, 0, stream, p, R, 1);
        }
        return int(hipGetLastError());
    }
    const int hpw = attn_mfma_heads_per_wg(p.KVH);
    const int spw = kMfmaWaves / hpw;
    const dim3 grid(unsigned(p.B) * unsigned(p.KVH / hpw) * unsigned((p.num_splits + spw - 1) / spw));
    if (HD == 64) {
        hipLaunchKernelGGL((attn_splitkv_mfma_kernel<64, false>), grid, block, 0, stream, p, R, hpw);
    } else {
        hipLaunchKernelGGL((attn_splitkv_mfma_kernel<128, false>), grid, block, 0, stream, p, R, hpw);
    }
    return int(hipGetLastError());
}

}  // namespace l3
