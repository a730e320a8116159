// Causal GQA prefill attention, workgroup-tiled form, for long prompts on the gfx950 matrix cores.
//
// Takes the place of the scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
// call of model.py:114-116.  Where the wavefront-private form (attn_prefill.hip) lets every
// wavefront stream the kv head's tokens on its own, here the NW wavefronts of a workgroup share
// each K/V tile: the tile is fetched from global memory once per workgroup, double-buffered in
// LDS, and every wavefront multiplies it against its own CB x 16 columns.  A column is a (query
// position, query head) pair as in the other form: 16 / R consecutive positions of the R query
// heads that share the kv head, so the whole GQA group rides on one pass over K and V.
//
//   S[16 tokens x 16 columns]  = K[16 x 32 dims]          . Q^T[32 dims x 16 columns]
//   O^T[16 dims x 16 columns] += V^T[16 dims x 32 tokens] . P[32 tokens x 16 columns]
//
// One K (or V^T) operand read from LDS feeds CB matrix instructions, which is what keeps the LDS
// pipe from bounding the kernel.  One workgroup barrier per tile: the global loads of tile i+1 are
// issued before the arithmetic on tile i and land in the other LDS buffer after it.
//
// Query i of T sits at absolute position S - T + i and attends to tokens 0 .. S - T + i.
#include "attn_mfma_core.hpp"

namespace l3 {

namespace {

template <int HD, int CB, int NW>
struct PrefillTile {
    static constexpr int NT = NW * kWaveSize;      // threads
    static constexpr int TK = 64;                  // tokens per K/V tile
    static constexpr int LPR = HD / 8;             // 16-byte chunks per token row
    static constexpr int CHUNKS = TK * LPR;        // chunks per K (or V) tile
    static constexpr int U = CHUNKS / NT;          // chunks per thread per operand
    static constexpr int NG = TK / 16;
    static constexpr int KC = HD / 32;
    static constexpr int NB = HD / 16;
    static constexpr int KS = TK / 32;
    static constexpr int KPITCH = HD * 2 + 16;
    static constexpr int VPITCH = HD * 2 + 32;
    static constexpr int KBYTES = TK * KPITCH;
    static constexpr int VBYTES = TK * VPITCH;
    static constexpr int STAGE = KBYTES + VBYTES;  // one buffer: a K tile followed by a V tile
    static_assert(CHUNKS % NT == 0, "tile must divide evenly over the workgroup");
};

template <int HD, int CB, int NW>
__global__ void __launch_bounds__(NW * kWaveSize)
attn_prefill_tiled_kernel(const PrefillParams p) {
    using T = PrefillTile<HD, CB, NW>;
    constexpr int NT = T::NT, TK = T::TK, LPR = T::LPR, U = T::U, NG = T::NG, KC = T::KC, NB = T::NB, KS = T::KS;
    constexpr int KPITCH = T::KPITCH, VPITCH = T::VPITCH, KBYTES = T::KBYTES, STAGE = T::STAGE;
    __shared__ __align__(16) unsigned char s_tiles[2 * STAGE];

    const int tid = threadIdx.x;
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid / kWaveSize;
    const int fn = lane & 15;
    const int fg = lane >> 4;

    const int R = p.QH / p.KVH;
    const int ppw = 16 / R;                              // query positions per 16-column block
    const int wg_pos = NW * CB * ppw;                    // query positions per workgroup
    const int wgs_per_head = (p.T + wg_pos - 1) / wg_pos;
    const int heads = p.B * p.KVH;
    // the workgroups with the longest token ranges are dispatched first
    const int wg = wgs_per_head - 1 - int(blockIdx.x) / heads;
    const int bh = int(blockIdx.x) % heads;
    const int kvh = bh % p.KVH;
    const int b = bh / p.KVH;

    const int wg_first_qi = wg * wg_pos;
    const int wg_last_qi = min(p.T, wg_first_qi + wg_pos) - 1;
    const int wg_t_end = p.S - p.T + wg_last_qi + 1;     // tokens any column of the workgroup may see
    const int wave_first_qi = wg_first_qi + wave * CB * ppw;
    const int wave_last_qi = min(p.T, wave_first_qi + CB * ppw) - 1;
    // tiles at or beyond this are skipped (all of them for a wavefront past the last query)
    const int wave_t_end = wave_first_qi < p.T ? p.S - p.T + wave_last_qi + 1 : 0;
    const int wave_limit_min = p.S - p.T + wave_first_qi + 1;          // tiles below this need no masking

    int col_limit[CB];
    bf16x8_t qfrag[CB][KC];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        const int qi = wave_first_qi + cb * ppw + fn / R;
        const int qh = kvh * R + fn % R;
        const bool valid = (fn < ppw * R) && (qi < p.T);
        col_limit[cb] = valid ? (p.S - p.T + qi + 1) : 0;
#pragma unroll
        for (int m = 0; m < KC; ++m) {
            uint4 qv = make_uint4(0u, 0u, 0u, 0u);
            if (valid) qv = load16(p.q + b * p.q_sb + int64_t(qh) * p.q_sh + int64_t(qi) * p.q_st + (m * 4 + fg) * 8);
            qfrag[cb][m] = __builtin_bit_cast(bf16x8_t, qv);
        }
    }

    // global -> LDS staging: chunk (tid + u*NT) of a tile is 16 bytes of token row chunk / LPR
    const uint16_t* kbase = p.k + b * p.k_sb + kvh * p.k_sh + (tid % LPR) * 8;
    const uint16_t* vbase = p.v + b * p.v_sb + kvh * p.v_sh + (tid % LPR) * 8;
    const int ld_row = tid / LPR;
    constexpr int ROWS_PER_LOAD = NT / LPR;
    uint4 kr[U], vr[U];
    auto issue = [&](int t0) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int tok = min(t0 + u * ROWS_PER_LOAD + ld_row, p.S - 1);  // rows past the data are masked
            kr[u] = load16(kbase + int64_t(tok) * p.k_st);
            vr[u] = load16(vbase + int64_t(tok) * p.v_st);
        }
    };
    auto stash = [&](unsigned char* stage) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int row = u * ROWS_PER_LOAD + ld_row;
            *reinterpret_cast<uint4*>(stage + row * KPITCH + (tid % LPR) * 16) = kr[u];
            *reinterpret_cast<uint4*>(stage + KBYTES + row * VPITCH + (tid % LPR) * 16) = vr[u];
        }
    };

    f32x4_t O[CB][NB];
    float m_run[CB], l_part[CB];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        m_run[cb] = kMaskedScore;
        l_part[cb] = 0.f;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) O[cb][nb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
    const float c = p.scale_log2e;

    issue(0);
    stash(s_tiles);
    __syncthreads();

    int buf = 0;
    for (int t0 = 0; t0 < wg_t_end; t0 += TK) {
        const int tn = t0 + TK;
        const bool more = tn < wg_t_end;   // workgroup-uniform
        if (more) issue(tn);

        if (t0 < wave_t_end) {             // wave-uniform: some column of this wavefront sees the tile
            const unsigned char* stage = s_tiles + buf * STAGE;
            const unsigned char* rd_k = stage + fn * KPITCH + fg * 16;
            const unsigned char* rd_v = stage + KBYTES + (4 * fg + (fn >> 2)) * VPITCH + (lane & 3) * 8;

            // ---- S = K Q^T for the CB column blocks
            f32x4_t S[CB][NG];
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
                for (int tg = 0; tg < NG; ++tg) S[cb][tg] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int tg = 0; tg < NG; ++tg) {
#pragma unroll
                for (int m = 0; m < KC; ++m) {
                    const uint4 a = *reinterpret_cast<const uint4*>(rd_k + tg * 16 * KPITCH + m * 64);
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) {
                        S[cb][tg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                                            qfrag[cb][m], S[cb][tg], 0, 0, 0);
                    }
                }
            }

            // ---- causal mask (only tiles that reach past the wavefront's first position) and softmax
            const bool mask_tile = tn > wave_limit_min;
            bf16x8_t pfrag[CB][KS];
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
                if (mask_tile) {
#pragma unroll
                    for (int tg = 0; tg < NG; ++tg) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            if (t0 + tg * 16 + 4 * fg + j >= col_limit[cb]) S[cb][tg][j] = kMaskedScore;
                        }
                    }
                }
                float mloc = S[cb][0][0];
#pragma unroll
                for (int tg = 0; tg < NG; ++tg) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) mloc = fmaxf(mloc, S[cb][tg][j]);
                }
                mloc = fmaxf(mloc, __shfl_xor(mloc, 16, kWaveSize));
                mloc = fmaxf(mloc, __shfl_xor(mloc, 32, kWaveSize));
                if (__builtin_amdgcn_ballot_w64(mloc > m_run[cb]) != 0) {
                    const float m_new = fmaxf(m_run[cb], mloc);
                    const float alpha = fast_exp2((m_run[cb] - m_new) * c);
                    l_part[cb] *= alpha;
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) O[cb][nb] *= alpha;
                    m_run[cb] = m_new;
                }
                const float mc = m_run[cb] * c;
                float psum = 0.f;
#pragma unroll
                for (int tg = 0; tg < NG; ++tg) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float pj = fast_exp2(fmaf(S[cb][tg][j], c, -mc));
                        S[cb][tg][j] = pj;
                        psum += pj;
                    }
                }
                l_part[cb] += psum;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    uint4 pw;
                    pw.x = pack_bf16x2(S[cb][2 * ks][0], S[cb][2 * ks][1]);
                    pw.y = pack_bf16x2(S[cb][2 * ks][2], S[cb][2 * ks][3]);
                    pw.z = pack_bf16x2(S[cb][2 * ks + 1][0], S[cb][2 * ks + 1][1]);
                    pw.w = pack_bf16x2(S[cb][2 * ks + 1][2], S[cb][2 * ks + 1][3]);
                    pfrag[cb][ks] = __builtin_bit_cast(bf16x8_t, pw);
                }
            }

            // ---- O^T += V^T P; the k slots of a 32-token step pair (fg, i) with token 4*fg + i of the
            //      step's first 16-token group for i < 4 and of its second group for i >= 4
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                    const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        L3_LDS_PTR(s16x4_t, rd_v + (2 * ks) * 16 * VPITCH + nb * 32));
                    const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        L3_LDS_PTR(s16x4_t, rd_v + (2 * ks + 1) * 16 * VPITCH + nb * 32));
                    const s16x8_t vv = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) {
                        O[cb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vv),
                                                                            pfrag[cb][ks], O[cb][nb], 0, 0, 0);
                    }
                }
            }
        }

        // the other buffer was last read before the previous barrier: refill it, then meet
        if (more) stash(s_tiles + (buf ^ 1) * STAGE);
        __syncthreads();
        buf ^= 1;
    }

#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        float l = l_part[cb];
        l += __shfl_xor(l, 16, kWaveSize);
        l += __shfl_xor(l, 32, kWaveSize);
        if (col_limit[cb] > 0) {
            const int qi = wave_first_qi + cb * ppw + fn / R;
            const int qh = kvh * R + fn % R;
            const float inv = 1.0f / l;
            uint16_t* orow = p.out + b * p.o_sb + int64_t(qh) * p.o_sh + int64_t(qi) * p.o_st + fg * 4;
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                uint2 w;
                w.x = pack_bf16x2(O[cb][nb][0] * inv, O[cb][nb][1] * inv);
                w.y = pack_bf16x2(O[cb][nb][2] * inv, O[cb][nb][3] * inv);
                *reinterpret_cast<uint2*>(orow + nb * 16) = w;
            }
        }
    }
}

template <int HD, int CB, int NW>
int launch_tiled(const PrefillParams& p, hipStream_t stream) {
    const int R = p.QH / p.KVH;
    const int wg_pos = NW * CB * (16 / R);
    const int wgs_per_head = (p.T + wg_pos - 1) / wg_pos;
    const dim3 grid(unsigned(p.B) * unsigned(p.KVH) * unsigned(wgs_per_head));
    hipLaunchKernelGGL((attn_prefill_tiled_kernel<HD, CB, NW>), grid, dim3(NW * kWaveSize), 0, stream, p);
    return int(hipGetLastError());
}

}  // namespace

int prefill_tiled_positions_per_wg(int R) { return kPrefillTiledWaves * kPrefillTiledColBlocks * (16 / R); }

int launch_attn_prefill_tiled(const PrefillParams& p, int HD, hipStream_t stream) {
    if (HD == 64) return launch_tiled<64, kPrefillTiledColBlocks, kPrefillTiledWaves>(p, stream);
    return launch_tiled<128, kPrefillTiledColBlocks, kPrefillTiledWaves>(p, stream);
}

}  // namespace l3
