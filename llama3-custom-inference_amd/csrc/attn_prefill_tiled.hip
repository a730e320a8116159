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
#include <type_traits>

#include "attn_mfma_core.hpp"

namespace l3 {

namespace {

// Maximum that hands a NaN on (v_maximum3_f32): unlike fmaxf it needs no quieting of its inputs, which
// costs an instruction per value that comes out of a matrix instruction or a lane swap.
__device__ __forceinline__ float maximum(float a, float b) { return __builtin_elementwise_maximum(a, b); }
// Maximum over the four k groups of a column (lanes l, l ^ 16, l ^ 32, l ^ 48), as column_max().
__device__ __forceinline__ float column_maximum(float x) {
    const uint32_t xi = __builtin_bit_cast(uint32_t, x);
    const auto h = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
    const float y = maximum(__builtin_bit_cast(float, uint32_t(h[0])), __builtin_bit_cast(float, uint32_t(h[1])));
    const uint32_t yi = __builtin_bit_cast(uint32_t, y);
    const auto r = __builtin_amdgcn_permlane16_swap(yi, yi, false, false);
    return maximum(__builtin_bit_cast(float, uint32_t(r[0])), __builtin_bit_cast(float, uint32_t(r[1])));
}

// Tiled form.  Few registers on purpose (128 at head size 64): WPE wavefronts per SIMD, i.e. several
// independent workgroups per compute unit whose matrix, vector and LDS phases, barriers, start-up and
// drain cover each other.  K/V tiles go from global memory straight into LDS
// (global_load_lds_dwordx4: a wavefront-wide load lands in 1 KiB of consecutive LDS), so rows are
// not padded; instead the 16-byte chunk c of token row r sits at chunk position c ^ key(r), which
// spreads the rows that an operand read touches together over all banks.  The two stages are separate
// arrays, so that the compiler can tell a read of one from the load in flight into the other.
template <int HD, int CB, int NW, int TK, int WPE, bool NOMAX>
__global__ void __launch_bounds__(NW * kWaveSize) __attribute__((amdgpu_waves_per_eu(WPE, WPE)))
attn_prefill_tiled_kernel(const PrefillParams p) {
    constexpr int NG = TK / 16, KS = TK / 32, KC = HD / 32, NB = HD / 16;
    constexpr int CPR = HD / 8;                  // 16-byte chunks per token row
    constexpr int ROWB = HD * 2;                 // bytes per token row
    constexpr int KBYTES = TK * ROWB;            // a K tile; a stage is a K tile followed by a V tile
    constexpr int STAGE = 2 * KBYTES;
    constexpr int LOADS = TK * CPR / kWaveSize;  // wavefront-wide loads per operand tile
    static_assert(LOADS % NW == 0, "a tile must divide evenly over the wavefronts");
    constexpr int IPW = LOADS / NW;
    constexpr bool PF = WPE <= 2 && CB == 2;                // the interleaved tile below (needs the registers of two wavefronts per SIMD)
    __shared__ __align__(1024) unsigned char s_stage0[STAGE];
    __shared__ __align__(1024) unsigned char s_stage1[STAGE];

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
    // The workgroups with the longest token ranges are dispatched first.  A launch that the device holds (almost)
    // all at once gets no balancing from the dispatcher: workgroup r lands on compute unit r % snake, which
    // would collect the longest block of every round.  Every second round of `snake` ranks is therefore taken
    // in reverse, so that a unit's blocks add up to about the same length (2 x 2048 tokens at head size 64:
    // 47.8 -> 45.3 us; launches of many rounds are left alone: -1 % there).
    int rank = int(blockIdx.x);
    if (p.snake > 0) {
        const int k = rank / p.snake, j = rank % p.snake;
        if ((k & 1) && (k + 1) * p.snake <= int(gridDim.x)) rank = k * p.snake + (p.snake - 1 - j);
    }
    const int wg = wgs_per_head - 1 - rank / heads;
    const int bh = rank % heads;
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

    // global -> LDS: load j of a wavefront covers slots inst*64 .. +63 of the tile, slot = row * CPR + position.
    // The loads are buffer loads: the resource describes the tile (a scalar base and the bytes from there to the
    // end of the kv head's data), the lane offset never changes from tile to tile (token strides are below 2^24
    // elements), so a load costs no vector instruction, and rows past the data come back as zeros (they are
    // masked: no query sees a token beyond the KV length).
    const char* kb = reinterpret_cast<const char*>(p.k) + wave_uniform((b * p.k_sb + kvh * p.k_sh) * 2);
    const char* vb = reinterpret_cast<const char*>(p.v) + wave_uniform((b * p.v_sb + kvh * p.v_sh) * 2);
    const int64_t k_pitch = wave_uniform(int(p.k_st)) * int64_t(2);   // bytes from a token to the next
    const int64_t v_pitch = wave_uniform(int(p.v_st)) * int64_t(2);
    const int wave_u = wave_uniform(wave);
    auto swz_key = [](int row) { return HD == 128 ? (row & 15) : ((row >> 1) & 7); };
    uint32_t koff[IPW], voff[IPW];
#pragma unroll
    for (int j = 0; j < IPW; ++j) {
        const int slot = (wave_u * IPW + j) * kWaveSize + lane;
        const int row = slot / CPR;
        const uint32_t chunk16 = uint32_t((slot % CPR) ^ swz_key(row)) * 16u;
        koff[j] = uint32_t(row) * uint32_t(k_pitch) + chunk16;
        voff[j] = uint32_t(row) * uint32_t(v_pitch) + chunk16;
    }
    auto dma = [&](int t0, unsigned char* stage) {
        const int64_t rows_left = p.S - t0;                              // scalar, at least 1
        const int64_t k_bytes = min((rows_left - 1) * k_pitch + ROWB, int64_t(0xffffffffLL));
        const int64_t v_bytes = min((rows_left - 1) * v_pitch + ROWB, int64_t(0xffffffffLL));
        const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<char*>(kb + int64_t(t0) * k_pitch), 0, int(uint32_t(k_bytes)), 0x00020000);
        const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<char*>(vb + int64_t(t0) * v_pitch), 0, int(uint32_t(v_bytes)), 0x00020000);
#pragma unroll
        for (int j = 0; j < IPW; ++j) {
            const int inst = wave_u * IPW + j;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, L3_LDS_PTR(void, stage + inst * 1024), 16, int(koff[j]), 0, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, L3_LDS_PTR(void, stage + KBYTES + inst * 1024), 16, int(voff[j]), 0, 0, 0);
        }
    };
    // operand addresses within a stage.  K: lane (fn, fg) reads chunk 4m + fg of row 16 tg + fn, whose
    // key depends on fn alone.  V (transposing read): lane reads 8 bytes of row 32 ks + 4 fg + (fn >> 2)
    // (+16) in the 32-byte column block nb, i.e. chunk 2 nb + ((lane & 3) >> 1); the key depends on the
    // lane alone as well.  One address per m / nb, the rest is instruction offsets.
    int ak[KC], av[NB];   // byte offsets within a stage
    {
        const int kkey = swz_key(fn);
#pragma unroll
        for (int m = 0; m < KC; ++m) ak[m] = fn * ROWB + (((m * 4 + fg) ^ kkey) << 4);
        const int vrow = 4 * fg + (fn >> 2);
        const int vkey = swz_key(vrow);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            av[nb] = KBYTES + vrow * ROWB + (((nb * 2 + ((lane & 3) >> 1)) ^ vkey) << 4) + (lane & 1) * 8;
        }
    }

    // The softmax denominator rides on the matrix pipe: V^T gets a block of rows that are all ones, so
    // that L = ones . P accumulates the column sums of P (every entry of L[cb] is the whole column's sum,
    // over all four k groups) next to O.  The vector pipe, which bounds this kernel at head size 64, is
    // spared one addition per score; P enters both sums rounded to bf16, so the weights of a column add
    // up to one exactly.
    f32x4_t O[CB][NB], L[CB];
    float Lsum[CB];    // the hand-laid tile keeps the denominator as one number per column (it looks at a tile's sum first)
    float m_run[CB];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        m_run[cb] = kMaskedScore;
        Lsum[cb] = 0.f;
        L[cb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) O[cb][nb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
    const float c = p.scale_log2e;
    // The running maximum only follows the scores when one of them exceeds it by more than 2^8 (in the
    // exponent's units): until then the exponentials are taken against the stale maximum -- they stay
    // below 256, which bf16 and the float32 sums hold as well as values below 1 -- and the accumulators
    // need no rescaling.  O / L is the same quotient either way.
    const float slack = 8.0f / c;
    bf16x8_t ones = __builtin_bit_cast(bf16x8_t, make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u));
    asm volatile("" : "+v"(ones));   // kept in registers: rebuilt from constants it costs two moves per use

    // One tile on its LDS stage: S = K Q^T, the online softmax of S, O^T += V^T P.
    auto tile = [&](const unsigned char* stage, int t0) __attribute__((always_inline)) {
        f32x4_t S[CB][NG];
#pragma unroll
        for (int tg = 0; tg < NG; ++tg) {
#pragma unroll
            for (int m = 0; m < KC; ++m) {
                const uint4 a = *reinterpret_cast<const uint4*>(stage + ak[m] + tg * 16 * ROWB);
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) {
                    const f32x4_t acc = (m == 0) ? f32x4_t{0.f, 0.f, 0.f, 0.f} : S[cb][tg];
                    S[cb][tg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), qfrag[cb][m],
                                                                        acc, 0, 0, 0);
                }
            }
        }

        // causal mask (only tiles that reach past the wavefront's first position) and softmax
        const bool mask_tile = t0 + TK > wave_limit_min;
        bf16x8_t pfrag[CB][KS];
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            if (mask_tile) {
                const int visible = col_limit[cb] - t0 - 4 * fg;   // this lane's scores 16 tg + j below it count
#pragma unroll
                for (int tg = 0; tg < NG; ++tg) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if (tg * 16 + j >= visible) S[cb][tg][j] = kMaskedScore;
                    }
                }
            }
            float mloc = S[cb][0][0];
#pragma unroll
            for (int tg = 0; tg < NG; ++tg) {
#pragma unroll
                for (int j = 0; j < 4; ++j) mloc = maximum(mloc, S[cb][tg][j]);
            }
            mloc = column_maximum(mloc);
            if (__builtin_amdgcn_ballot_w64(mloc > m_run[cb] + slack) != 0) {
                const float m_new = maximum(m_run[cb], mloc);
                const float alpha = fast_exp2((m_run[cb] - m_new) * c);
                L[cb] *= alpha;
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) O[cb][nb] *= alpha;
                m_run[cb] = m_new;
            }
            const float mc = m_run[cb] * c;
#pragma unroll
            for (int tg = 0; tg < NG; ++tg) {
#pragma unroll
                for (int j = 0; j < 4; ++j) S[cb][tg][j] = fast_exp2(fmaf(S[cb][tg][j], c, -mc));   // masked scores give exactly 0
            }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                uint4 pw;
                pw.x = pack_bf16x2(S[cb][2 * ks][0], S[cb][2 * ks][1]);
                pw.y = pack_bf16x2(S[cb][2 * ks][2], S[cb][2 * ks][3]);
                pw.z = pack_bf16x2(S[cb][2 * ks + 1][0], S[cb][2 * ks + 1][1]);
                pw.w = pack_bf16x2(S[cb][2 * ks + 1][2], S[cb][2 * ks + 1][3]);
                pfrag[cb][ks] = __builtin_bit_cast(bf16x8_t, pw);
                L[cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pfrag[cb][ks], L[cb], 0, 0, 0);
            }
        }

        // O^T += V^T P; the k slots of a 32-token step pair (fg, i) with token 4*fg + i of the step's first
        // 16-token group for i < 4 and of its second group for i >= 4
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    L3_LDS_PTR(s16x4_t, stage + av[nb] + (2 * ks) * 16 * ROWB));
                const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    L3_LDS_PTR(s16x4_t, stage + av[nb] + (2 * ks + 1) * 16 * ROWB));
                const s16x8_t vv = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) {
                    O[cb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vv), pfrag[cb][ks],
                                                                        O[cb][nb], 0, 0, 0);
                }
            }
        }
    };
    // Pieces of the hand-laid tile below.  It computes no maximum as long as the reference maximum is good enough:
    // the exponentials are taken against the reference as it stands, and the column sum of the tile's weights,
    // which the matrix pipe forms anyway (against a block of ones), tells whether that was safe -- a sum of at
    // most kTileSumLimit means every weight stayed below it, which bf16 and the float32 sums hold as well as values
    // below 1, and O / L is the same quotient for any reference.  Only when a column's sum exceeds the limit or is
    // not a number (the first tile, whose reference is still the masked score; a score that leaves the reference
    // far behind) the scores of that column block are formed once more, their maximum becomes the reference, the
    // accumulators are rescaled and the weights redone.
    constexpr float kTileSumLimit = 1024.0f;
    auto mask_scores = [&](f32x4_t (&Z)[NG], int visible) __attribute__((always_inline)) {
#pragma unroll
        for (int tg = 0; tg < NG; ++tg) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (tg * 16 + j >= visible) Z[tg][j] = kMaskedScore;   // this lane's scores 16 tg + j beyond `visible` do not count
            }
        }
    };
    auto redo_column_block = [&](const unsigned char* stage, int cb, f32x4_t (&Z)[NG], int visible, bool masked,
                                 bf16x8_t (&pf)[KS]) __attribute__((always_inline)) -> float {
#pragma unroll
        for (int tg = 0; tg < NG; ++tg) {
#pragma unroll
            for (int m = 0; m < KC; ++m) {
                const uint4 a = *reinterpret_cast<const uint4*>(stage + ak[m] + tg * 16 * ROWB);
                const f32x4_t acc = (m == 0) ? f32x4_t{0.f, 0.f, 0.f, 0.f} : Z[tg];
                Z[tg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), qfrag[cb][m], acc, 0, 0, 0);
            }
        }
        if (masked) mask_scores(Z, visible);
        float mloc = Z[0][0];
#pragma unroll
        for (int tg = 0; tg < NG; ++tg) {
#pragma unroll
            for (int j = 0; j < 4; ++j) mloc = maximum(mloc, Z[tg][j]);
        }
        mloc = column_maximum(mloc);
        const float m_new = maximum(m_run[cb], mloc);
        const float alpha = fast_exp2((m_run[cb] - m_new) * c);
        Lsum[cb] *= alpha;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) O[cb][nb] *= alpha;
        m_run[cb] = m_new;
        const float mc = m_new * c;
#pragma unroll
        for (int tg = 0; tg < NG; ++tg) {
#pragma unroll
            for (int j = 0; j < 4; ++j) Z[tg][j] = fast_exp2(fmaf(Z[tg][j], c, -mc));
        }
        f32x4_t sum = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            uint4 pw;
            pw.x = pack_bf16x2(Z[2 * ks][0], Z[2 * ks][1]);
            pw.y = pack_bf16x2(Z[2 * ks][2], Z[2 * ks][3]);
            pw.z = pack_bf16x2(Z[2 * ks + 1][0], Z[2 * ks + 1][1]);
            pw.w = pack_bf16x2(Z[2 * ks + 1][2], Z[2 * ks + 1][3]);
            pf[ks] = __builtin_bit_cast(bf16x8_t, pw);
            sum = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pf[ks], sum, 0, 0, 0);
        }
        return sum[0];
    };

    // The compiler-scheduled tile without a maximum (head size 64, launches of many workgroups): the weights are
    // taken against the reference as it stands, 32 tokens at a time (their scores live in 16 registers), and
    // their column sums, which the matrix pipe forms anyway, are checked before anything reaches the accumulators.
    // A sum out of range or not a number stops the wavefront at that tile: nothing is repaired here, so that the
    // loop carries no second path (with one, at 128 registers, the loop's invariants end up in scratch memory).
    // The tiles from there on are done afterwards by the maximum-first tile above, which takes over m_run, O and
    // the denominator as they stand.  The reference is the maximum of the first tile's scores, per column: a row
    // leaves the range only when a later score exceeds everything among its first 64 by a factor of hundreds.
    __shared__ int s_first_careful;   // the earliest tile at which a wavefront of the workgroup stopped (NOMAX)
    int first_careful_tile = NOMAX ? 0x7fffffff : 0;   // wave-uniform: the tile from which this wavefront takes the maximum first
    auto scores32 = [&](const unsigned char* stage, int t0, int ks, f32x4_t (&Z)[CB][2]) __attribute__((always_inline)) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int m = 0; m < KC; ++m) {
                const uint4 a = *reinterpret_cast<const uint4*>(stage + ak[m] + (2 * ks + h) * 16 * ROWB);
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) {
                    const f32x4_t acc = (m == 0) ? f32x4_t{0.f, 0.f, 0.f, 0.f} : Z[cb][h];
                    Z[cb][h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), qfrag[cb][m],
                                                                       acc, 0, 0, 0);
                }
            }
        }
        if (t0 + TK > wave_limit_min) {
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
                const int visible = col_limit[cb] - t0 - 4 * fg;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if ((2 * ks + h) * 16 + j >= visible) Z[cb][h][j] = kMaskedScore;
                    }
                }
            }
        }
    };
    auto tile_lz = [&](const unsigned char* stage, int t0) __attribute__((always_inline)) {
        bf16x8_t pfrag[CB][KS];
        f32x4_t sum[CB];
        float mc[CB];
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            sum[cb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            mc[cb] = m_run[cb] * c;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            f32x4_t Z[CB][2];
            scores32(stage, t0, ks, Z);
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) Z[cb][h][j] = fast_exp2(fmaf(Z[cb][h][j], c, -mc[cb]));
                }
                uint4 pw;
                pw.x = pack_bf16x2(Z[cb][0][0], Z[cb][0][1]);
                pw.y = pack_bf16x2(Z[cb][0][2], Z[cb][0][3]);
                pw.z = pack_bf16x2(Z[cb][1][0], Z[cb][1][1]);
                pw.w = pack_bf16x2(Z[cb][1][2], Z[cb][1][3]);
                pfrag[cb][ks] = __builtin_bit_cast(bf16x8_t, pw);
                sum[cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pfrag[cb][ks], sum[cb], 0, 0, 0);
            }
        }
        bool out_of_range = false;
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) out_of_range = out_of_range || !(sum[cb][0] <= kTileSumLimit);
        if (__builtin_amdgcn_ballot_w64(out_of_range) != 0) {   // nothing of this tile has reached the accumulators
            first_careful_tile = t0;
            if (lane == 0) atomicMin(&s_first_careful, t0);   // the workgroup looks at this every eighth tile
            return;
        }
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) Lsum[cb] += sum[cb][0];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    L3_LDS_PTR(s16x4_t, stage + av[nb] + (2 * ks) * 16 * ROWB));
                const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    L3_LDS_PTR(s16x4_t, stage + av[nb] + (2 * ks + 1) * 16 * ROWB));
                const s16x8_t vv = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) {
                    O[cb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vv), pfrag[cb][ks],
                                                                        O[cb][nb], 0, 0, 0);
                }
            }
        }
    };
    auto reference_from_first_tile = [&](const unsigned char* stage) __attribute__((always_inline)) {
        float mloc[CB];
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) mloc[cb] = kMaskedScore;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            f32x4_t Z[CB][2];
            scores32(stage, 0, ks, Z);
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) mloc[cb] = maximum(mloc[cb], Z[cb][h][j]);
                }
            }
        }
        // a column that belongs to no query (padding of the 16-column block, positions past the prompt) gets a
        // reference that turns its weights to zero instead of one that every unmasked tile would overflow
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) m_run[cb] = col_limit[cb] > 0 ? column_maximum(mloc[cb]) : 1e30f;
    };

    // The same tile for wavefronts with registers to spare (two per SIMD, head size 128), laid out so that the
    // vector work of one column block issues between the matrix instructions of the other:
    //   K operands (all of the tile, one wait)    S0 = K Q0^T
    //   [S1 = K Q1^T          | exponentials of S0]      V^T operands of the first 32 tokens requested half way
    //   [O0^T += V^T P0       | exponentials of S1]      V^T operands of the last 32 tokens requested first
    //    O1^T += V^T P1
    // A matrix instruction occupies its pipe for 16 cycles and the wavefront may issue independent vector
    // instructions meanwhile; left to itself the compiler keeps the phases apart and puts every LDS read next
    // to the product that needs it, with a full wait.  sched_barrier(0) pins the order written here.
    auto tile_pf = [&](const unsigned char* stage, int t0, auto mask_tag) __attribute__((always_inline)) {
        constexpr bool MASK = decltype(mask_tag)::value;
        static_assert(CB == 2, "two column blocks take turns");
        constexpr int NQ = KC * NG;   // matrix instructions of a column block's scores
        constexpr int NP = KS * NB;   // ... and of its output
        constexpr int NS = NG * 4;    // scores per lane and column block
        static_assert(NS % NQ == 0 && NS % NP == 0, "whole scores per matrix instruction");
        f32x4_t S[CB][NG];
        uint4 ka[NG][KC];
#pragma unroll
        for (int m = 0; m < KC; ++m) {
#pragma unroll
            for (int tg = 0; tg < NG; ++tg) ka[tg][m] = *reinterpret_cast<const uint4*>(stage + ak[m] + tg * 16 * ROWB);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int m = 0; m < KC; ++m) {
#pragma unroll
            for (int tg = 0; tg < NG; ++tg) {
                const f32x4_t acc = (m == 0) ? f32x4_t{0.f, 0.f, 0.f, 0.f} : S[0][tg];
                S[0][tg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ka[tg][m]), qfrag[0][m], acc, 0, 0, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        uint32_t pw[CB][NS / 2];
        auto score = [&](int cb, int i, float mc) __attribute__((always_inline)) {
            const int tg = i / 4, j = i % 4;
            S[cb][tg][j] = fast_exp2(fmaf(S[cb][tg][j], c, -mc));   // masked scores give exactly 0
            if (j & 1) pw[cb][i / 2] = pack_bf16x2(S[cb][tg][j - 1], S[cb][tg][j]);
        };
        bf16x8_t pfrag[CB][KS];
        auto weights = [&](int cb) __attribute__((always_inline)) {
            f32x4_t sum = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                pfrag[cb][ks] = __builtin_bit_cast(bf16x8_t, make_uint4(pw[cb][4 * ks], pw[cb][4 * ks + 1], pw[cb][4 * ks + 2], pw[cb][4 * ks + 3]));
                sum = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pfrag[cb][ks], sum, 0, 0, 0);
            }
            float tile_sum = sum[0];   // every entry of the block is its column's sum
            if (__builtin_amdgcn_ballot_w64(!(tile_sum <= kTileSumLimit)) != 0) {
                tile_sum = redo_column_block(stage, cb, S[cb], col_limit[cb] - t0 - 4 * fg, MASK, pfrag[cb]);
            }
            Lsum[cb] += tile_sum;
        };
        s16x8_t vt[KS][NB];
        auto v_operands = [&](int ks) __attribute__((always_inline)) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(L3_LDS_PTR(s16x4_t, stage + av[nb] + (2 * ks) * 16 * ROWB));
                const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(L3_LDS_PTR(s16x4_t, stage + av[nb] + (2 * ks + 1) * 16 * ROWB));
                vt[ks][nb] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
        };

        if constexpr (MASK) mask_scores(S[0], col_limit[0] - t0 - 4 * fg);
        const float mc0 = m_run[0] * c;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const int m = q / NG, tg = q % NG;
            const f32x4_t acc = (m == 0) ? f32x4_t{0.f, 0.f, 0.f, 0.f} : S[1][tg];
            S[1][tg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ka[tg][m]), qfrag[1][m], acc, 0, 0, 0);
#pragma unroll
            for (int i = q * (NS / NQ); i < (q + 1) * (NS / NQ); ++i) score(0, i, mc0);
            __builtin_amdgcn_sched_barrier(0);
            if (q == NQ / 2 - 1) {   // half of the K operands are spent: their registers take the first V^T operands
                v_operands(0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if constexpr (MASK) mask_scores(S[1], col_limit[1] - t0 - 4 * fg);
        const float mc1 = m_run[1] * c;
        weights(0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) asm volatile("" : "+v"(vt[0][nb]));   // the wait for these precedes the next requests
        v_operands(1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int q = 0; q < NP; ++q) {
            const int ks = q / NB, nb = q % NB;
            O[0][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vt[ks][nb]), pfrag[0][ks], O[0][nb], 0, 0, 0);
#pragma unroll
            for (int i = q * (NS / NP); i < (q + 1) * (NS / NP); ++i) score(1, i, mc1);
            __builtin_amdgcn_sched_barrier(0);
        }
        weights(1);
#pragma unroll
        for (int q = 0; q < NP; ++q) {
            const int ks = q / NB, nb = q % NB;
            O[1][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vt[ks][nb]), pfrag[1][ks], O[1][nb], 0, 0, 0);
        }
    };
    // One barrier per tile: the loads of tile i + 1 are issued before the arithmetic on tile i and land in
    // the other stage, which was last read before the previous barrier.
    auto step = [&](auto parity_tag, auto careful_tag, int t0) __attribute__((always_inline)) {
        constexpr int PAR = decltype(parity_tag)::value;
        if (t0 + TK < wg_t_end) dma(t0 + TK, PAR ? s_stage0 : s_stage1);   // workgroup-uniform
        if (t0 < wave_t_end) {                                              // wave-uniform
            const unsigned char* stage = PAR ? s_stage1 : s_stage0;
            if constexpr (PF) {
                // only tiles that reach past the wavefront's first position need the causal mask
                if (t0 + TK > wave_limit_min) tile_pf(stage, t0, std::true_type{});
                else tile_pf(stage, t0, std::false_type{});
            } else if constexpr (decltype(careful_tag)::value) {
                if (t0 >= first_careful_tile) tile(stage, t0);
            } else {
                if (t0 < first_careful_tile) tile_lz(stage, t0);
            }
        }
        __builtin_amdgcn_s_waitcnt(0xF70);   // vmcnt(0): this wavefront's part of the next stage has landed
        __syncthreads();
    };
    // tiles from t_begin (a multiple of TK) on; the stage of a tile is its index's parity
    auto tiles_from = [&](auto careful_tag, int t_begin) __attribute__((always_inline)) -> int {
        const bool odd = ((t_begin / TK) & 1) != 0;
        dma(t_begin, odd ? s_stage1 : s_stage0);
        __builtin_amdgcn_s_waitcnt(0xF70);
        __syncthreads();
        if constexpr (!PF && !decltype(careful_tag)::value) {
            if (wave_t_end > 0) reference_from_first_tile(s_stage0);
        }
        int t0 = t_begin;
        if (odd) {
            step(std::integral_constant<int, 1>{}, careful_tag, t0);
            t0 += TK;
        }
        for (; t0 < wg_t_end; t0 += 2 * TK) {
            step(std::integral_constant<int, 0>{}, careful_tag, t0);
            if (t0 + TK < wg_t_end) step(std::integral_constant<int, 1>{}, careful_tag, t0 + TK);
            if constexpr (NOMAX && !decltype(careful_tag)::value) {
                // Every eighth tile: once a wavefront has stopped, the workgroup leaves this loop, so that the tiles
                // it would only load and not use are few.  Read between two barriers: wavefronts write the word
                // only inside a tile, so all of them see the same value here.
                if (((t0 / (2 * TK)) & 3) == 3) {
                    __syncthreads();
                    const int stopped_at = wave_uniform(s_first_careful);
                    __syncthreads();
                    if (stopped_at != 0x7fffffff) {
                        t0 += 2 * TK;
                        break;
                    }
                }
            }
        }
        return t0;   // the first tile this loop has not been offered
    };
    if constexpr (PF) {
        tiles_from(std::false_type{}, 0);
    } else if constexpr (!NOMAX) {
        tiles_from(std::true_type{}, 0);
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) Lsum[cb] = L[cb][0];
    } else {
        // First the tiles without a maximum; a wavefront whose column sums leave the range stops there with its
        // accumulators untouched by that tile, and the workgroup ends that loop within eight tiles.  Then, from the
        // earliest such tile of the workgroup on (the loads are the workgroup's), the tiles with the maximum taken
        // first, each wavefront joining at its own tile.
        if (tid == 0) s_first_careful = 0x7fffffff;
        const int offered = tiles_from(std::false_type{}, 0);
        first_careful_tile = min(first_careful_tile, offered);   // a wavefront that had not stopped goes on from where the loop ended
        if (lane == 0 && first_careful_tile < wave_t_end) atomicMin(&s_first_careful, first_careful_tile);
        __syncthreads();
        const int t_begin = wave_uniform(s_first_careful);
        if (t_begin < wg_t_end) {
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) L[cb] = f32x4_t{Lsum[cb], Lsum[cb], Lsum[cb], Lsum[cb]};
            tiles_from(std::true_type{}, t_begin);
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) Lsum[cb] = L[cb][0];
        }
    }

#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        if (col_limit[cb] > 0) {
            const int qi = wave_first_qi + cb * ppw + fn / R;
            const int qh = kvh * R + fn % R;
            const float inv = 1.0f / Lsum[cb];
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

template <class Kernel>
int launch_blocks(Kernel kernel, const PrefillParams& p, int waves, int col_blocks, hipStream_t stream) {
    const int R = p.QH / p.KVH;
    const int wg_pos = waves * col_blocks * (16 / R);
    const int wgs_per_head = (p.T + wg_pos - 1) / wg_pos;
    const dim3 grid(unsigned(p.B) * unsigned(p.KVH) * unsigned(wgs_per_head));
    PrefillParams q = p;
    const int cus = current_device_cus();
    q.snake = (int64_t(grid.x) <= 4 * int64_t(cus)) ? cus : 0;
    hipLaunchKernelGGL(kernel, grid, dim3(waves * kWaveSize), 0, stream, q);
    return int(hipGetLastError());
}

}  // namespace

int launch_attn_prefill_tiled(const PrefillParams& p, int HD, hipStream_t stream) {
    constexpr int CB = kPrefillColBlocks, NW = kPrefillTiledWaves;
    // tiles of 64 tokens; four wavefronts per SIMD at head size 64 (four workgroups per compute unit), two
    // at 128 (two workgroups: a stage pair is 64 KiB)
    const int R = p.QH / p.KVH;
    const int wg_pos = NW * CB * (16 / R);
    const int64_t wgs = int64_t(p.B) * p.KVH * ((p.T + wg_pos - 1) / wg_pos);
    const int64_t cus = current_device_cus();
    // A launch that leaves much of the device empty runs with one column block per wavefront instead of two: twice
    // the workgroups, each K/V operand read feeding one matrix instruction.  Graph-timed at head size 128 against
    // the two-block kernel: 512 tokens -22 %, 1024 -14 %, 1536 -12 %, 1792 -2.5 %, 1920 +2 %; at head size 64:
    // 1024 tokens -23 %, 2048 -17 %, 2560 -10 %, 2816 -3.5 %, 3072 +2 %, 5 x 512 +2.5 %.  Only the library's own
    // choice does this: a forced TILED form is the two-block kernel whatever the size.
    if (HD == 64) {
        // The tiles that take no maximum gain where the device is refilled as workgroups finish and the rows are
        // long (8192 tokens: -4.5 %, 6144: -4.2 %, 2 x 4096: -3 %); a launch that the device holds at once gains
        // nothing, and short rows lose to the extra pass over the first tile (4 x 2048: 0, 32 x 256: +8 %,
        // 64 x 128: +18 %).
        if (p.no_max_tiles || (p.auto_form && wgs > 4 * cus && p.S >= 4096)) {
            return launch_blocks(attn_prefill_tiled_kernel<64, CB, NW, 64, 4, true>, p, NW, CB, stream);
        }
        if (p.auto_form && 4 * wgs <= 9 * cus) {
            return launch_blocks(attn_prefill_tiled_kernel<64, 1, NW, 64, 4, false>, p, NW, 1, stream);
        }
        return launch_blocks(attn_prefill_tiled_kernel<64, CB, NW, 64, 4, false>, p, NW, CB, stream);
    }
    // ... on 32-token tiles with four workgroups per compute unit where three or more sequences share the launch
    // (finer tiles waste less of a short row's diagonal; graph-timed against 64-token tiles: 3 x 512 tokens -12 %,
    // 8 x 256 -9 %, 4 x 512 and 16 x 128 -4 %, 2 x 1024 -2 %, 2 x 256 +2 %; one prompt alone: 512 tokens +5 %,
    // 2048 +2.5 %).
    if (p.auto_form && wgs <= 2 * cus && p.B >= 3) {
        return launch_blocks(attn_prefill_tiled_kernel<128, 1, NW, 32, 4, false>, p, NW, 1, stream);
    }
    if (p.auto_form && 4 * wgs <= 7 * cus) {
        return launch_blocks(attn_prefill_tiled_kernel<128, 1, NW, 64, 2, false>, p, NW, 1, stream);
    }
    // Long prompts in launches of more workgroups than the device holds at once: the loop that takes no maximum, left
    // to the compiler's schedule, on 32-token tiles (three workgroups per compute unit at 165 registers) is a little
    // ahead of the hand-laid tile (same run: 8192 tokens -1 %, 2 x 8192 -4 %, 4096 -1.3 %; 2 x 2048 -1 %, 2048 +15 %).
    if (p.no_max_tiles || (p.auto_form && wgs > 2 * cus && p.S >= 4096)) {
        return launch_blocks(attn_prefill_tiled_kernel<128, CB, NW, 32, 3, true>, p, NW, CB, stream);
    }
    return launch_blocks(attn_prefill_tiled_kernel<128, CB, NW, 64, 2, false>, p, NW, CB, stream);
}

}  // namespace l3
