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
#include <utility>

#include "attn_mfma_core.hpp"

namespace l3 {

namespace {

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop that is unrolled by
// construction, with indices that are constant expressions inside the body.
template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

// Tiled form.  Few registers on purpose (128 at head size 64): WPE wavefronts per SIMD, i.e. several
// independent workgroups per compute unit whose matrix, vector and LDS phases, barriers, start-up and
// drain cover each other.  K/V tiles go from global memory straight into LDS
// (global_load_lds_dwordx4: a wavefront-wide load lands in 1 KiB of consecutive LDS), so rows are
// not padded; instead the 16-byte chunk c of token row r sits at chunk position c ^ key(r), which
// spreads the rows that an operand read touches together over all banks.  The two stages are separate
// arrays, so that the compiler can tell a read of one from the load in flight into the other.
template <int HD, int CB, int NW, int TK, int WPE>
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

    // global -> LDS: load j of a wavefront covers slots inst*64 .. +63 of the tile, slot = row * CPR + position.
    // An address is a scalar tile base plus a 32-bit lane offset that does not change from tile to tile
    // (token strides are below 2^24 elements); rows past the data are clamped to the last row and masked.
    const char* kb = reinterpret_cast<const char*>(p.k) + wave_uniform((b * p.k_sb + kvh * p.k_sh) * 2);
    const char* vb = reinterpret_cast<const char*>(p.v) + wave_uniform((b * p.v_sb + kvh * p.v_sh) * 2);
    const int64_t k_pitch = wave_uniform(int(p.k_st)) * int64_t(2);   // bytes from a token to the next
    const int64_t v_pitch = wave_uniform(int(p.v_st)) * int64_t(2);
    const int wave_u = wave_uniform(wave);
    auto swz_key = [](int row) { return HD == 128 ? (row & 15) : ((row >> 1) & 7); };
    uint32_t krow[IPW], vrow[IPW], chunk16[IPW];
#pragma unroll
    for (int j = 0; j < IPW; ++j) {
        const int slot = (wave_u * IPW + j) * kWaveSize + lane;
        const int row = slot / CPR;
        krow[j] = uint32_t(row) * uint32_t(k_pitch);
        vrow[j] = uint32_t(row) * uint32_t(v_pitch);
        chunk16[j] = uint32_t((slot % CPR) ^ swz_key(row)) * 16u;
    }
    auto dma = [&](int t0, unsigned char* stage) {
        const int last_row = min(p.S - 1 - t0, TK - 1);                  // scalar
        const char* kt = kb + int64_t(t0) * k_pitch;
        const char* vt = vb + int64_t(t0) * v_pitch;
        const uint32_t k_last = uint32_t(last_row) * uint32_t(k_pitch);
        const uint32_t v_last = uint32_t(last_row) * uint32_t(v_pitch);
#pragma unroll
        for (int j = 0; j < IPW; ++j) {
            const int inst = wave_u * IPW + j;
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(kt + (min(krow[j], k_last) + chunk16[j])),
                L3_LDS_PTR(void, stage + inst * 1024), 16, 0, 0);
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(vt + (min(vrow[j], v_last) + chunk16[j])),
                L3_LDS_PTR(void, stage + KBYTES + inst * 1024), 16, 0, 0);
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
    float m_run[CB];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        m_run[cb] = kMaskedScore;
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
    const bf16x8_t ones = __builtin_bit_cast(bf16x8_t, make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u));

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
            mloc = column_max(mloc);
            if (__builtin_amdgcn_ballot_w64(mloc > m_run[cb] + slack) != 0) {
                const float m_new = fmaxf(m_run[cb], mloc);
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
    // One barrier per tile: the loads of tile i + 1 are issued before the arithmetic on tile i and land in
    // the other stage, which was last read before the previous barrier.
    auto step = [&](auto parity_tag, int t0) __attribute__((always_inline)) {
        constexpr int PAR = decltype(parity_tag)::value;
        if (t0 + TK < wg_t_end) dma(t0 + TK, PAR ? s_stage0 : s_stage1);   // workgroup-uniform
        if (t0 < wave_t_end) tile(PAR ? s_stage1 : s_stage0, t0);          // wave-uniform
        __builtin_amdgcn_s_waitcnt(0xF70);   // vmcnt(0): this wavefront's part of the next stage has landed
        __syncthreads();
    };

    dma(0, s_stage0);
    __builtin_amdgcn_s_waitcnt(0xF70);
    __syncthreads();
    for (int t0 = 0; t0 < wg_t_end; t0 += 2 * TK) {
        step(std::integral_constant<int, 0>{}, t0);
        if (t0 + TK < wg_t_end) step(std::integral_constant<int, 1>{}, t0 + TK);
    }

#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        if (col_limit[cb] > 0) {
            const int qi = wave_first_qi + cb * ppw + fn / R;
            const int qh = kvh * R + fn % R;
            const float inv = 1.0f / L[cb][0];
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

// Software-pipelined form of the kernel above.  The three phases of a tile -- S = K Q^T, the
// softmax of S, O^T += V^T P -- depend on each other, so a wavefront that runs them in turn
// leaves the matrix pipe idle during the softmax and the vector pipe idle during the products
// (and the wavefronts of a workgroup, held in step by the per-tile barrier, do so together).
// Here iteration `it` multiplies K of tile it, takes the softmax of tile it - 1 and adds tile
// it - 2 to the output: three independent pieces of work in one basic block, placed by hand in
// the steady state.  An LDS stage therefore holds K of one tile and V of the tile two before it;
// the next stage is fetched while the current one is used, by loads that write LDS directly
// (no registers, no copy).  The rescale that a softmax finds is applied to the output accumulators at the
// start of the NEXT iteration (after the P of tile it - 2, which still refers to the previous
// maximum, has been added); the two sets of score / probability registers swap roles every
// iteration, hence the loop unrolled by two.
template <int HD, int CB, int NW>
__global__ void __launch_bounds__(NW * kWaveSize) __attribute__((amdgpu_waves_per_eu(2, 2)))
attn_prefill_pipe_kernel(const PrefillParams p) {
    constexpr int TK = 64;                      // tokens per K/V tile
    constexpr int NG = TK / 16, KC = HD / 32, NB = HD / 16, KS = TK / 32;
    // K/V tiles reach LDS as in the tiled kernel: direct loads, swizzled rows.
    constexpr int CPR = HD / 8;                 // 16-byte chunks per token row
    constexpr int ROWB = HD * 2;                // bytes per token row
    constexpr int KBYTES = TK * ROWB;           // a K tile; a stage is a K tile followed by a V tile
    constexpr int STAGE = 2 * KBYTES;
    constexpr int IPW = CPR / NW;               // wavefront-wide loads per wavefront and tile
    static_assert(CPR % NW == 0, "a tile must divide evenly over the wavefronts");
    // (with a single array the compiler waits for the load in flight before every LDS read)
    __shared__ __align__(1024) unsigned char s_stage0[STAGE];
    __shared__ __align__(1024) unsigned char s_stage1[STAGE];

    const int tid = threadIdx.x;
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid / kWaveSize;
    const int fn = lane & 15;
    const int fg = lane >> 4;

    const int R = p.QH / p.KVH;
    const int ppw = 16 / R;
    const int wg_pos = NW * CB * ppw;
    const int wgs_per_head = (p.T + wg_pos - 1) / wg_pos;
    const int heads = p.B * p.KVH;
    const int wg = wgs_per_head - 1 - int(blockIdx.x) / heads;   // longest token ranges first
    const int bh = int(blockIdx.x) % heads;
    const int kvh = bh % p.KVH;
    const int b = bh / p.KVH;

    const int wg_first_qi = wg * wg_pos;
    const int wg_last_qi = min(p.T, wg_first_qi + wg_pos) - 1;
    const int wg_t_end = p.S - p.T + wg_last_qi + 1;
    const int wave_first_qi = wg_first_qi + wave * CB * ppw;
    const int wave_last_qi = min(p.T, wave_first_qi + CB * ppw) - 1;
    const int wave_t_end = wave_first_qi < p.T ? p.S - p.T + wave_last_qi + 1 : 0;
    const int wave_limit_min = p.S - p.T + wave_first_qi + 1;    // tokens below this are seen by every column
    const int wg_tiles = (wg_t_end + TK - 1) / TK;
    const int wt = (wave_t_end + TK - 1) / TK;                   // tiles this wavefront works on
    const int n_it = wg_tiles + 2;                               // workgroup-uniform trip count

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

    // global -> LDS, addressed as in the tiled kernel (scalar tile base + loop-invariant lane offset)
    const char* kb = reinterpret_cast<const char*>(p.k) + wave_uniform((b * p.k_sb + kvh * p.k_sh) * 2);
    const char* vb = reinterpret_cast<const char*>(p.v) + wave_uniform((b * p.v_sb + kvh * p.v_sh) * 2);
    const int64_t k_pitch = wave_uniform(int(p.k_st)) * int64_t(2);
    const int64_t v_pitch = wave_uniform(int(p.v_st)) * int64_t(2);
    const int wave_u = wave_uniform(wave);
    auto swz_key = [](int row) { return HD == 128 ? (row & 15) : ((row >> 1) & 7); };
    uint32_t krow[IPW], vrow[IPW], chunk16[IPW];
#pragma unroll
    for (int j = 0; j < IPW; ++j) {
        const int slot = (wave_u * IPW + j) * kWaveSize + lane;
        const int row = slot / CPR;
        krow[j] = uint32_t(row) * uint32_t(k_pitch);
        vrow[j] = uint32_t(row) * uint32_t(v_pitch);
        chunk16[j] = uint32_t((slot % CPR) ^ swz_key(row)) * 16u;
    }
    // the stage of iteration `it`: K of tile it, V of tile it - 2 (tiles outside the data are replaced by
    // valid rows that are never used)
    auto dma = [&](int it, unsigned char* stage) {
        const int tk = min(it * TK, p.S - 1), tv = min(max(it - 2, 0) * TK, p.S - 1);   // scalar
        const char* kt = kb + int64_t(tk) * k_pitch;
        const char* vt = vb + int64_t(tv) * v_pitch;
        const uint32_t k_last = uint32_t(min(p.S - 1 - tk, TK - 1)) * uint32_t(k_pitch);
        const uint32_t v_last = uint32_t(min(p.S - 1 - tv, TK - 1)) * uint32_t(v_pitch);
#pragma unroll
        for (int j = 0; j < IPW; ++j) {
            const int inst = wave_u * IPW + j;
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(kt + (min(krow[j], k_last) + chunk16[j])),
                L3_LDS_PTR(void, stage + inst * 1024), 16, 0, 0);
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(vt + (min(vrow[j], v_last) + chunk16[j])),
                L3_LDS_PTR(void, stage + KBYTES + inst * 1024), 16, 0, 0);
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
    float alpha[CB];   // rescale found by an iteration's softmax; the accumulators meet it at the start of the next
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) alpha[cb] = 1.f;

    static_assert(NG == 4, "the maximum tree below is written for 16 scores per column block and lane");
    constexpr int GQ = NG * KC;         // LDS operands of the first product (each feeds CB matrix instructions)
    constexpr int GP = KS * NB;         // LDS operands of the second product
    constexpr int NM = CB * (GQ + GP);  // matrix instructions per tile
    constexpr int NE = CB * NG * 4;     // scores per lane and tile
    constexpr int MS = 11;              // steps of the maximum phase

    // One iteration on its LDS stage.  STEADY: all three phases are live and the softmax tile needs no
    // causal mask.
    auto body = [&](auto steady_tag, auto parity_tag, int it, f32x4_t (&Sprod)[CB][NG], f32x4_t (&Scons)[CB][NG],
                    uint4 (&Pcons)[CB][KS], uint4 (&Pprod)[CB][KS]) {
        constexpr bool STEADY = decltype(steady_tag)::value;
        const unsigned char* stage = decltype(parity_tag)::value ? s_stage1 : s_stage0;   // this iteration's stage
        const bool do_qk = STEADY || it < wt;
        const bool do_sm = STEADY || (it >= 1 && it <= wt);
        const bool do_pv = STEADY || (it >= 2 && it <= wt + 1);

        // the accumulators (tiles <= it - 3) move to the maximum the previous iteration found; P(it - 2),
        // added below, already refers to it
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            if (__builtin_amdgcn_ballot_w64(alpha[cb] != 1.f) != 0) {
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) O[cb][nb] *= alpha[cb];
            }
            alpha[cb] = 1.f;
        }

        // ---- the softmax of S(it - 1) as a list of small steps.
        // Maximum phase: steps 0..7 reduce the lane's 16 scores of each column block with a tree of
        // three-input maxima, 8 and 9 fold the four k groups of a column, 10 derives the factors.
        float t1[CB][5], t2[CB][2], mloc[CB], mc[CB], psum[CB];
        auto sc = [&](int cb, int idx) -> float { return Scons[cb][idx >> 2][idx & 3]; };
        auto max_step = [&](int k) {
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
                if (k < 5) t1[cb][k] = fmaxf(fmaxf(sc(cb, 3 * k), sc(cb, 3 * k + 1)), sc(cb, 3 * k + 2));
                else if (k == 5) t2[cb][0] = fmaxf(fmaxf(t1[cb][0], t1[cb][1]), t1[cb][2]);
                else if (k == 6) t2[cb][1] = fmaxf(fmaxf(t1[cb][3], t1[cb][4]), sc(cb, 15));
                else if (k == 7) mloc[cb] = fmaxf(t2[cb][0], t2[cb][1]);
                else if (k == 8) mloc[cb] = fmaxf(mloc[cb], __shfl_xor(mloc[cb], 16, kWaveSize));
                else if (k == 9) mloc[cb] = fmaxf(mloc[cb], __shfl_xor(mloc[cb], 32, kWaveSize));
                else {
                    const float m_new = fmaxf(m_run[cb], mloc[cb]);
                    alpha[cb] = fast_exp2((m_run[cb] - m_new) * c);
                    l_part[cb] *= alpha[cb];
                    m_run[cb] = m_new;
                    mc[cb] = m_new * c;
                    psum[cb] = 0.f;
                }
            }
        };
        // Exponential phase in half steps: 2e turns score e into 2^(s c - m c), 2e + 1 adds it to the
        // row sum and, for odd e, packs scores e - 1 and e into a word of P.
        auto exp_half = [&](int hs) {
            const int e = hs >> 1;
            const int cb = e / (NG * 4), tg = (e >> 2) % NG, j = e & 3;
            if ((hs & 1) == 0) {
                Scons[cb][tg][j] = fast_exp2(fmaf(Scons[cb][tg][j], c, -mc[cb]));
            } else {
                psum[cb] += Scons[cb][tg][j];
                if (j & 1) {
                    const uint32_t w = pack_bf16x2(Scons[cb][tg][j - 1], Scons[cb][tg][j]);
                    uint4& dst = Pprod[cb][tg >> 1];
                    const int slot = (tg & 1) * 2 + (j >> 1);
                    if (slot == 0) dst.x = w; else if (slot == 1) dst.y = w; else if (slot == 2) dst.z = w; else dst.w = w;
                }
            }
        };
        auto mask_scores = [&]() {
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
                for (int tg = 0; tg < NG; ++tg) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if ((it - 1) * TK + tg * 16 + 4 * fg + j >= col_limit[cb]) Scons[cb][tg][j] = kMaskedScore;
                    }
                }
            }
        };

        auto qk_mfma = [&](const uint4& a, int g, int cb) {
            const int tg = g / KC, m = g % KC;
            const f32x4_t acc = (m == 0) ? f32x4_t{0.f, 0.f, 0.f, 0.f} : Sprod[cb][tg];
            Sprod[cb][tg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), qfrag[cb][m], acc, 0, 0, 0);
        };
        auto pv_mfma = [&](const s16x8_t& vv, int h, int cb) {
            const int ks = h / NB, nb = h % NB;
            O[cb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vv),
                                                                __builtin_bit_cast(bf16x8_t, Pcons[cb][ks]), O[cb][nb], 0, 0, 0);
        };
        auto read_k = [&](int g) {
            return *reinterpret_cast<const uint4*>(stage + ak[g % KC] + (g / KC) * 16 * ROWB);
        };
        // the k slots of a 32-token step pair (fg, i) with token 4*fg + i of the step's first 16-token
        // group for i < 4 and of its second group for i >= 4
        auto read_v = [&](int h) {
            const int ks = h / NB, nb = h % NB;
            const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                L3_LDS_PTR(s16x4_t, stage + av[nb] + (2 * ks) * 16 * ROWB));
            const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                L3_LDS_PTR(s16x4_t, stage + av[nb] + (2 * ks + 1) * 16 * ROWB));
            return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        };

        if constexpr (STEADY) {
            // Hand-placed order: O^T += V^T P(it - 2) first, then S(it) = K Q^T, so that the registers of
            // P(it - 2) and of the exponentiated scores are free when S(it) needs its own.  Every matrix
            // instruction is followed by the vector work that fits into the cycles it occupies the
            // matrix pipe; an LDS operand is requested one group ahead.  Nothing moves across the fences.
            // LDS operands travel through a ring of four register slots, requested three groups ahead.
            constexpr int AHEAD = 3, PRE = 4;   // PRE: maximum-phase steps taken while the first operands are on their way
            uint4 ring[AHEAD + 1];
            auto request = [&](auto gc) {
                constexpr int g = decltype(gc)::value;
                if constexpr (g < GP) ring[g % (AHEAD + 1)] = __builtin_bit_cast(uint4, read_v(g));
                else if constexpr (g < GP + GQ) ring[g % (AHEAD + 1)] = read_k(g - GP);
            };
            static_for<AHEAD>([&](auto gc) { request(gc); });
            static_for<PRE>([&](auto kc) { max_step(decltype(kc)::value); });
            __builtin_amdgcn_sched_barrier(0);
            static_for<GP + GQ>([&](auto gc) {
                constexpr int g = decltype(gc)::value;
                request(std::integral_constant<int, g + AHEAD>{});
                static_for<CB>([&](auto cc) {
                    constexpr int cb = decltype(cc)::value;
                    constexpr int i = g * CB + cb;   // matrix instruction index
                    if constexpr (g < GP) pv_mfma(__builtin_bit_cast(s16x8_t, ring[g % (AHEAD + 1)]), g, cb);
                    else qk_mfma(ring[g % (AHEAD + 1)], g - GP, cb);
                    if constexpr (i + PRE < MS) {
                        max_step(i + PRE);
                    } else {
                        constexpr int n = NM - (MS - PRE), k = i - (MS - PRE);
                        constexpr int h0 = k * (2 * NE) / n, h1 = (k + 1) * (2 * NE) / n;
                        static_for<h1 - h0>([&](auto hc) { exp_half(h0 + decltype(hc)::value); });
                    }
                    __builtin_amdgcn_sched_barrier(0);
                });
            });
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) l_part[cb] += psum[cb];
        } else {
            if (do_sm) {
                mask_scores();
#pragma unroll
                for (int k = 0; k < MS; ++k) max_step(k);
#pragma unroll
                for (int hs = 0; hs < 2 * NE; ++hs) exp_half(hs);
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) l_part[cb] += psum[cb];
            }
            if (do_pv) {
#pragma unroll
                for (int h = 0; h < GP; ++h) {
                    const s16x8_t vv = read_v(h);
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) pv_mfma(vv, h, cb);
                }
            }
            if (do_qk) {
#pragma unroll
                for (int g = 0; g < GQ; ++g) {
                    const uint4 a = read_k(g);
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) qk_mfma(a, g, cb);
                }
            }
        }
    };

    auto run = [&](auto parity_tag, int it, f32x4_t (&Sprod)[CB][NG], f32x4_t (&Scons)[CB][NG],
                   uint4 (&Pcons)[CB][KS], uint4 (&Pprod)[CB][KS]) {
        constexpr int PAR = decltype(parity_tag)::value;
        const bool more = it + 1 < n_it;   // workgroup-uniform
        // the other stage was last read before the previous barrier: its refill can start now
        if (more) dma(it + 1, PAR ? s_stage0 : s_stage1);
        if (it >= 2 && it < wt && it * TK <= wave_limit_min) {
            body(std::true_type{}, parity_tag, it, Sprod, Scons, Pcons, Pprod);
        } else {
            body(std::false_type{}, parity_tag, it, Sprod, Scons, Pcons, Pprod);
        }
        __builtin_amdgcn_s_waitcnt(0xF70);   // vmcnt(0): this wavefront's part of the next stage has landed
        __syncthreads();
    };

    dma(0, s_stage0);
    __builtin_amdgcn_s_waitcnt(0xF70);
    __syncthreads();

    f32x4_t SA[CB][NG], SB[CB][NG];
    uint4 PA[CB][KS], PB[CB][KS];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
        for (int tg = 0; tg < NG; ++tg) SA[cb][tg] = SB[cb][tg] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) PA[cb][ks] = PB[cb][ks] = make_uint4(0u, 0u, 0u, 0u);
    }
    for (int it = 0; it < n_it; it += 2) {
        run(std::integral_constant<int, 0>{}, it, SA, SB, PA, PB);
        if (it + 1 < n_it) run(std::integral_constant<int, 1>{}, it + 1, SB, SA, PB, PA);
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

template <class Kernel>
int launch_blocks(Kernel kernel, const PrefillParams& p, int waves, int col_blocks, hipStream_t stream) {
    const int R = p.QH / p.KVH;
    const int wg_pos = waves * col_blocks * (16 / R);
    const int wgs_per_head = (p.T + wg_pos - 1) / wg_pos;
    const dim3 grid(unsigned(p.B) * unsigned(p.KVH) * unsigned(wgs_per_head));
    hipLaunchKernelGGL(kernel, grid, dim3(waves * kWaveSize), 0, stream, p);
    return int(hipGetLastError());
}

}  // namespace

int launch_attn_prefill_tiled(const PrefillParams& p, int HD, bool pipelined, hipStream_t stream) {
    constexpr int CB = kPrefillColBlocks, TW = kPrefillTiledWaves;
    if (pipelined) {
        if (HD == 64) return launch_blocks(attn_prefill_pipe_kernel<64, CB, prefill_pipe_waves(64)>, p, prefill_pipe_waves(64), CB, stream);
        return launch_blocks(attn_prefill_pipe_kernel<128, CB, prefill_pipe_waves(128)>, p, prefill_pipe_waves(128), CB, stream);
    }
    // tiles of 64 tokens; four wavefronts per SIMD at head size 64 (four workgroups per compute unit), two
    // at 128 (two workgroups: a stage pair is 64 KiB)
    if (HD == 64) return launch_blocks(attn_prefill_tiled_kernel<64, CB, TW, 64, 4>, p, TW, CB, stream);
    return launch_blocks(attn_prefill_tiled_kernel<128, CB, TW, 64, 2>, p, TW, CB, stream);
}

}  // namespace l3
