// The tile loop shared by the MFMA attention kernels (decode: attn_mfma.hip, prefill:
// attn_prefill.hip): one wavefront streams K/V tiles of a single kv head through its private LDS
// slab and keeps an online softmax for the 16 columns of its MFMA tiles.  A column is a query
// row: a query head of the GQA group (decode) or a (query position, query head) pair (prefill).
//
//   S[16 tokens x 16 columns]  = K[16 x 32 dims]          . Q^T[32 dims x 16 columns]  (per 32-dim chunk)
//   O^T[16 dims x 16 columns] += V^T[16 dims x 32 tokens] . P[32 tokens x 16 columns]  (per 16-dim block)
//
// with v_mfma_f32_16x16x32_bf16.  A tile (32 tokens at HD 128, 64 at HD 64: 16 KiB of K+V) is
// loaded with 16-byte global loads that each cover whole head rows, written to the slab and read
// back in operand layout: ds_read_b128 for K (lane = token row, 8 consecutive dims),
// ds_read_b64_tr_b16 for V, whose transpose turns token-major rows into "8 tokens of one dim" per
// lane.  Slab rows are padded (16 bytes for K, 32 for V) to keep both read patterns off the same
// banks.  The S accumulator layout (lane = column, 4 token rows) is exactly the B-operand layout
// of the second product, so P never moves between lanes.  LDS executes one wavefront's accesses in
// order, which is all the synchronisation the slab needs.
#pragma once

#include <type_traits>

#include "attn_common.hpp"

namespace l3 {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(8))) short s16x8_t;

#define L3_LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))

// Keeps the compiler from moving LDS accesses across a phase boundary of the slab (the
// hardware already executes one wavefront's LDS accesses in order).
__device__ __forceinline__ void lds_phase_fence() { asm volatile("" ::: "memory"); }

template <int HD, int LOADS = 8>
struct MfmaTile {
    static constexpr int LPR = HD / 8;            // lanes per token row in a global load
    static constexpr int G = kWaveSize / LPR;     // token rows per wavefront-wide load
    static constexpr int U = LOADS;               // loads of K (and of V) per tile and lane (8; 4 = a half tile)
    static constexpr int WT = U * G;              // tokens per wavefront tile: 32 (HD 128) or 64 (HD 64)
    static constexpr int NG = WT / 16;            // 16-token groups per tile (rows of one S tile)
    static constexpr int KC = HD / 32;            // 32-dim chunks of the head dimension
    static constexpr int NB = HD / 16;            // 16-dim blocks of the output
    static constexpr int KS = WT / 32;            // 32-token steps of the second product
    static constexpr int KPITCH = HD * 2 + 16;    // slab row pitch while it holds K
    static constexpr int VPITCH = HD * 2 + 32;    // slab row pitch while it holds V
    static constexpr int SLAB = WT * VPITCH;      // bytes of LDS per wavefront
};

// A wave-uniform value as the compiler sees it (kept in scalar registers, so that address arithmetic
// built on it runs on the scalar unit).  The caller guarantees that all lanes hold the same value.
__device__ __forceinline__ int wave_uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }
__device__ __forceinline__ int64_t wave_uniform(int64_t x) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane(uint32_t(uint64_t(x)));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(uint32_t(uint64_t(x) >> 32));
    return int64_t((uint64_t(hi) << 32) | lo);
}

// Makes every element of a register array a live value at this point: the loads that produce them
// have all been issued before anything that follows can wait for the first one.  (Left alone, the
// scheduler sinks each LDS read next to its consumer and the wavefront pays the LDS latency once per
// product instead of once per phase.)
template <typename V>
__device__ __forceinline__ void pin_all(V (&x)[4]) {
    asm volatile("" : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]));
}
template <typename V>
__device__ __forceinline__ void pin_all(V (&x)[8]) {
    asm volatile("" : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "+v"(x[4]), "+v"(x[5]), "+v"(x[6]), "+v"(x[7]));
}
template <typename V>
__device__ __forceinline__ void pin_all(V (&x)[16]) {
    asm volatile("" : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "+v"(x[4]), "+v"(x[5]), "+v"(x[6]), "+v"(x[7]),
                      "+v"(x[8]), "+v"(x[9]), "+v"(x[10]), "+v"(x[11]), "+v"(x[12]), "+v"(x[13]), "+v"(x[14]),
                      "+v"(x[15]));
}

// Maximum over the four lanes l, l^16, l^32, l^48 (the four k groups of an MFMA column), in every
// one of them: two v_permlane*_swap and two v_max instead of two trips through the LDS crossbar.
// permlane32_swap(x, x) yields (x with its upper half replaced by the lower half, x with its lower
// half replaced by the upper half), whose maximum is max(x[l], x[l^32]); permlane16_swap does the
// same with the odd and even rows of 16 lanes.
__device__ __forceinline__ float column_max(float x) {
    const uint32_t xi = __builtin_bit_cast(uint32_t, x);
    const auto h = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
    const float y = fmaxf(__builtin_bit_cast(float, uint32_t(h[0])), __builtin_bit_cast(float, uint32_t(h[1])));
    const uint32_t yi = __builtin_bit_cast(uint32_t, y);
    const auto r = __builtin_amdgcn_permlane16_swap(yi, yi, false, false);
    return fmaxf(__builtin_bit_cast(float, uint32_t(r[0])), __builtin_bit_cast(float, uint32_t(r[1])));
}

// Streams the tiles t_first, t_first + step, ... < t_end of one kv head (token 0 of the head is
// element k[k_head] / v[v_head] of the K / V arrays; token strides in elements, below 2^24) and
// updates the wavefront's softmax state.  k_head, v_head, t_first, t_end and step are wave-uniform.  `qfrag` is the B operand of the
// first product: lane (column fn, k group fg) holds dims (m*4 + fg)*8 .. +8 of its column's query
// row.  A score of token t against this lane's column counts only if t < col_limit (col_limit_min =
// the smallest limit in the wavefront, wave-uniform; tiles below it skip the masking).  On return
// O[nb][r] is dim 16*nb + 4*fg + r of column fn (unnormalised), m_run the column's running maximum
// of the raw scores (shared by its four k groups) and l_part this lane's share of the column's
// softmax denominator.
// STREAM: K/V are read once by the whole grid (decode), so they are loaded non-temporally; the
// prefill form, whose column groups re-read the same tiles from cache, keeps plain loads.
//
// A load's address is a scalar 64-bit tile base plus a 32-bit lane offset that does not change from
// tile to tile (row of the load times the token pitch, clamped to the last valid row of a ragged
// final tile, plus the lane's 16-byte chunk), so the loop spends two vector instructions per load on
// addresses.  Every tile but the last issues the next tile's loads unconditionally, which lets the
// K wait leave the V loads in flight.
// ROTATE: the tiles are taken in rotated order -- the wavefront's i-th tile is tile (first + rot + i step)
// modulo the number of tiles between t_first0 (the first token of the whole range the workgroup shares;
// t_first = t_first0 + first tiles) and t_end, so that workgroups whose ranges start a power of two apart
// do not all begin at addresses a power of two apart.  The order does not change the result beyond
// float32 rounding: the softmax state is order-free.
template <int HD, int LOADS = 8, bool STREAM = false, bool ROTATE = false>
__device__ __forceinline__ void mfma_tile_loop(const uint16_t* __restrict__ k, const uint16_t* __restrict__ v,
                                               int64_t k_head, int64_t v_head, int64_t k_st, int64_t v_st,
                                               unsigned char* slab,
                                               const bf16x8_t (&qfrag)[MfmaTile<HD>::KC], int t_first, int t_end,
                                               int step, int col_limit, int col_limit_min, float c,
                                               f32x4_t (&O)[MfmaTile<HD>::NB], float& m_run, float& l_part,
                                               int t_first0 = 0, int rot = 0) {
    using T = MfmaTile<HD, LOADS>;
    static_assert(T::WT % 32 == 0, "a tile is a whole number of 32-token steps of the second product");
    constexpr int LPR = T::LPR, G = T::G, U = T::U, WT = T::WT, NG = T::NG, KC = T::KC, NB = T::NB, KS = T::KS;
    constexpr int KPITCH = T::KPITCH, VPITCH = T::VPITCH;
    const int lane = threadIdx.x & (kWaveSize - 1);
    const int ld_row = lane / LPR;   // role in a global load: token row within the load ...
    const int ld_c = lane % LPR;     // ... and 16-byte chunk of that row
    const int fg = lane >> 4;        // role in an MFMA operand: k group (lane & 15 = row/column index)

    unsigned char* wr_k = slab + ld_row * KPITCH + ld_c * 16;
    unsigned char* wr_v = slab + ld_row * VPITCH + ld_c * 16;
    const unsigned char* rd_k = slab + (lane & 15) * KPITCH + fg * 16;
    // transpose read: the 16 lanes of k group fg present a 4-token x 16-dim patch, row-major
    const unsigned char* rd_v = slab + (4 * fg + ((lane & 15) >> 2)) * VPITCH + (lane & 3) * 8;

    const char* kh = reinterpret_cast<const char*>(k) + wave_uniform(k_head) * 2;
    const char* vh = reinterpret_cast<const char*>(v) + wave_uniform(v_head) * 2;
    const int64_t k_pitch = wave_uniform(int(k_st)) * int64_t(2);   // bytes from a token to the next (< 2^25)
    const int64_t v_pitch = wave_uniform(int(v_st)) * int64_t(2);
    t_first = wave_uniform(t_first);
    t_end = wave_uniform(t_end);
    step = wave_uniform(step);
    const uint32_t chunk = uint32_t(ld_c) * 16u;
    uint32_t krow[U], vrow[U];   // byte offset of this lane's row of load u inside a tile
#pragma unroll
    for (int u = 0; u < U; ++u) {
        krow[u] = uint32_t(u * G + ld_row) * uint32_t(k_pitch);
        vrow[u] = uint32_t(u * G + ld_row) * uint32_t(v_pitch);
    }

    uint4 kr[U], vr[U];
    auto load_tile = [&](uint4 (&dst)[U], const char* head, int64_t pitch, const uint32_t (&row)[U], int tbase) {
        const char* tb = head + int64_t(tbase) * pitch;                               // scalar
        const uint32_t last = uint32_t(min(t_end - 1 - tbase, WT - 1)) * uint32_t(pitch);   // scalar: last valid row
#pragma unroll
        for (int u = 0; u < U; ++u) {
            // rows past the end of a ragged tile re-read its last row and are masked below
            const uint16_t* src = reinterpret_cast<const uint16_t*>(tb + (min(row[u], last) + chunk));
            dst[u] = STREAM ? load16_stream(src) : load16(src);
        }
    };

    auto tile = [&](const int t0, const int tn, auto has_next) {
        constexpr bool NEXT = decltype(has_next)::value;
        // ---- K tile -> slab; its registers are free again, so the next K tile starts loading
#pragma unroll
        for (int u = 0; u < U; ++u) *reinterpret_cast<uint4*>(wr_k + u * G * KPITCH) = kr[u];
        lds_phase_fence();
        if constexpr (NEXT) load_tile(kr, kh, k_pitch, krow, tn);

        // ---- S = K Q^T: all operand reads first, then the products with the NG chains interleaved
        u32x4_t a[NG * KC];
#pragma unroll
        for (int tg = 0; tg < NG; ++tg) {
#pragma unroll
            for (int m = 0; m < KC; ++m) {
                a[tg * KC + m] = *reinterpret_cast<const u32x4_t*>(rd_k + tg * 16 * KPITCH + m * 64);
            }
        }
        pin_all(a);   // all eight reads are in flight before the first product waits
        f32x4_t S[NG];
#pragma unroll
        for (int tg = 0; tg < NG; ++tg) S[tg] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int m = 0; m < KC; ++m) {
#pragma unroll
            for (int tg = 0; tg < NG; ++tg) {
                S[tg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[tg * KC + m]), qfrag[m],
                                                                S[tg], 0, 0, 0);
            }
        }
        lds_phase_fence();

        // S[tg][j] is token t0 + tg*16 + 4*fg + j against column fn.  Mask what the column may not
        // see (the ragged tail of the range; for prefill, tokens after the query's position).
        if (t0 + WT > col_limit_min) {
#pragma unroll
            for (int tg = 0; tg < NG; ++tg) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (t0 + tg * 16 + 4 * fg + j >= col_limit) S[tg][j] = kMaskedScore;
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
        mloc = column_max(mloc);
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
        if constexpr (NEXT) load_tile(vr, vh, v_pitch, vrow, tn);

        // ---- O^T += V^T P.  k slot (fg, i) of a 32-token step is token 4*fg + i of its first
        //      16-token group for i < 4 and of its second group for i >= 4, on both operands.
        s16x4_t vt[KS * NB * 2];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                vt[(ks * NB + nb) * 2] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    L3_LDS_PTR(s16x4_t, rd_v + (2 * ks) * 16 * VPITCH + nb * 32));
                vt[(ks * NB + nb) * 2 + 1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    L3_LDS_PTR(s16x4_t, rd_v + (2 * ks + 1) * 16 * VPITCH + nb * 32));
            }
        }
        pin_all(vt);   // sixteen transpose reads in flight, then the products back to back
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
                const s16x8_t vv = __builtin_shufflevector(vt[(ks * NB + nb) * 2], vt[(ks * NB + nb) * 2 + 1], 0, 1, 2,
                                                           3, 4, 5, 6, 7);
                O[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vv), pfrag, O[nb],
                                                                0, 0, 0);
            }
        }
        lds_phase_fence();
    };

    if (t_first >= t_end) return;   // a wavefront without a tile keeps its empty softmax state
    if constexpr (ROTATE) {
        t_first0 = wave_uniform(t_first0);
        const int tiles = (t_end - t_first0 + WT - 1) / WT;              // of the whole range
        const int tstep = step / WT;
        int left = (tiles - (t_first - t_first0) / WT + tstep - 1) / tstep;   // tiles of this wavefront (>= 1)
        int idx = ((t_first - t_first0) / WT + wave_uniform(rot)) % tiles;
        int t0 = t_first0 + idx * WT;
        load_tile(kr, kh, k_pitch, krow, t0);
        load_tile(vr, vh, v_pitch, vrow, t0);
        for (; left > 1; --left) {
            idx += tstep;
            if (idx >= tiles) idx -= tiles;
            const int tn = t_first0 + idx * WT;
            tile(t0, tn, std::true_type{});
            t0 = tn;
        }
        tile(t0, t0, std::false_type{});
    } else {
        int t0 = t_first;
        load_tile(kr, kh, k_pitch, krow, t0);
        load_tile(vr, vh, v_pitch, vrow, t0);
        for (; t0 + step < t_end; t0 += step) tile(t0, t0 + step, std::true_type{});
        tile(t0, t0, std::false_type{});
    }
}

}  // namespace l3
