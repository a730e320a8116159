// y[M, N] = x[M, K] . W[N, K]^T for the few rows of a decode step (M <= 16), bf16 in and out,
// float32 accumulation: the nn.Linear calls of model.py:95,121,134,225 when T == 1.  With so few
// rows the product is a stream over the weight matrix, so the kernel is built like the attention
// kernels: HBM-bound, every weight byte read once, 16-byte loads kept in flight.
//
//   C[16 weight rows x 16 activation rows] += W[16 x 32 k] . x^T[32 k x 16]   (v_mfma_f32_16x16x32_bf16)
//
// A lane of the A operand holds 8 consecutive k of one weight row, which is exactly a 16-byte
// global load: weights go from HBM into operand registers with no staging.  A wavefront owns 16
// weight rows over a slice of K; the `sk` wavefronts that share a row block meet in LDS.
//
// What a transformer block does around its linears rides along (each optional):
//   * RMSNorm of the input (model.py:147-148, ln_1 / ln_2 in front of c_attn / the MLP): with at
//     most 16 activation rows the workgroup first writes the normalised x into LDS, with the
//     rounding of the stand-alone operator (bf16(x * inv_rms * w)), and the B operands come
//     from there;
//   * SwiGLU: the wavefront streams the same rows of two matrices and writes
//     bf16(silu(x.Wg^T)) * bf16(x.Wu^T) with torch's rounding points (model.py:134);
//   * the residual addition that follows c_proj and the MLP (model.py:147-148):
//     y = bf16(residual + bf16(x.W^T)), the two roundings of the separate operators.
#include "attn_mfma_core.hpp"

namespace l3 {

namespace {

// Epilogue of the fused qkv projection: features n, n + 1 (n even) of activation row m, already
// rounded to bf16 and packed in xw.  Query and key pairs are rotated at the device-side position,
// keys and values land in the KV cache row of that position (model.py:100-106).
__device__ __forceinline__ void store_qkv_pair(const LinearParams& p, int m, int n, uint32_t xw) {
    const int pos = *p.rope_pos;
    if (pos < 0 || pos >= p.cache_len || pos >= p.table_rows) return;   // never write outside the cache
    const int slot = n / p.HD;
    const int d = n % p.HD;
    if (slot >= p.NH + p.KVH) {
        *reinterpret_cast<uint32_t*>(p.cache_v + m * p.c_sb + pos * p.c_st + (slot - p.NH - p.KVH) * p.HD + d) = xw;
        return;
    }
    const float2 cs = *reinterpret_cast<const float2*>(p.rope_table + int64_t(pos) * p.HD + d);
    const uint32_t yw = rotate_pair(xw, cs.x, cs.y);
    if (slot < p.NH) {
        *reinterpret_cast<uint32_t*>(p.q_out + (int64_t(m) * p.NH + slot) * p.HD + d) = yw;
    } else {
        *reinterpret_cast<uint32_t*>(p.cache_k + m * p.c_sb + pos * p.c_st + (slot - p.NH) * p.HD + d) = yw;
    }
}

// Elements of LDS the staged activations may take (rows are padded by 8 elements).
constexpr int kXldsMaxElems = 24576;

// RW = weight rows per wavefront.  16: the plain mapping above.  4 (at most 4 activation rows):
// the 16 rows and the 16 columns of a matrix instruction are both split into four k
// ranges -- tile row i is weight row i % 4 over k range i / 4, tile column j is activation row
// j % 4 over k range j / 4 -- so one instruction covers 4 weight rows x 128 k, the blocks on the
// diagonal (i / 4 == j / 4) hold the products and the rest is ignored.  Four times as many
// wavefronts share a matrix with few rows, and a weight row is read 256 contiguous bytes at a time.
template <int NW, int CBLK, int U, bool SWIGLU, bool XLDS, int RW>
__global__ void __launch_bounds__(NW * kWaveSize)
linear_skinny_kernel(const LinearParams p) {
    static_assert(!XLDS || CBLK == 1, "activations are staged in LDS only for up to 16 rows");
    static_assert(RW == 16 || (RW == 4 && CBLK == 1), "the four-row mapping takes at most four activation rows");
    constexpr int KQ = 16 / RW;                            // k ranges per matrix instruction
    constexpr int KSTEP = 32 * KQ;                         // k covered by one step
    constexpr int ACC = SWIGLU ? 2 : 1;
    __shared__ float s_red[NW][ACC][CBLK][256];
    extern __shared__ __align__(16) uint16_t s_x[];        // XLDS: M rows of K + 8 elements

    const int lane = threadIdx.x & (kWaveSize - 1);
    const int wave = __builtin_amdgcn_readfirstlane(int(threadIdx.x) / kWaveSize);   // scalar: what derives from it is wave-uniform
    const int fn = lane & 15;
    const int fg = lane >> 4;

    const int sk = p.sk;                                   // wavefronts per row block (divides NW)
    const int rb = int(blockIdx.x) * (NW / sk) + wave / sk;
    const int kslice = wave % sk;
    const int n0 = rb * RW;
    const int ksteps = p.K / KSTEP;
    const int kpw = (ksteps + sk - 1) / sk;
    const int ks0 = kslice * kpw;
    const int ks1 = min(ksteps, ks0 + kpw);

    const int row = min(n0 + fn % RW, p.N - 1);            // rows past N are loaded clamped and never stored
    const int koff = (fn / RW) * 32 + fg * 8;              // this lane's k offset within a step
    const uint16_t* wp0 = p.w0 + int64_t(row) * p.w_stride + koff;
    const uint16_t* wp1 = SWIGLU ? p.w1 + int64_t(row) * p.w_stride + koff : nullptr;
    const uint16_t* xp[CBLK];
    bool xvalid[CBLK];
#pragma unroll
    for (int cb = 0; cb < CBLK; ++cb) {
        xvalid[cb] = cb * 16 + fn % RW < p.M;
        xp[cb] = p.x + int64_t(xvalid[cb] ? cb * 16 + fn % RW : 0) * p.x_stride + koff;
    }

    f32x4_t acc[ACC][CBLK];
#pragma unroll
    for (int a = 0; a < ACC; ++a) {
#pragma unroll
        for (int cb = 0; cb < CBLK; ++cb) acc[a][cb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }

    // A ring of U k steps in registers: a slot is refilled for step ks + U as soon as the matrix
    // instructions of step ks have read it, so about U loads per operand stay in flight.
    uint4 rw0[U], rw1[SWIGLU ? U : 1], rx[XLDS ? 1 : CBLK][XLDS ? 1 : U];
    auto fill = [&](int u, int ks) {
        rw0[u] = load16_stream(wp0 + ks * KSTEP);   // every weight byte is read once (batch-1 decode: +3.5 % tokens/s)
        if constexpr (SWIGLU) rw1[u] = load16_stream(wp1 + ks * KSTEP);
        if constexpr (!XLDS) {
#pragma unroll
            for (int cb = 0; cb < CBLK; ++cb) {
                rx[cb][u] = xvalid[cb] ? load16(xp[cb] + ks * KSTEP) : make_uint4(0u, 0u, 0u, 0u);
            }
        }
    };
    // RMSNorm of the activations into LDS (XLDS).  The workgroup shares the 16-byte chunks of all
    // rows; K % 512 == 0, so the 64 chunks of a wavefront lie in one row and the row's sum of squares
    // is a fixed-order sum of per-wavefront parts.  A thread's first chunk stays in registers and
    // its loads are issued BEFORE the weight ring is filled (loads return in order, and the norm
    // must not wait behind kilobytes of weights coming from HBM); with more than two rows the
    // further chunks go through LDS, one at a time, so that the prologue costs few registers.
    constexpr int NT = NW * kWaveSize;
    const int KP = p.K + 8;                                // LDS row pitch in elements
    const int cpr = p.K / 8;                               // chunks per row
    const int nchunks = p.M * cpr;
    uint4 xv0 = make_uint4(0u, 0u, 0u, 0u), gv0 = xv0;
    if constexpr (XLDS) {
        const int c = int(threadIdx.x);
        if (c < nchunks) {                                 // wave-uniform
            xv0 = load16(p.x + int64_t(c / cpr) * p.x_stride + (c % cpr) * 8);
            gv0 = load16(p.norm_w + (c % cpr) * 8);
        }
    }
    auto norm_prologue = [&]() {
        __shared__ float s_part[kXldsMaxElems / 8 / kWaveSize];
        const int parts_per_row = cpr / kWaveSize;
        for (int c = int(threadIdx.x), it = 0; c < nchunks; c += NT, ++it) {
            const int r = c / cpr, col = c % cpr;
            uint4 v = xv0;
            if (it > 0) {
                v = load16(p.x + int64_t(r) * p.x_stride + col * 8);
                *reinterpret_cast<uint4*>(s_x + r * KP + col * 8) = v;   // raw, re-read by this thread below
            }
            float f[8];
            unpack8(v, f);
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) ss = fmaf(f[i], f[i], ss);
            ss = wave_sum(ss);
            if (lane == 0) s_part[c / kWaveSize] = ss;
        }
        __syncthreads();
        for (int c = int(threadIdx.x), it = 0; c < nchunks; c += NT, ++it) {
            const int r = c / cpr, col = c % cpr;
            float ss = 0.f;
            for (int q = 0; q < parts_per_row; ++q) ss += s_part[r * parts_per_row + q];
            const float inv = rsqrtf(ss / float(p.K) + p.norm_eps);
            float f[8], g[8];
            unpack8(it == 0 ? xv0 : *reinterpret_cast<const uint4*>(s_x + r * KP + col * 8), f);
            unpack8(it == 0 ? gv0 : load16(p.norm_w + col * 8), g);
            uint4 o;
            o.x = pack_bf16x2(f[0] * inv * g[0], f[1] * inv * g[1]);
            o.y = pack_bf16x2(f[2] * inv * g[2], f[3] * inv * g[3]);
            o.z = pack_bf16x2(f[4] * inv * g[4], f[5] * inv * g[5]);
            o.w = pack_bf16x2(f[6] * inv * g[6], f[7] * inv * g[7]);
            *reinterpret_cast<uint4*>(s_x + r * KP + col * 8) = o;
        }
        __syncthreads();
    };
    // Initial ring fill, then the norm.  The weight loads sit BEHIND the activation loads in the
    // wavefront's in-order memory queue; when their number is known at compile time (a full ring
    // or half of one: the common cases) the compiler waits for the activations alone, otherwise
    // it has to wait for everything.
    const int nst = ks1 - ks0;
    if (nst >= U) {
#pragma unroll
        for (int u = 0; u < U; ++u) fill(u, ks0 + u);
        if constexpr (XLDS) norm_prologue();
    } else if (nst == U / 2) {
#pragma unroll
        for (int u = 0; u < U / 2; ++u) fill(u, ks0 + u);
        if constexpr (XLDS) norm_prologue();
    } else {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (ks0 + u < ks1) fill(u, ks0 + u);
        }
        if constexpr (XLDS) norm_prologue();
    }
    const uint16_t* lx = s_x + (xvalid[0] ? fn % RW : 0) * KP + koff;

    for (int ks = ks0; ks < ks1; ks += U) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (ks + u < ks1) {                            // wave-uniform
#pragma unroll
                for (int cb = 0; cb < CBLK; ++cb) {
                    uint4 xv;
                    if constexpr (XLDS) {
                        xv = *reinterpret_cast<const uint4*>(lx + (ks + u) * KSTEP);
                        if (!xvalid[0]) xv = make_uint4(0u, 0u, 0u, 0u);
                    } else {
                        xv = rx[cb][u];
                    }
                    const bf16x8_t xf = __builtin_bit_cast(bf16x8_t, xv);
                    acc[0][cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, rw0[u]), xf,
                                                                         acc[0][cb], 0, 0, 0);
                    if constexpr (SWIGLU) {
                        acc[ACC - 1][cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(bf16x8_t, rw1[u]), xf, acc[ACC - 1][cb], 0, 0, 0);
                    }
                }
                if (ks + U + u < ks1) fill(u, ks + U + u);
            }
        }
    }

    if constexpr (RW == 4) {
        // acc[0][0][t] of lane l is tile row 4*(l/16) + t, column l % 16: weight row n0 + t over k
        // range l / 16 against activation row (l % 16) % 4 over k range (l % 16) / 4.  The lanes
        // whose two k ranges agree hold products; they meet, with the other wavefronts of the row
        // group, in LDS, and the group's first wavefront finishes its 4 x 4 results.
        if ((fn >> 2) == fg) {
#pragma unroll
            for (int a = 0; a < ACC; ++a) {
#pragma unroll
                for (int t = 0; t < 4; ++t) s_red[wave][a][0][(fg * 4 + (fn & 3)) * 4 + t] = acc[a][0][t];
            }
        }
        __syncthreads();
        if (kslice != 0 || lane >= 16) return;
        const int m = lane >> 2, t = lane & 3;             // activation row, weight row within the group
        const int n = n0 + t;
        float oa[ACC];
#pragma unroll
        for (int a = 0; a < ACC; ++a) {
            oa[a] = 0.f;
            for (int w = 0; w < sk; ++w) {
#pragma unroll
                for (int q = 0; q < 4; ++q) oa[a] += s_red[wave + w][a][0][(q * 4 + m) * 4 + t];
            }
        }
        float o = oa[0];
        if constexpr (SWIGLU) {
            const float g = __uint_as_float(f32_to_bf16_bits(oa[0]) << 16);
            const float u = __uint_as_float(f32_to_bf16_bits(oa[ACC - 1]) << 16);
            o = silu_rounded(g) * u;
        }
        if (p.rope_table) {   // the even lane of a pair takes its partner's value and stores both
            const float o1 = __shfl_xor(o, 1, kWaveSize);
            if ((t & 1) == 0 && m < p.M && n < p.N) store_qkv_pair(p, m, n, pack_bf16x2(o, o1));
            return;
        }
        if (m >= p.M || n >= p.N) return;
        if (p.res) o = bf16_to_f32(p.res[int64_t(m) * p.y_stride + n]) + __uint_as_float(f32_to_bf16_bits(o) << 16);
        p.y[int64_t(m) * p.y_stride + n] = uint16_t(f32_to_bf16_bits(o));
        return;
    }

    // ---- the sk wavefronts of a row block add up in LDS; the first of them finishes the rows
    if (sk > 1) {
        if (kslice != 0) {
#pragma unroll
            for (int a = 0; a < ACC; ++a) {
#pragma unroll
                for (int cb = 0; cb < CBLK; ++cb) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) s_red[wave][a][cb][r * 64 + lane] = acc[a][cb][r];
                }
            }
        }
        __syncthreads();
        if (kslice != 0) return;
        for (int o = 1; o < sk; ++o) {
#pragma unroll
            for (int a = 0; a < ACC; ++a) {
#pragma unroll
                for (int cb = 0; cb < CBLK; ++cb) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[a][cb][r] += s_red[wave + o][a][cb][r * 64 + lane];
                }
            }
        }
    }

    // acc[.][cb][r] is weight row n0 + 4*fg + r against activation row cb*16 + fn
    const int n = n0 + 4 * fg;
    if (n >= p.N) return;
#pragma unroll
    for (int cb = 0; cb < CBLK; ++cb) {
        const int m = cb * 16 + fn;
        if (m >= p.M) continue;
        float o[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            if constexpr (SWIGLU) {
                const float g = __uint_as_float(f32_to_bf16_bits(acc[0][cb][r]) << 16);
                const float u = __uint_as_float(f32_to_bf16_bits(acc[1][cb][r]) << 16);
                o[r] = silu_rounded(g) * u;
            } else {
                o[r] = acc[0][cb][r];
            }
        }
        if (p.rope_table) {
            store_qkv_pair(p, m, n, pack_bf16x2(o[0], o[1]));
            store_qkv_pair(p, m, n + 2, pack_bf16x2(o[2], o[3]));
            continue;
        }
        if (p.res) {   // bf16(residual + bf16(product)), as the separate addition would give
            const uint2 rv = *reinterpret_cast<const uint2*>(p.res + int64_t(m) * p.y_stride + n);
            o[0] = bf16lo_to_f32(rv.x) + __uint_as_float(f32_to_bf16_bits(o[0]) << 16);
            o[1] = bf16hi_to_f32(rv.x) + __uint_as_float(f32_to_bf16_bits(o[1]) << 16);
            o[2] = bf16lo_to_f32(rv.y) + __uint_as_float(f32_to_bf16_bits(o[2]) << 16);
            o[3] = bf16hi_to_f32(rv.y) + __uint_as_float(f32_to_bf16_bits(o[3]) << 16);
        }
        uint2 w;
        w.x = pack_bf16x2(o[0], o[1]);
        w.y = pack_bf16x2(o[2], o[3]);
        *reinterpret_cast<uint2*>(p.y + int64_t(m) * p.y_stride + n) = w;
    }
}

template <int NW, int CBLK, int U, bool SWIGLU, bool XLDS, int RW = 16>
int launch_variant(const LinearParams& p, hipStream_t stream) {
    const int row_blocks = (p.N + RW - 1) / RW;
    const int rb_per_wg = NW / p.sk;
    const dim3 grid(unsigned((row_blocks + rb_per_wg - 1) / rb_per_wg));
    const size_t lds = XLDS ? size_t(p.M) * size_t(p.K + 8) * sizeof(uint16_t) : 0;
    hipLaunchKernelGGL((linear_skinny_kernel<NW, CBLK, U, SWIGLU, XLDS, RW>), grid, dim3(NW * kWaveSize), lds, stream,
                       p);
    return int(hipGetLastError());
}

}  // namespace

// Wavefronts per row block (of `rows_per_wave` weight rows, `kstep` k per step): split K until
// the launch has about two workgroups per CU, as long as every wavefront keeps at least four steps.
int linear_skinny_plan(int N, int K, int waves_per_wg, int num_cus, int rows_per_wave, int kstep) {
    const int row_blocks = (N + rows_per_wave - 1) / rows_per_wave;
    const int ksteps = K / kstep;
    int sk = 1;
    while (sk < waves_per_wg && int64_t(row_blocks) * sk / waves_per_wg < 2 * int64_t(num_cus) &&
           ksteps / (2 * sk) >= 4) {
        sk *= 2;
    }
    return sk;
}

// The input RMSNorm needs the activations staged in LDS: at most 16 rows that fit there, of a
// width that lets every wavefront of the staging pass stay within one row.
bool linear_skinny_can_stage(int M, int K) {
    return M <= 16 && K % 512 == 0 && int64_t(M) * (K + 8) <= kXldsMaxElems;
}

int launch_linear_skinny(LinearParams p, bool swiglu, int num_cus, hipStream_t stream) {
    if (p.M > 16) return int(hipErrorInvalidValue);   // one 16-column MFMA block of activation rows (checked by the caller)
    const bool stage = p.norm_w != nullptr;   // the caller has checked linear_skinny_can_stage
    const int row_blocks = (p.N + 15) / 16;
    // At most four activation rows: four weight rows per wavefront, each read 256 contiguous bytes at a
    // time.  A matrix with too few 16-row blocks to fill the device gets its K split by the plan; a
    // large one (the vocabulary projection: 105 -> 86 us at 128256 x 2048) two wavefronts per row
    // group (one: 92 us, four: 125 us).  A ring of four k steps per wavefront: eight cost 0.1 us per
    // small matrix and 0.3 us on the gate|up pair, sixteen 2 ... 50 us; more bytes in flight per compute
    // unit than the memory system wants slow it down (a ring kept full across rounds, with exact load
    // counts instead of a wait for the whole ring per round, made the vocabulary projection 89 us
    // instead of 77).
    if (p.M <= 4 && p.K % 128 == 0) {
        if (row_blocks < 2 * num_cus) {
            p.sk = linear_skinny_plan(p.N, p.K, 8, num_cus, 4, 128);
        } else {
            p.sk = (p.K / 128 >= 16) ? 2 : 1;
        }
        if (swiglu) {
            return stage ? launch_variant<8, 1, 4, true, true, 4>(p, stream)
                         : launch_variant<8, 1, 4, true, false, 4>(p, stream);
        }
        return stage ? launch_variant<8, 1, 4, false, true, 4>(p, stream)
                     : launch_variant<8, 1, 4, false, false, 4>(p, stream);
    }
    // few row blocks and a long K (the MLP's down projection): sixteen wavefronts share a row block
    const bool big_wg = !swiglu && row_blocks < num_cus && p.K / 32 >= 128;
    p.sk = linear_skinny_plan(p.N, p.K, big_wg ? 16 : 8, num_cus, 16, 32);
    if (swiglu) {
        return stage ? launch_variant<8, 1, 8, true, true>(p, stream) : launch_variant<8, 1, 8, true, false>(p, stream);
    }
    if (big_wg) {
        return stage ? launch_variant<16, 1, 8, false, true>(p, stream)
                     : launch_variant<16, 1, 8, false, false>(p, stream);
    }
    return stage ? launch_variant<8, 1, 8, false, true>(p, stream) : launch_variant<8, 1, 8, false, false>(p, stream);
}

}  // namespace l3
