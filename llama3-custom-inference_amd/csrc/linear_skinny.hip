// y[M, N] = x[M, K] . W[N, K]^T for the few rows of a decode step (M <= 64), bf16 in and out,
// float32 accumulation: the nn.Linear calls of model.py:95,121,134,225 when T == 1.  With so few
// rows the product is a stream over the weight matrix, so the kernel is built like the attention
// kernels: HBM-bound, every weight byte read once, 16-byte loads kept in flight.
//
//   C[16 weight rows x 16 activation rows] += W[16 x 32 k] . x^T[32 k x 16]   (v_mfma_f32_16x16x32_bf16)
//
// A lane of the A operand holds 8 consecutive k of one weight row, which is exactly a 16-byte
// global load: weights go from HBM into operand registers with no staging.  A wavefront owns 16
// weight rows over a slice of K; the `sk` wavefronts that share a row block meet in LDS.  With
// SWIGLU the wavefront streams the same rows of two matrices and writes
// bf16(silu(x.Wg^T)) * bf16(x.Wu^T) with torch's rounding points (model.py:134).
#include "attn_mfma_core.hpp"

namespace l3 {

namespace {

template <int NW, int CBLK, int U, bool SWIGLU>
__global__ void __launch_bounds__(NW * kWaveSize)
linear_skinny_kernel(const LinearParams p) {
    constexpr int ACC = SWIGLU ? 2 : 1;
    __shared__ float s_red[NW][ACC][CBLK][256];

    const int lane = threadIdx.x & (kWaveSize - 1);
    const int wave = threadIdx.x / kWaveSize;
    const int fn = lane & 15;
    const int fg = lane >> 4;

    const int sk = p.sk;                                   // wavefronts per row block (divides NW)
    const int rb = int(blockIdx.x) * (NW / sk) + wave / sk;
    const int kslice = wave % sk;
    const int n0 = rb * 16;
    const int ksteps = p.K / 32;
    const int kpw = (ksteps + sk - 1) / sk;
    const int ks0 = kslice * kpw;
    const int ks1 = min(ksteps, ks0 + kpw);

    const int row = min(n0 + fn, p.N - 1);                 // rows past N are loaded clamped and never stored
    const uint16_t* wp0 = p.w0 + int64_t(row) * p.w_stride + fg * 8;
    const uint16_t* wp1 = SWIGLU ? p.w1 + int64_t(row) * p.w_stride + fg * 8 : nullptr;
    const uint16_t* xp[CBLK];
    bool xvalid[CBLK];
#pragma unroll
    for (int cb = 0; cb < CBLK; ++cb) {
        xvalid[cb] = cb * 16 + fn < p.M;
        xp[cb] = p.x + int64_t(xvalid[cb] ? cb * 16 + fn : 0) * p.x_stride + fg * 8;
    }

    f32x4_t acc[ACC][CBLK];
#pragma unroll
    for (int a = 0; a < ACC; ++a) {
#pragma unroll
        for (int cb = 0; cb < CBLK; ++cb) acc[a][cb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }

    // A ring of U k steps in registers: a slot is refilled for step ks + U as soon as the matrix
    // instructions of step ks have read it, so about U loads per operand stay in flight.
    uint4 rw0[U], rw1[SWIGLU ? U : 1], rx[CBLK][U];
    auto fill = [&](int u, int ks) {
        rw0[u] = load16(wp0 + ks * 32);
        if constexpr (SWIGLU) rw1[u] = load16(wp1 + ks * 32);
#pragma unroll
        for (int cb = 0; cb < CBLK; ++cb) {
            rx[cb][u] = xvalid[cb] ? load16(xp[cb] + ks * 32) : make_uint4(0u, 0u, 0u, 0u);
        }
    };
#pragma unroll
    for (int u = 0; u < U; ++u) {
        if (ks0 + u < ks1) fill(u, ks0 + u);
    }
    for (int ks = ks0; ks < ks1; ks += U) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (ks + u < ks1) {                            // wave-uniform
#pragma unroll
                for (int cb = 0; cb < CBLK; ++cb) {
                    const bf16x8_t xf = __builtin_bit_cast(bf16x8_t, rx[cb][u]);
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
        uint2 w;
        w.x = pack_bf16x2(o[0], o[1]);
        w.y = pack_bf16x2(o[2], o[3]);
        *reinterpret_cast<uint2*>(p.y + int64_t(m) * p.y_stride + n) = w;
    }
}

template <int NW, int CBLK, int U, bool SWIGLU>
int launch_variant(const LinearParams& p, hipStream_t stream) {
    const int row_blocks = (p.N + 15) / 16;
    const int rb_per_wg = NW / p.sk;
    const dim3 grid(unsigned((row_blocks + rb_per_wg - 1) / rb_per_wg));
    hipLaunchKernelGGL((linear_skinny_kernel<NW, CBLK, U, SWIGLU>), grid, dim3(NW * kWaveSize), 0, stream, p);
    return int(hipGetLastError());
}

}  // namespace

// Wavefronts per row block: split K until the launch has about two workgroups per CU, as long
// as every wavefront keeps at least four k steps.
int linear_skinny_plan(int N, int K, int waves_per_wg, int num_cus) {
    const int row_blocks = (N + 15) / 16;
    const int ksteps = K / 32;
    int sk = 1;
    while (sk < waves_per_wg && int64_t(row_blocks) * sk / waves_per_wg < 2 * int64_t(num_cus) &&
           ksteps / (2 * sk) >= 4) {
        sk *= 2;
    }
    return sk;
}

int launch_linear_skinny(LinearParams p, bool swiglu, int num_cus, hipStream_t stream) {
    const bool wide = p.M > 16;
    // few row blocks and a long K (the MLP's down projection): sixteen wavefronts share a row block
    const int row_blocks = (p.N + 15) / 16;
    const bool big_wg = !wide && !swiglu && row_blocks < num_cus && p.K / 32 >= 128;
    p.sk = linear_skinny_plan(p.N, p.K, big_wg ? 16 : 8, num_cus);
    if (swiglu) {
        return wide ? launch_variant<8, 4, 4, true>(p, stream) : launch_variant<8, 1, 8, true>(p, stream);
    }
    if (wide) return launch_variant<8, 4, 8, false>(p, stream);
    return big_wg ? launch_variant<16, 1, 8, false>(p, stream) : launch_variant<8, 1, 16, false>(p, stream);
}

}  // namespace l3
