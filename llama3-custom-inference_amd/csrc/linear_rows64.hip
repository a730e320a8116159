// y[M, N] = x[M, K] . W[N, K]^T for 17 .. 64 activation rows in ONE launch, for matrices whose
// rows alone fill the device: the gate|up pair of the MLP with the SwiGLU product in the epilogue
// (model.py:134 at batch 64), and wide single matrices.
//
// As in the split-K kernel (linear_splitk.hip) the eight wavefronts of a workgroup share the
// activations of a k range through LDS and take their weights straight from global memory into
// operand registers.  Here a workgroup walks over the WHOLE of K in rounds of 512 k: the
// activations of a round (64 rows x 512 k) and the weights of a round sit in one of two LDS
// buffers / register sets while the next round's loads are in flight into the other, so the
// weight stream never stops and no partial products leave the workgroup.
//
//   plain:   8 wavefronts = 8 blocks of 16 weight rows (128 output columns)
//   SwiGLU:  2 blocks of gate rows and the same 2 blocks of up rows (32 output columns), each taken
//            by two wavefronts that split the k range of a round; the halves meet in LDS, then the
//            up sums go to the gate wavefronts, which write bf16(silu(g)) * bf16(u)
//            with the rounding points of the separate torch operators.
#include <type_traits>

#include "attn_mfma_core.hpp"

namespace l3 {

namespace {

constexpr int kR64Waves = 8;
constexpr int kR64Chunk = 128;                   // k per staged activation chunk (4 k steps)
constexpr int kR64Pitch = kR64Chunk * 2 + 16;    // bytes per staged activation row
constexpr int kR64RoundChunks = 4;               // chunks per round (512 k)
constexpr int kR64Stage = 64 * kR64Pitch;        // one chunk of 64 activation rows in LDS

template <bool SWIGLU>
__global__ void __launch_bounds__(kR64Waves * kWaveSize)
linear_rows64_kernel(const LinearParams p) {
    constexpr int NW = kR64Waves, KC = kR64Chunk, PITCH = kR64Pitch, STAGE = kR64Stage, RC = kR64RoundChunks;
    constexpr int CB = 4;                    // 16-row blocks of activations
    constexpr int SPC = KC / 32;             // k steps per chunk
    constexpr int KH = SWIGLU ? 2 : 1;       // wavefronts that split a round's k range
    constexpr int WC = RC / KH;              // chunks of a round one wavefront multiplies
    constexpr int RBW = SWIGLU ? 2 : NW;     // blocks of 16 output columns per workgroup
    __shared__ __align__(16) unsigned char s_x[2 * RC * STAGE];

    const int tid = threadIdx.x;
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid / kWaveSize;
    const int fn = lane & 15;
    const int fg = lane >> 4;

    // SwiGLU: wave = khalf * 4 + mat * 2 + block
    const int khalf = SWIGLU ? wave / 4 : 0;
    const int mat = SWIGLU ? (wave / 2) & 1 : 0;
    const int blk = SWIGLU ? wave & 1 : wave;
    const int n0 = (int(blockIdx.x) * RBW + blk) * 16;
    const int64_t row = min(n0 + fn, p.N - 1);   // rows past N are loaded clamped and never stored
    const uint16_t* wp = (mat ? p.w1 : p.w0) + row * p.w_stride + fg * 8;

    const int total_chunks = p.K / KC;
    const int rounds = (total_chunks + RC - 1) / RC;
    // Workgroups walk over K in the same cyclic order but start at different rounds: weight rows are
    // a power of two apart in memory, and with every workgroup of the device on the same 1 KiB column
    // strip at the same time only a fraction of the memory channels would be busy.  (With a ragged
    // last round everyone starts at round 0, so that the ragged round stays the last.)
    const int first_round = (total_chunks % RC == 0) ? int(blockIdx.x) % rounds : 0;

    // staging roles: 64 rows x 16 pieces of 16 bytes per chunk = 1024 pieces over 512 threads
    const int st_row = tid / 16, st_col = tid % 16;           // rows st_row and st_row + 32
    const bool st_valid0 = st_row < p.M, st_valid1 = st_row + 32 < p.M;
    const uint16_t* xs0 = p.x + int64_t(st_valid0 ? st_row : 0) * p.x_stride + st_col * 8;
    const uint16_t* xs1 = p.x + int64_t(st_valid1 ? st_row + 32 : 0) * p.x_stride + st_col * 8;

    uint4 rwA[WC][SPC], rwB[WC][SPC];
    uint4 xr[RC][2];
    f32x4_t acc[CB];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) acc[cb] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // Loads of round r: the activations first, the weights behind them -- loads return in order, so
    // the activations can be staged while the weights are still on their way, provided the number
    // of weight loads is known at compile time (FULL: a whole round; else a ragged last round, which
    // simply waits for everything).
    auto request = [&](auto full_tag, int r, uint4 (&rw)[WC][SPC]) {
        constexpr bool FULL = decltype(full_tag)::value;
        const int c0 = ((r + first_round) % rounds) * RC;
        const int n = FULL ? RC : total_chunks - c0;
#pragma unroll
        for (int j = 0; j < RC; ++j) {
            if (FULL || j < n) {
                xr[j][0] = st_valid0 ? load16(xs0 + (c0 + j) * KC) : make_uint4(0u, 0u, 0u, 0u);
                xr[j][1] = st_valid1 ? load16(xs1 + (c0 + j) * KC) : make_uint4(0u, 0u, 0u, 0u);
            }
        }
#pragma unroll
        for (int j = 0; j < WC; ++j) {
            const int ch = khalf * WC + j;   // chunk of the round this wavefront multiplies
            if (FULL || ch < n) {
#pragma unroll
                for (int s = 0; s < SPC; ++s) rw[j][s] = load16(wp + ((c0 + ch) * SPC + s) * 32);
            }
        }
    };
    auto stage = [&](auto full_tag, int r, unsigned char* buf) {
        constexpr bool FULL = decltype(full_tag)::value;
        const int n = FULL ? RC : total_chunks - r * RC;
#pragma unroll
        for (int j = 0; j < RC; ++j) {
            if (FULL || j < n) {
                *reinterpret_cast<uint4*>(buf + j * STAGE + st_row * PITCH + st_col * 16) = xr[j][0];
                *reinterpret_cast<uint4*>(buf + j * STAGE + (st_row + 32) * PITCH + st_col * 16) = xr[j][1];
            }
        }
    };
    auto compute = [&](auto full_tag, int r, const unsigned char* buf, const uint4 (&rw)[WC][SPC]) {
        constexpr bool FULL = decltype(full_tag)::value;
        const int n = FULL ? RC : total_chunks - r * RC;
#pragma unroll
        for (int j = 0; j < WC; ++j) {
            const int ch = khalf * WC + j;
            if (FULL || ch < n) {   // wave-uniform
                const unsigned char* rd = buf + ch * STAGE + fn * PITCH + fg * 16;
#pragma unroll
                for (int s = 0; s < SPC; ++s) {
                    const bf16x8_t wf = __builtin_bit_cast(bf16x8_t, rw[j][s]);
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) {
                        const uint4 xv = *reinterpret_cast<const uint4*>(rd + cb * 16 * PITCH + s * 64);
                        acc[cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, __builtin_bit_cast(bf16x8_t, xv),
                                                                          acc[cb], 0, 0, 0);
                    }
                }
            }
        }
    };
    // One round: request round r + 1, multiply round r, stage round r + 1, meet -- as straight-line
    // code per case (NEXT: 0 = no next round, 1 = a whole one, 2 = a ragged one), so that the waits
    // between the three parts count loads instead of draining them.
    auto step_as = [&](auto cur_full, auto next_kind, int r, const unsigned char* buf_cur, unsigned char* buf_nxt,
                       const uint4 (&rw_cur)[WC][SPC], uint4 (&rw_nxt)[WC][SPC]) {
        constexpr int NEXT = decltype(next_kind)::value;
        using next_full = std::integral_constant<bool, NEXT == 1>;
        if constexpr (NEXT != 0) request(next_full{}, r + 1, rw_nxt);
        compute(cur_full, r, buf_cur, rw_cur);
        if constexpr (NEXT != 0) stage(next_full{}, r + 1, buf_nxt);
        __syncthreads();
    };
    auto step = [&](int r, const unsigned char* buf_cur, unsigned char* buf_nxt, const uint4 (&rw_cur)[WC][SPC],
                    uint4 (&rw_nxt)[WC][SPC]) {
        using std::integral_constant;
        const bool has_next = r + 1 < rounds;                   // all three workgroup-uniform
        const bool next_full = (r + 2) * RC <= total_chunks;
        const bool cur_full = (r + 1) * RC <= total_chunks;     // a ragged round is the last one
        if (cur_full && has_next && next_full) {
            step_as(std::true_type{}, integral_constant<int, 1>{}, r, buf_cur, buf_nxt, rw_cur, rw_nxt);
        } else if (cur_full && has_next) {
            step_as(std::true_type{}, integral_constant<int, 2>{}, r, buf_cur, buf_nxt, rw_cur, rw_nxt);
        } else if (cur_full) {
            step_as(std::true_type{}, integral_constant<int, 0>{}, r, buf_cur, buf_nxt, rw_cur, rw_nxt);
        } else {
            step_as(std::false_type{}, integral_constant<int, 0>{}, r, buf_cur, buf_nxt, rw_cur, rw_nxt);
        }
    };

    unsigned char* buf0 = s_x;
    unsigned char* buf1 = s_x + RC * STAGE;
    if (RC <= total_chunks) {
        request(std::true_type{}, 0, rwA);
        stage(std::true_type{}, 0, buf0);
    } else {
        request(std::false_type{}, 0, rwA);
        stage(std::false_type{}, 0, buf0);
    }
    __syncthreads();
    for (int r = 0; r < rounds; r += 2) {
        step(r, buf0, buf1, rwA, rwB);
        if (r + 1 < rounds) step(r + 1, buf1, buf0, rwB, rwA);
    }
    // every step ends with a barrier: the staging area is free for the exchanges below

    float* red = reinterpret_cast<float*>(s_x);
    constexpr int PER_WAVE = CB * 4 * kWaveSize;   // floats one wavefront hands over
    if constexpr (SWIGLU) {
        // Every wavefront stays until the last barrier.  First the second k half hands its sums to the
        // first; then the up wavefronts hand theirs to the gate wavefronts of the same block (through
        // another part of the area, since others may still be reading the first).
        if (khalf == 1) {
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
                for (int r = 0; r < 4; ++r) red[(wave & 3) * PER_WAVE + (cb * 4 + r) * kWaveSize + lane] = acc[cb][r];
            }
        }
        __syncthreads();
        float* xch = red + 4 * PER_WAVE;
        if (khalf == 0) {
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[cb][r] += red[(wave & 3) * PER_WAVE + (cb * 4 + r) * kWaveSize + lane];
            }
            if (mat == 1) {
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) xch[blk * PER_WAVE + (cb * 4 + r) * kWaveSize + lane] = acc[cb][r];
                }
            }
        }
        __syncthreads();
        const int n = n0 + 4 * fg;
        if (khalf == 0 && mat == 0 && n < p.N) {
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
                const int m = cb * 16 + fn;
                if (m >= p.M) continue;
                float o[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float g = __uint_as_float(f32_to_bf16_bits(acc[cb][r]) << 16);
                    const float u = __uint_as_float(
                        f32_to_bf16_bits(xch[blk * PER_WAVE + (cb * 4 + r) * kWaveSize + lane]) << 16);
                    o[r] = silu_rounded(g) * u;
                }
                uint2 w;
                w.x = pack_bf16x2(o[0], o[1]);
                w.y = pack_bf16x2(o[2], o[3]);
                *reinterpret_cast<uint2*>(p.y + int64_t(m) * p.y_stride + n) = w;
            }
        }
    } else {
        // acc[cb][r]: weight row n0 + 4*fg + r against activation row cb*16 + fn
        const int n = n0 + 4 * fg;
        if (n >= p.N) return;
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            const int m = cb * 16 + fn;
            if (m >= p.M) continue;
            float o[4] = {acc[cb][0], acc[cb][1], acc[cb][2], acc[cb][3]};
            if (p.res) {
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
}

}  // namespace

// 17 .. 64 rows in one launch; needs K % 128 == 0 (the caller has checked).
int launch_linear_rows64(const LinearParams& p, bool swiglu, hipStream_t stream) {
    const dim3 block(kR64Waves * kWaveSize);
    if (swiglu) {
        hipLaunchKernelGGL(linear_rows64_kernel<true>, dim3(unsigned((p.N + 31) / 32)), block, 0, stream, p);
    } else {
        hipLaunchKernelGGL(linear_rows64_kernel<false>, dim3(unsigned((p.N + 127) / 128)), block, 0, stream, p);
    }
    return int(hipGetLastError());
}

}  // namespace l3
