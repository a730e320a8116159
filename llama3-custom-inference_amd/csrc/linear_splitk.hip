// y[M, N] = x[M, K] . W[N, K]^T for 17 .. 64 activation rows, split over K across workgroups.
//
// With this many rows the activation operand of a k step (64 rows x 32 k = 4 KiB) is four times
// the weight operand of a wavefront (16 rows x 32 k), so the activations must be shared: the eight
// wavefronts of a workgroup take eight consecutive blocks of 16 weight rows over the SAME k range,
// the workgroup stages the activations of that range in LDS, and every wavefront reads its B
// operands from there while its weights come straight from global memory into operand registers.
// A workgroup covers at most 512 k (1024 with 64-row groups), so all its loads are requested at once and a single barrier
// separates staging from arithmetic.  K is split across workgroups (which also gives a matrix
// with few rows enough workgroups to fill the device): workgroup (row group g, split s) writes
// the float32 partial products of its k range to part[s][m][n], and whatever elementwise kernel
// follows the linear in the decode step adds the splits up (residual + norm, SwiGLU product,
// rotary embedding), in a fixed order, without atomics.
#include <type_traits>

#include "attn_mfma_core.hpp"

namespace l3 {

namespace {

constexpr int kSplitkWaves = 8;
constexpr int kSplitkChunk = 128;                    // k per staged activation chunk (4 k steps)
constexpr int kSplitkPitch = kSplitkChunk * 2 + 16;  // bytes per staged activation row
constexpr int kSplitkMaxChunks = 4;                  // chunks (of 128 k) whose weights one wavefront holds at most

// KH = 1: the eight wavefronts take eight blocks of 16 weight rows (128 rows) over the workgroup's
// whole k range.  KH = 2: four blocks (64 rows), and the two halves of the wavefronts take the two
// halves of the k range and meet in LDS -- twice the k per workgroup for the same number of
// workgroups, i.e. half as many splits and half the partial-product traffic, for matrices with so
// few rows that 128-row groups would need 16 splits to fill the device.
template <int KH>
__global__ void __launch_bounds__(kSplitkWaves * kWaveSize)
linear_splitk_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, float* __restrict__ part, int M,
                     int N, int K, int64_t x_stride, int64_t w_stride, int chunks_per_split) {
    constexpr int NW = kSplitkWaves, KC = kSplitkChunk, PITCH = kSplitkPitch, CB = 4;
    constexpr int RBW = NW / KH;        // blocks of 16 weight rows per workgroup
    constexpr int STAGE = 64 * PITCH;
    constexpr int MAXC = kSplitkMaxChunks * KH;   // chunks one workgroup covers at most
    constexpr int MAXW = kSplitkMaxChunks;        // chunks whose weights one wavefront holds
    __shared__ __align__(16) unsigned char s_x[MAXC * STAGE];

    const int tid = threadIdx.x;
    const int lane = tid & (kWaveSize - 1);
    const int wave = wave_uniform(tid / kWaveSize);   // scalar: what derives from it is wave-uniform
    const int fn = lane & 15;
    const int fg = lane >> 4;

    const int row_groups = (N + 16 * RBW - 1) / (16 * RBW);
    const int g = int(blockIdx.x) % row_groups;
    const int split = int(blockIdx.x) / row_groups;
    const int n0 = (g * RBW + wave % RBW) * 16;
    const int khalf = wave / RBW;       // which part of the workgroup's k range this wavefront multiplies
    const int total_chunks = K / KC;
    const int c0 = split * chunks_per_split;
    const int c1 = min(total_chunks, c0 + chunks_per_split);

    const int64_t row = min(n0 + fn, N - 1);
    const uint16_t* wp = w + row * w_stride + fg * 8;
    constexpr int SPC = KC / 32;        // k steps per chunk
    const int nch = c1 - c0;            // 1 .. MAXC chunks, all in flight at once
    // chunks of this wavefront: [w0, w0 + nw) of the workgroup's nch
    const int nw = (KH == 1) ? nch : (khalf == 0 ? (nch + 1) / 2 : nch / 2);
    const int w0 = (KH == 1 || khalf == 0) ? 0 : (nch + 1) / 2;

    // Everything this workgroup needs is requested up front: first the activations of the whole k
    // range (registers, then LDS), behind them the weights of every k step into operand registers.
    // Loads return in order, so the activations are staged while the weights are still on their
    // way -- provided the compiler knows how many weight loads follow, hence one copy of the
    // sequence per chunk count.
    // staging roles: 64 rows x 16 chunks of 16 bytes = 1024 pieces over 512 threads
    const int st_row = tid / 16, st_col = tid % 16;           // rows st_row and st_row + 32
    const bool st_valid0 = st_row < M, st_valid1 = st_row + 32 < M;
    const uint16_t* xs0 = x + int64_t(st_valid0 ? st_row : 0) * x_stride + st_col * 8;
    const uint16_t* xs1 = x + int64_t(st_valid1 ? st_row + 32 : 0) * x_stride + st_col * 8;
    uint4 rw[MAXW][SPC];
    uint4 xr[MAXC][2];
    auto request_and_stage = [&](auto count, auto wcount) {
        constexpr int NCH = decltype(count)::value;
        constexpr int NWC = decltype(wcount)::value;
#pragma unroll
        for (int j = 0; j < NCH; ++j) {
            xr[j][0] = st_valid0 ? load16(xs0 + (c0 + j) * KC) : make_uint4(0u, 0u, 0u, 0u);
            xr[j][1] = st_valid1 ? load16(xs1 + (c0 + j) * KC) : make_uint4(0u, 0u, 0u, 0u);
        }
#pragma unroll
        for (int j = 0; j < NWC; ++j) {
#pragma unroll
            for (int s = 0; s < SPC; ++s) rw[j][s] = load16_stream(wp + ((c0 + w0 + j) * SPC + s) * 32);
        }
#pragma unroll
        for (int j = 0; j < NCH; ++j) {
            *reinterpret_cast<uint4*>(s_x + j * STAGE + st_row * PITCH + st_col * 16) = xr[j][0];
            *reinterpret_cast<uint4*>(s_x + j * STAGE + (st_row + 32) * PITCH + st_col * 16) = xr[j][1];
        }
    };
    // one copy of the sequence per (chunks staged by the workgroup, chunks multiplied by this wavefront)
    auto pick = [&](auto count) {
        constexpr int NCH = decltype(count)::value;
        if constexpr (KH == 1) {
            request_and_stage(count, count);
        } else if (khalf == 0) {   // wave-uniform
            request_and_stage(count, std::integral_constant<int, (NCH + 1) / 2>{});
        } else {
            request_and_stage(count, std::integral_constant<int, NCH / 2>{});
        }
    };
    switch (nch) {
        case 1: pick(std::integral_constant<int, 1>{}); break;
        case 2: pick(std::integral_constant<int, 2>{}); break;
        case 3: pick(std::integral_constant<int, 3>{}); break;
        case 4: pick(std::integral_constant<int, 4>{}); break;
        default:
            if constexpr (KH == 2) {
                switch (nch) {
                    case 5: pick(std::integral_constant<int, 5>{}); break;
                    case 6: pick(std::integral_constant<int, 6>{}); break;
                    case 7: pick(std::integral_constant<int, 7>{}); break;
                    case 8: pick(std::integral_constant<int, 8>{}); break;
                    default: break;
                }
            }
            break;
    }
    __syncthreads();

    f32x4_t acc[CB];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) acc[cb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < MAXW; ++j) {
        if (j < nw) {   // wave-uniform
            const unsigned char* rd = s_x + (w0 + j) * STAGE + fn * PITCH + fg * 16;
#pragma unroll
            for (int s = 0; s < SPC; ++s) {
                const bf16x8_t wf = __builtin_bit_cast(bf16x8_t, rw[j][s]);
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) {
                    const uint4 xv = *reinterpret_cast<const uint4*>(rd + cb * 16 * PITCH + s * 64);
                    acc[cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, __builtin_bit_cast(bf16x8_t, xv), acc[cb],
                                                                      0, 0, 0);
                }
            }
        }
    }

    if constexpr (KH == 2) {
        // the second half hands its sums to the first through the staging area (all reads of it are done)
        __syncthreads();
        float* red = reinterpret_cast<float*>(s_x) + (wave % RBW) * (CB * 4 * kWaveSize);
        if (khalf == 1) {
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
                for (int r = 0; r < 4; ++r) red[(cb * 4 + r) * kWaveSize + lane] = acc[cb][r];
            }
        }
        __syncthreads();
        if (khalf == 1) return;
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[cb][r] += red[(cb * 4 + r) * kWaveSize + lane];
        }
    }

    // acc[cb][r]: weight row n0 + 4*fg + r against activation row cb*16 + fn
    const int n = n0 + 4 * fg;
    if (n >= N) return;
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        const int m = cb * 16 + fn;
        if (m < M) {
            *reinterpret_cast<float4*>(part + (int64_t(split) * M + m) * N + n) =
                make_float4(acc[cb][0], acc[cb][1], acc[cb][2], acc[cb][3]);
        }
    }
}

// y[m][n] = bf16(sum over splits of part[s][m][n]) (+ residual, with the rounding of a separate
// bf16 addition): the split-K linear finished on its own, for callers with no elementwise
// operator to fold the sum into.  Eight outputs per lane.
__global__ void __launch_bounds__(256)
linear_splitk_finish_kernel(const float* __restrict__ part, int ksplit, int64_t split_stride,
                            const uint16_t* __restrict__ res, uint16_t* __restrict__ y, int N, int64_t y_stride) {
    const int vi = int(blockIdx.x) * 256 + threadIdx.x;   // blockIdx.y is the activation row
    if (vi >= N / 8) return;
    const int m = blockIdx.y;
    const int n = vi * 8;
    uint4 o = sum_splits_bf16x8(part + int64_t(m) * N + n, ksplit, split_stride);
    if (res) {
        float a[8], b[8];
        unpack8(o, a);
        unpack8(load16(res + int64_t(m) * y_stride + n), b);
        o.x = pack_bf16x2(a[0] + b[0], a[1] + b[1]);
        o.y = pack_bf16x2(a[2] + b[2], a[3] + b[3]);
        o.z = pack_bf16x2(a[4] + b[4], a[5] + b[5]);
        o.w = pack_bf16x2(a[6] + b[6], a[7] + b[7]);
    }
    store16(y + int64_t(m) * y_stride + n, o);
}

}  // namespace

int launch_linear_splitk_finish(const float* part, int ksplit, const uint16_t* res, uint16_t* y, int M, int N,
                                int64_t y_stride, hipStream_t stream) {
    hipLaunchKernelGGL(linear_splitk_finish_kernel, dim3(unsigned((N / 8 + 255) / 256), unsigned(M)), dim3(256), 0,
                       stream, part, ksplit, int64_t(M) * N, res, y, N, y_stride);
    return int(hipGetLastError());
}

// Rows per workgroup: 128, or 64 (with the k range halved inside the workgroup) for a matrix whose
// 128-row groups alone are fewer than a quarter of the compute units.
static bool splitk_half_rows(int N, int num_cus) {
    return (N + 16 * kSplitkWaves - 1) / (16 * kSplitkWaves) < num_cus / 4;
}

// Chunks of 128 k one workgroup covers at most: what its wavefronts can hold in operand registers.
int linear_splitk_max_chunks(int N, int num_cus) {
    return splitk_half_rows(N, num_cus) ? 2 * kSplitkMaxChunks : kSplitkMaxChunks;
}

// Splits of K: a workgroup covers 128, 256, 512 (or with 64-row groups 1024) k; the largest of these
// that still gives about one workgroup per CU (fewer splits mean less partial-product traffic).
int linear_splitk_plan(int N, int K, int num_cus) {
    const int rows_per_wg = splitk_half_rows(N, num_cus) ? 8 * kSplitkWaves : 16 * kSplitkWaves;
    const int row_groups = (N + rows_per_wg - 1) / rows_per_wg;
    const int total_chunks = K / kSplitkChunk;
    int per = linear_splitk_max_chunks(N, num_cus);
    while (per > 1 && int64_t(row_groups) * ((total_chunks + per - 1) / per) < (3 * int64_t(num_cus)) / 4) per /= 2;
    return (total_chunks + per - 1) / per;
}

int launch_linear_splitk(const uint16_t* x, const uint16_t* w, float* part, int M, int N, int K, int64_t x_stride,
                         int64_t w_stride, int ksplit, int num_cus, hipStream_t stream) {
    const int total_chunks = K / kSplitkChunk;
    const int chunks_per_split = (total_chunks + ksplit - 1) / ksplit;   // <= linear_splitk_max_chunks, checked by the caller
    if (splitk_half_rows(N, num_cus)) {
        const int row_groups = (N + 8 * kSplitkWaves - 1) / (8 * kSplitkWaves);
        hipLaunchKernelGGL(linear_splitk_kernel<2>, dim3(unsigned(row_groups * ksplit)),
                           dim3(kSplitkWaves * kWaveSize), 0, stream, x, w, part, M, N, K, x_stride, w_stride,
                           chunks_per_split);
    } else {
        const int row_groups = (N + 16 * kSplitkWaves - 1) / (16 * kSplitkWaves);
        hipLaunchKernelGGL(linear_splitk_kernel<1>, dim3(unsigned(row_groups * ksplit)),
                           dim3(kSplitkWaves * kWaveSize), 0, stream, x, w, part, M, N, K, x_stride, w_stride,
                           chunks_per_split);
    }
    return int(hipGetLastError());
}

}  // namespace l3
