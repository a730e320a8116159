// Fused RMSNorm for gfx950.  Takes the place of custom_rms_norm_kernel
// (custom_kernels.cu:340-367).  Differences by design: each row is read from HBM once
// (16-byte loads kept in registers between the sum of squares and the scaling), the
// product x * inv_rms * w is formed in float32 and rounded to bf16 once (the reference
// rounds inv_rms and both products to bf16, custom_kernels.cu:362-366), and the row is
// reduced with wave64 DPP steps instead of 32-lane shuffles plus a 32-entry shared stage.
#include <algorithm>

#include "l3_device.hpp"
#include "l3_host.hpp"

namespace l3 {

namespace {

constexpr int kRmsThreads = 256;

// One row per group of LANES threads (the launcher uses 256: the whole workgroup on one row,
// for fewer than 1024 rows and for rows too wide for the streaming kernel further down).  A
// thread keeps up to MAXV 16-byte vectors of its row in registers; requires C % 8 == 0 and
// C / 8 <= LANES * MAXV.
//
// ADD = true fuses the residual addition that precedes every RMSNorm but the first in a
// transformer block (model.py:147-148: x = x + attn(...); ...ln_2(x)): s = bf16(x + res) is
// written to `sum_out` and the norm is taken of the ROUNDED s, so the pair of outputs is
// bit-identical to torch's bf16 add followed by the unfused kernel.
template <int LANES, int MAXV, bool ADD>
__global__ void __launch_bounds__(kRmsThreads)
rms_norm_rows_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ res,
                     const uint16_t* __restrict__ w, uint16_t* __restrict__ sum_out, uint16_t* __restrict__ y,
                     int64_t rows, int C, float eps) {
    constexpr int ROWS_PER_BLOCK = kRmsThreads / LANES;
    const int tid = threadIdx.x;
    const int sub = tid / LANES;
    const int t = tid % LANES;
    const int64_t row = int64_t(blockIdx.x) * ROWS_PER_BLOCK + sub;
    const bool live = row < rows;
    const int nvec = C / 8;
    const uint16_t* xr = x + (live ? row : 0) * int64_t(C);

    uint4 xv[MAXV];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
        const int vi = t + j * LANES;
        if (vi < nvec) {
            xv[j] = load16(xr + vi * 8);
            float f[8];
            unpack8(xv[j], f);
            if constexpr (ADD) {
                float r[8];
                unpack8(load16(res + (live ? row : 0) * int64_t(C) + vi * 8), r);
                xv[j].x = pack_bf16x2(f[0] + r[0], f[1] + r[1]);
                xv[j].y = pack_bf16x2(f[2] + r[2], f[3] + r[3]);
                xv[j].z = pack_bf16x2(f[4] + r[4], f[5] + r[5]);
                xv[j].w = pack_bf16x2(f[6] + r[6], f[7] + r[7]);
                if (live) store16(sum_out + row * int64_t(C) + vi * 8, xv[j]);
                unpack8(xv[j], f);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) ss = fmaf(f[i], f[i], ss);
        }
    }
    ss = wave_sum(ss);
    if constexpr (LANES > kWaveSize) {
        __shared__ float s_part[kRmsThreads / kWaveSize];
        if ((tid & (kWaveSize - 1)) == 0) s_part[tid / kWaveSize] = ss;
        __syncthreads();
        ss = (s_part[0] + s_part[1]) + (s_part[2] + s_part[3]);
    }
    const float inv = rsqrtf(ss / float(C) + eps);
    if (!live) return;

    uint16_t* yr = y + row * int64_t(C);
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
        const int vi = t + j * LANES;
        if (vi < nvec) {
            float f[8], g[8];
            unpack8(xv[j], f);
            unpack8(load16(w + vi * 8), g);
            uint4 o;
            o.x = pack_bf16x2(f[0] * inv * g[0], f[1] * inv * g[1]);
            o.y = pack_bf16x2(f[2] * inv * g[2], f[3] * inv * g[3]);
            o.z = pack_bf16x2(f[4] * inv * g[4], f[5] * inv * g[5]);
            o.w = pack_bf16x2(f[6] * inv * g[6], f[7] * inv * g[7]);
            store16(yr + vi * 8, o);
        }
    }
}

// Thousands of rows (prefill): a wavefront walks over rows row, row + stride, ... and requests
// the next row before it reduces the current one, so that the device reads and writes at the same
// time instead of reading every row first and writing every row afterwards.  The norm weights stay
// in registers.  C % 8 == 0 and C / 8 <= 64 * MAXV.  ADD as in the kernel above.
template <int MAXV, bool ADD>
__global__ void __launch_bounds__(kRmsThreads)
rms_norm_stream_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ res,
                       const uint16_t* __restrict__ w, uint16_t* __restrict__ sum_out, uint16_t* __restrict__ y,
                       int64_t rows, int C, float eps) {
    const int lane = threadIdx.x & (kWaveSize - 1);
    const int64_t stride = int64_t(gridDim.x) * (kRmsThreads / kWaveSize);
    int64_t row = int64_t(blockIdx.x) * (kRmsThreads / kWaveSize) + threadIdx.x / kWaveSize;
    if (row >= rows) return;
    const int nvec = C / 8;
    uint4 wv[MAXV], cur[MAXV], nxt[MAXV], rcur[ADD ? MAXV : 1], rnxt[ADD ? MAXV : 1];
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
        const int vi = lane + j * kWaveSize;
        if (vi < nvec) {
            cur[j] = load16_stream(x + row * int64_t(C) + vi * 8);
            if constexpr (ADD) rcur[j] = load16_stream(res + row * int64_t(C) + vi * 8);
            wv[j] = load16(w + vi * 8);
        }
    }
    const float inv_c = 1.0f / float(C);
    while (true) {
        const int64_t nrow = row + stride;
        const bool has_next = nrow < rows;   // wave-uniform
        if (has_next) {
#pragma unroll
            for (int j = 0; j < MAXV; ++j) {
                const int vi = lane + j * kWaveSize;
                if (vi < nvec) {
                    nxt[j] = load16_stream(x + nrow * int64_t(C) + vi * 8);
                    if constexpr (ADD) rnxt[j] = load16_stream(res + nrow * int64_t(C) + vi * 8);
                }
            }
        }
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < MAXV; ++j) {
            const int vi = lane + j * kWaveSize;
            if (vi < nvec) {
                float f[8];
                unpack8(cur[j], f);
                if constexpr (ADD) {
                    // s = bf16(x + res) goes out, and the norm is taken of the rounded s
                    float r[8];
                    unpack8(rcur[j], r);
                    cur[j].x = pack_bf16x2(f[0] + r[0], f[1] + r[1]);
                    cur[j].y = pack_bf16x2(f[2] + r[2], f[3] + r[3]);
                    cur[j].z = pack_bf16x2(f[4] + r[4], f[5] + r[5]);
                    cur[j].w = pack_bf16x2(f[6] + r[6], f[7] + r[7]);
                    store16(sum_out + row * int64_t(C) + vi * 8, cur[j]);
                    unpack8(cur[j], f);
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) ss = fmaf(f[i], f[i], ss);
            }
        }
        ss = wave_sum(ss);
        const float inv = rsqrtf(ss * inv_c + eps);
#pragma unroll
        for (int j = 0; j < MAXV; ++j) {
            const int vi = lane + j * kWaveSize;
            if (vi < nvec) {
                float f[8], g[8];
                unpack8(cur[j], f);
                unpack8(wv[j], g);
                uint4 o;
                o.x = pack_bf16x2(f[0] * inv * g[0], f[1] * inv * g[1]);
                o.y = pack_bf16x2(f[2] * inv * g[2], f[3] * inv * g[3]);
                o.z = pack_bf16x2(f[4] * inv * g[4], f[5] * inv * g[5]);
                o.w = pack_bf16x2(f[6] * inv * g[6], f[7] * inv * g[7]);
                store16(y + row * int64_t(C) + vi * 8, o);
            }
        }
        if (!has_next) break;
        for (int j = 0; j < MAXV; ++j) {
            cur[j] = nxt[j];
            if constexpr (ADD) rcur[j] = rnxt[j];
        }
        row = nrow;
    }
}

// Any C, any alignment: one workgroup per row, 2-byte accesses, the row is read twice.
template <bool ADD>
__global__ void __launch_bounds__(kRmsThreads)
rms_norm_generic_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ res,
                        const uint16_t* __restrict__ w, uint16_t* __restrict__ sum_out, uint16_t* __restrict__ y,
                        int C, float eps) {
    const int tid = threadIdx.x;
    const uint16_t* xr = x + int64_t(blockIdx.x) * C;
    uint16_t* yr = y + int64_t(blockIdx.x) * C;
    float ss = 0.f;
    if constexpr (ADD) {
        // first pass writes the rounded sum; the passes below then read it back as the input row
        const uint16_t* rr = res + int64_t(blockIdx.x) * C;
        uint16_t* sr = sum_out + int64_t(blockIdx.x) * C;
        for (int i = tid; i < C; i += kRmsThreads) {
            sr[i] = uint16_t(f32_to_bf16_bits(bf16_to_f32(xr[i]) + bf16_to_f32(rr[i])));
        }
        xr = sr;  // each thread re-reads only what it wrote itself
    }
    for (int i = tid; i < C; i += kRmsThreads) {
        const float f = bf16_to_f32(xr[i]);
        ss = fmaf(f, f, ss);
    }
    ss = wave_sum(ss);
    __shared__ float s_part[kRmsThreads / kWaveSize];
    if ((tid & (kWaveSize - 1)) == 0) s_part[tid / kWaveSize] = ss;
    __syncthreads();
    ss = (s_part[0] + s_part[1]) + (s_part[2] + s_part[3]);
    const float inv = rsqrtf(ss / float(C) + eps);
    for (int i = tid; i < C; i += kRmsThreads) {
        yr[i] = uint16_t(f32_to_bf16_bits(bf16_to_f32(xr[i]) * inv * bf16_to_f32(w[i])));
    }
}

// add_rms_norm whose residual operand is the output of a split-K linear that has not been added
// up yet: r = bf16(sum over splits of part[s][row][:]) first (what the unsplit linear would have
// written), then exactly the ADD path above.  One workgroup per row (decode steps have few rows);
// C % 8 == 0 and C / 8 <= 256 * 4.
__global__ void __launch_bounds__(kRmsThreads)
add_rms_norm_partials_kernel(const uint16_t* __restrict__ x, const float* __restrict__ part, int ksplit,
                             int64_t split_stride, const uint16_t* __restrict__ w, uint16_t* __restrict__ sum_out,
                             uint16_t* __restrict__ y, int C, float eps) {
    constexpr int MAXV = 4;
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    const int nvec = C / 8;
    uint4 xv[MAXV];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
        const int vi = tid + j * kRmsThreads;
        if (vi < nvec) {
            float f[8], r[8];
            unpack8(load16(x + row * C + vi * 8), f);
            unpack8(sum_splits_bf16x8(part + row * C + vi * 8, ksplit, split_stride), r);
            xv[j].x = pack_bf16x2(f[0] + r[0], f[1] + r[1]);
            xv[j].y = pack_bf16x2(f[2] + r[2], f[3] + r[3]);
            xv[j].z = pack_bf16x2(f[4] + r[4], f[5] + r[5]);
            xv[j].w = pack_bf16x2(f[6] + r[6], f[7] + r[7]);
            store16(sum_out + row * C + vi * 8, xv[j]);
            unpack8(xv[j], f);
#pragma unroll
            for (int i = 0; i < 8; ++i) ss = fmaf(f[i], f[i], ss);
        }
    }
    ss = wave_sum(ss);
    __shared__ float s_part[kRmsThreads / kWaveSize];
    if ((tid & (kWaveSize - 1)) == 0) s_part[tid / kWaveSize] = ss;
    __syncthreads();
    ss = (s_part[0] + s_part[1]) + (s_part[2] + s_part[3]);
    const float inv = rsqrtf(ss / float(C) + eps);
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
        const int vi = tid + j * kRmsThreads;
        if (vi < nvec) {
            float f[8], g[8];
            unpack8(xv[j], f);
            unpack8(load16(w + vi * 8), g);
            uint4 o;
            o.x = pack_bf16x2(f[0] * inv * g[0], f[1] * inv * g[1]);
            o.y = pack_bf16x2(f[2] * inv * g[2], f[3] * inv * g[3]);
            o.z = pack_bf16x2(f[4] * inv * g[4], f[5] * inv * g[5]);
            o.w = pack_bf16x2(f[6] * inv * g[6], f[7] * inv * g[7]);
            store16(y + row * C + vi * 8, o);
        }
    }
}

}  // namespace

int launch_add_rms_norm_partials(const uint16_t* x, const float* part, int ksplit, int64_t split_stride,
                                 const uint16_t* w, uint16_t* sum_out, uint16_t* y, int rows, int C, float eps,
                                 hipStream_t stream) {
    hipLaunchKernelGGL(add_rms_norm_partials_kernel, dim3(unsigned(rows)), dim3(kRmsThreads), 0, stream, x, part,
                       ksplit, split_stride, w, sum_out, y, C, eps);
    return int(hipGetLastError());
}

namespace {

template <bool ADD>
int launch_rms_norm_impl(const uint16_t* x, const uint16_t* res, const uint16_t* w, uint16_t* sum_out, uint16_t* y,
                         int64_t rows, int C, float eps, bool vec_ok, hipStream_t stream) {
    const int nvec = C / 8;
    const dim3 block(kRmsThreads);
    if (vec_ok && rows >= 1024 && nvec <= 64 * 8) {
        // a thousand rows or more: every wavefront takes several, reads overlapping writes
        const int64_t waves = std::min<int64_t>(rows / 2, int64_t(current_device_cus()) * 8);
        const dim3 grid(unsigned((waves + 3) / 4));
        if (nvec <= 64 * 4) {
            hipLaunchKernelGGL((rms_norm_stream_kernel<4, ADD>), grid, block, 0, stream, x, res, w, sum_out, y, rows, C,
                               eps);
        } else {
            hipLaunchKernelGGL((rms_norm_stream_kernel<8, ADD>), grid, block, 0, stream, x, res, w, sum_out, y, rows,
                               C, eps);
        }
    } else if (vec_ok && nvec <= 256 * 4) {
        // few rows (decode): the whole workgroup on one row keeps the latency short
        const dim3 grid{unsigned(rows)};
        if (nvec <= 256) {
            hipLaunchKernelGGL((rms_norm_rows_kernel<256, 1, ADD>), grid, block, 0, stream, x, res, w, sum_out, y,
                               rows, C, eps);
        } else if (nvec <= 512) {
            hipLaunchKernelGGL((rms_norm_rows_kernel<256, 2, ADD>), grid, block, 0, stream, x, res, w, sum_out, y,
                               rows, C, eps);
        } else {
            hipLaunchKernelGGL((rms_norm_rows_kernel<256, 4, ADD>), grid, block, 0, stream, x, res, w, sum_out, y,
                               rows, C, eps);
        }
    } else {
        hipLaunchKernelGGL((rms_norm_generic_kernel<ADD>), dim3(unsigned(rows)), block, 0, stream, x, res, w, sum_out,
                           y, C, eps);
    }
    return int(hipGetLastError());
}

}  // namespace

int launch_rms_norm(const uint16_t* x, const uint16_t* w, uint16_t* y, int64_t rows, int C, float eps,
                    bool vec_ok, hipStream_t stream) {
    return launch_rms_norm_impl<false>(x, nullptr, w, nullptr, y, rows, C, eps, vec_ok, stream);
}

int launch_add_rms_norm(const uint16_t* x, const uint16_t* res, const uint16_t* w, uint16_t* sum_out, uint16_t* y,
                        int64_t rows, int C, float eps, bool vec_ok, hipStream_t stream) {
    return launch_rms_norm_impl<true>(x, res, w, sum_out, y, rows, C, eps, vec_ok, stream);
}

}  // namespace l3
