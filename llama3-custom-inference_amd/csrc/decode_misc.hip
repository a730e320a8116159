// Two small decode-step kernels next to the three operators: the SwiGLU elementwise product
// silu(a) * b (model.py:134 evaluates it with two torch kernels) and the greedy argmax over the
// logits row (model.py:371).  In a graph-replayed decode step both are dispatch-bound; one
// launch each instead of two resp. a 40 us single-workgroup library reduction.
#include <algorithm>

#include "l3_device.hpp"
#include "l3_host.hpp"

namespace l3 {

namespace {

constexpr int kMiscThreads = 256;

// y = bf16( bf16(silu(a)) * b ) with silu_rounded of l3_device.hpp.

// blockIdx.y walks over the rows (no index division in the lanes); rows of a and b may be strided
// (the two halves of one fused gate|up projection), y is dense.
__global__ void __launch_bounds__(kMiscThreads)
silu_mul_kernel(const uint16_t* __restrict__ a, const uint16_t* __restrict__ b, uint16_t* __restrict__ y,
                int64_t rows, int64_t vec_per_row, int64_t a_row_stride, int64_t b_row_stride) {
    const int64_t col = int64_t(blockIdx.x) * kMiscThreads + threadIdx.x;
    if (col >= vec_per_row) return;
    for (int64_t row = blockIdx.y; row < rows; row += gridDim.y) {
        float fa[8], fb[8];
        unpack8(load16(a + row * a_row_stride + col * 8), fa);
        unpack8(load16(b + row * b_row_stride + col * 8), fb);
        uint4 o;
        o.x = pack_bf16x2(silu_rounded(fa[0]) * fb[0], silu_rounded(fa[1]) * fb[1]);
        o.y = pack_bf16x2(silu_rounded(fa[2]) * fb[2], silu_rounded(fa[3]) * fb[3]);
        o.z = pack_bf16x2(silu_rounded(fa[4]) * fb[4], silu_rounded(fa[5]) * fb[5]);
        o.w = pack_bf16x2(silu_rounded(fa[6]) * fb[6], silu_rounded(fa[7]) * fb[7]);
        store16(y + (row * vec_per_row + col) * 8, o);
    }
}

__global__ void __launch_bounds__(kMiscThreads)
silu_mul_scalar_kernel(const uint16_t* __restrict__ a, const uint16_t* __restrict__ b, uint16_t* __restrict__ y,
                       int64_t n) {
    const int64_t i = int64_t(blockIdx.x) * kMiscThreads + threadIdx.x;
    if (i >= n) return;
    y[i] = uint16_t(f32_to_bf16_bits(silu_rounded(bf16_to_f32(a[i])) * bf16_to_f32(b[i])));
}

// (value, index) pairs ordered by value, then by smaller index: the first maximum wins, as
// torch.argmax documents.  A NaN ranks above every number (the first NaN wins), which is how
// torch.argmax treats it: a numerical blow-up shows up in the token stream the same way on both paths.
__device__ __forceinline__ void argmax_merge(float& v, int& idx, float ov, int oidx) {
    const bool o_nan = ov != ov, v_nan = v != v;
    if (o_nan ? (!v_nan || oidx < idx) : (!v_nan && (ov > v || (ov == v && oidx < idx)))) {
        v = ov;
        idx = oidx;
    }
}

// Stage 1: each workgroup scans a contiguous chunk of one row (bf16 logits) and writes its
// best (value, index).  Stage 2 (one workgroup per row) merges the chunks.
__global__ void __launch_bounds__(kMiscThreads)
argmax_partial_kernel(const uint16_t* __restrict__ logits, int64_t row_stride, int V, int chunk,
                      float* __restrict__ part_val, int* __restrict__ part_idx) {
    const int row = blockIdx.y;
    const int c0 = blockIdx.x * chunk;
    const int c1 = min(V, c0 + chunk);
    const uint16_t* r = logits + row * row_stride;
    float v = -INFINITY;
    int idx = 0x7fffffff;
    for (int i = c0 + threadIdx.x; i < c1; i += kMiscThreads) argmax_merge(v, idx, bf16_to_f32(r[i]), i);
#pragma unroll
    for (int off = 1; off < kWaveSize; off <<= 1) {
        argmax_merge(v, idx, __shfl_xor(v, off, kWaveSize), __shfl_xor(idx, off, kWaveSize));
    }
    __shared__ float s_v[kMiscThreads / kWaveSize];
    __shared__ int s_i[kMiscThreads / kWaveSize];
    if ((threadIdx.x & (kWaveSize - 1)) == 0) {
        s_v[threadIdx.x / kWaveSize] = v;
        s_i[threadIdx.x / kWaveSize] = idx;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 1; w < kMiscThreads / kWaveSize; ++w) argmax_merge(v, idx, s_v[w], s_i[w]);
        part_val[row * gridDim.x + blockIdx.x] = v;
        part_idx[row * gridDim.x + blockIdx.x] = idx;
    }
}

__global__ void __launch_bounds__(kWaveSize)
argmax_final_kernel(const float* __restrict__ part_val, const int* __restrict__ part_idx, int nparts,
                    int64_t* __restrict__ out) {
    const int row = blockIdx.x;
    float v = -INFINITY;
    int idx = 0x7fffffff;
    for (int i = threadIdx.x; i < nparts; i += kWaveSize) {
        argmax_merge(v, idx, part_val[row * nparts + i], part_idx[row * nparts + i]);
    }
#pragma unroll
    for (int off = 1; off < kWaveSize; off <<= 1) {
        argmax_merge(v, idx, __shfl_xor(v, off, kWaveSize), __shfl_xor(idx, off, kWaveSize));
    }
    if (threadIdx.x == 0) out[row] = (idx == 0x7fffffff) ? 0 : idx;  // V == 0 cannot happen (checked by the caller)
}

// Second argmax stage fused with the bookkeeping generate() does per greedy token
// (model.py:371-378): with next = pos + 1 (clamped to the last column),
//   nxt = text_mask[b, next] ? tokens[b, next] : argmax(logits[b])     (a prompt token is kept)
//   tokens[b, next] = nxt;  tok[b] = nxt (the token fed to the next step)
//   eos[b] |= !text_mask[b, next] && nxt is a stop token
// and, once every row is done, pos += 1 and kv_len += 1.  One workgroup handles all rows (a
// wavefront per four rows in turn), so the two counters are read by everybody before one thread bumps
// them.  In a graph-replayed decode step this stands for the second argmax stage plus about a
// dozen tiny elementwise launches.
constexpr int kGreedyThreads = 1024;
constexpr int kGreedyRowsPerPass = 4;   // rows a wavefront takes per pass, loads of all of them in flight together
__global__ void __launch_bounds__(kGreedyThreads)
greedy_step_kernel(const float* __restrict__ part_val, const int* __restrict__ part_idx, int nparts, int rows,
                   int64_t* __restrict__ tokens, const uint8_t* __restrict__ text_mask, int64_t total_len,
                   int64_t* __restrict__ tok, int* __restrict__ pos, int* __restrict__ kv_len,
                   uint8_t* __restrict__ eos, const int64_t* __restrict__ stop, int n_stop) {
    constexpr int NWAVES = kGreedyThreads / kWaveSize;
    constexpr int RP = kGreedyRowsPerPass;
    const int lane = threadIdx.x & (kWaveSize - 1);
    const int wave = threadIdx.x / kWaveSize;
    const int p0 = *pos;
    const int64_t next = min(int64_t(p0) + 1, total_len - 1);
    for (int base = wave * RP; base < rows; base += NWAVES * RP) {
        // everything that is only read first, for all rows of the pass (independent loads) ...
        float v[RP];
        int idx[RP];
        bool keep[RP];
        int64_t prompt_tok[RP];
#pragma unroll
        for (int j = 0; j < RP; ++j) {
            const int row = min(base + j, rows - 1);
            v[j] = -INFINITY;
            idx[j] = 0x7fffffff;
            for (int i = lane; i < nparts; i += kWaveSize) {
                argmax_merge(v[j], idx[j], part_val[row * nparts + i], part_idx[row * nparts + i]);
            }
            keep[j] = text_mask[row * total_len + next] != 0;
            prompt_tok[j] = tokens[row * total_len + next];
        }
        // ... then the reductions and the stores
#pragma unroll
        for (int j = 0; j < RP; ++j) {
#pragma unroll
            for (int off = 1; off < kWaveSize; off <<= 1) {
                argmax_merge(v[j], idx[j], __shfl_xor(v[j], off, kWaveSize), __shfl_xor(idx[j], off, kWaveSize));
            }
            const int row = base + j;
            if (lane == 0 && row < rows) {
                int64_t nxt = (idx[j] == 0x7fffffff) ? 0 : idx[j];
                if (keep[j]) nxt = prompt_tok[j];
                tokens[row * total_len + next] = nxt;
                tok[row] = nxt;
                bool is_stop = false;
                for (int i = 0; i < n_stop; ++i) is_stop |= (stop[i] == nxt);
                if (!keep[j] && is_stop) eos[row] = 1;
            }
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        *pos = p0 + 1;
        *kv_len = *kv_len + 1;
    }
}

}  // namespace

int launch_greedy_step(const uint16_t* logits, int64_t row_stride, int rows, int V, float* part_val, int* part_idx,
                       int64_t* tokens, const uint8_t* text_mask, int64_t total_len, int64_t* tok, int* pos,
                       int* kv_len, uint8_t* eos, const int64_t* stop, int n_stop, hipStream_t stream) {
    const int parts = argmax_parts(V);
    hipLaunchKernelGGL(argmax_partial_kernel, dim3(unsigned(parts), unsigned(rows)), dim3(kMiscThreads), 0, stream,
                       logits, row_stride, V, kArgmaxChunk, part_val, part_idx);
    hipLaunchKernelGGL(greedy_step_kernel, dim3(1), dim3(kGreedyThreads), 0, stream, part_val, part_idx, parts, rows,
                       tokens, text_mask, total_len, tok, pos, kv_len, eos, stop, n_stop);
    return int(hipGetLastError());
}

int launch_silu_mul_rows(const uint16_t* a, const uint16_t* b, uint16_t* y, int64_t rows, int64_t cols,
                         int64_t a_row_stride, int64_t b_row_stride, hipStream_t stream) {
    const int64_t vpr = cols / 8;
    const dim3 grid(unsigned((vpr + kMiscThreads - 1) / kMiscThreads), unsigned(std::min<int64_t>(rows, 65535)));
    hipLaunchKernelGGL(silu_mul_kernel, grid, dim3(kMiscThreads), 0, stream, a, b, y, rows, vpr, a_row_stride,
                       b_row_stride);
    return int(hipGetLastError());
}

int launch_silu_mul(const uint16_t* a, const uint16_t* b, uint16_t* y, int64_t n, bool vec_ok, hipStream_t stream) {
    if (vec_ok) {
        const int64_t nvec = n / 8;
        hipLaunchKernelGGL(silu_mul_kernel, dim3(unsigned((nvec + kMiscThreads - 1) / kMiscThreads)),
                           dim3(kMiscThreads), 0, stream, a, b, y, int64_t(1), nvec, int64_t(0), int64_t(0));
    } else {
        hipLaunchKernelGGL(silu_mul_scalar_kernel, dim3(unsigned((n + kMiscThreads - 1) / kMiscThreads)),
                           dim3(kMiscThreads), 0, stream, a, b, y, n);
    }
    return int(hipGetLastError());
}

int argmax_parts(int V) { return (V + kArgmaxChunk - 1) / kArgmaxChunk; }

int launch_argmax(const uint16_t* logits, int64_t row_stride, int rows, int V, float* part_val, int* part_idx,
                  int64_t* out, hipStream_t stream) {
    const int parts = argmax_parts(V);
    hipLaunchKernelGGL(argmax_partial_kernel, dim3(unsigned(parts), unsigned(rows)), dim3(kMiscThreads), 0, stream,
                       logits, row_stride, V, kArgmaxChunk, part_val, part_idx);
    hipLaunchKernelGGL(argmax_final_kernel, dim3(unsigned(rows)), dim3(kWaveSize), 0, stream, part_val, part_idx,
                       parts, out);
    return int(hipGetLastError());
}

}  // namespace l3
