// Softmax cross-entropy (mean over rows) with its gradient, one pass over the logits.
//
// Not part of the reference's primitive layer: its drivers call torch's
// F.cross_entropy (evaluation/test_gcn.py:256).  On the benchmark's epoch that
// call is two slow library kernels over a [232965, 41] matrix; this kernel reads
// the logits once, writes (softmax - onehot) / rows, and reduces the loss in a
// fixed order (one partial per workgroup, then one finishing workgroup), so the
// result is deterministic.  HBM-bound: 8 bytes per logit.
#include "common.hpp"

namespace tango {

// A group of `gl` lanes (power of two >= ceil(C / 4), at most 64) owns one row; each lane holds
// up to 4 * T consecutive-strided classes in registers (T = 1 covers C <= 256).
__global__ __launch_bounds__(256) void softmax_xent_kernel(
    const float* __restrict__ logits, int64_t ld, const int64_t* __restrict__ labels, int64_t rows,
    int C, int gl_log2, float* __restrict__ grad, int64_t ldg, float* __restrict__ partial) {
    __shared__ float wsum[4];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int gl = 1 << gl_log2;
    const int rpw = kWave >> gl_log2;  // rows per wavefront
    const int sub = lane >> gl_log2, l = lane & (gl - 1);
    const float inv_rows = 1.0f / static_cast<float>(rows);
    float loss = 0.0f;
    const int64_t step = static_cast<int64_t>(gridDim.x) * 4 * rpw;
    // Two rows per lane group in flight: the loads of both (and their labels) are asked for before either is used, from
    // clamped addresses without a branch around them (a guarded load makes the wave wait at the join behind it).
    constexpr int RU = 2;
    for (int64_t row0 = (static_cast<int64_t>(blockIdx.x) * 4 + wave) * rpw + sub; row0 < rows; row0 += RU * step) {
        float v[RU][4];
        int64_t lab[RU];
#pragma unroll
        for (int u = 0; u < RU; ++u) {
            const int64_t row = row0 + u * step;
            const int64_t rr = row < rows ? row : rows - 1;
            const float* x = logits + rr * ld;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int c = l * 4 + k;
                const float a = x[c < C ? c : C - 1];
                v[u][k] = c < C ? a : -INFINITY;
            }
            lab[u] = labels[rr];
        }
#pragma unroll
        for (int u = 0; u < RU; ++u) {
            const int64_t row = row0 + u * step;
            float mx = fmaxf(fmaxf(v[u][0], v[u][1]), fmaxf(v[u][2], v[u][3]));
            for (int off = 1; off < gl; off <<= 1) mx = fmaxf(mx, __shfl_xor(mx, off, kWave));
            float e[4], s = 0.0f;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                e[k] = (l * 4 + k < C) ? expf(v[u][k] - mx) : 0.0f;
                s += e[k];
            }
            for (int off = 1; off < gl; off <<= 1) s += __shfl_xor(s, off, kWave);
            if (row >= rows) continue;  // after the shuffles: every lane of the wave takes part in them
            const float inv = 1.0f / s;
            float* g = grad + row * ldg;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int c = l * 4 + k;
                if (c < C) {
                    const float p = e[k] * inv;
                    g[c] = (p - (c == lab[u] ? 1.0f : 0.0f)) * inv_rows;
                    if (c == lab[u]) loss += (logf(s) + mx) - v[u][k];  // -log softmax[label]
                }
            }
        }
    }
    // fixed-order reduction: lanes, then the block's four wavefronts
    loss = wave_sum(loss);
    if (lane == 0) wsum[wave] = loss;
    __syncthreads();
    if (threadIdx.x == 0) partial[blockIdx.x] = ((wsum[0] + wsum[1]) + wsum[2]) + wsum[3];
}

__global__ __launch_bounds__(256) void xent_finish_kernel(const float* __restrict__ partial, int n,
                                                          int64_t rows, float* __restrict__ loss) {
    __shared__ float red[256];
    float s = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256) s += partial[i];
    red[threadIdx.x] = s;
    __syncthreads();
    for (int off = 128; off > 0; off >>= 1) {
        if (static_cast<int>(threadIdx.x) < off) red[threadIdx.x] += red[threadIdx.x + off];
        __syncthreads();
    }
    if (threadIdx.x == 0) loss[0] = red[0] / static_cast<float>(rows);
}

static int xent_grid(int64_t rows) {
    const int64_t b = ceil_div(rows, 4);
    return static_cast<int>(b < 1 ? 1 : (b > 2048 ? 2048 : b));
}

}  // namespace tango

using namespace tango;

extern "C" {

size_t tango_softmax_xent_workspace(int64_t rows) { return static_cast<size_t>(xent_grid(rows)) * sizeof(float); }

int tango_softmax_xent_f32(const float* logits, int64_t ld, const int64_t* labels, int64_t rows,
                           int64_t classes, float* loss_out, float* grad_out, int64_t ldg,
                           void* workspace, size_t workspace_bytes, tango_stream_t stream) {
    if (rows <= 0 || classes <= 0 || ld < classes || ldg < classes || !logits || !labels || !loss_out || !grad_out)
        return TANGO_ERR_INVALID_ARG;
    if (classes > 256) return TANGO_ERR_UNSUPPORTED;
    if (!workspace || workspace_bytes < tango_softmax_xent_workspace(rows)) return TANGO_ERR_WORKSPACE;
    hipStream_t s = as_stream(stream);
    int gl_log2 = 0;
    while ((4 << gl_log2) < classes) ++gl_log2;
    const int grid = xent_grid(rows);
    float* partial = static_cast<float*>(workspace);
    hipLaunchKernelGGL(softmax_xent_kernel, dim3(grid), dim3(256), 0, s, logits, ld, labels, rows,
                       static_cast<int>(classes), gl_log2, grad_out, ldg, partial);
    hipLaunchKernelGGL(xent_finish_kernel, dim3(1), dim3(256), 0, s, partial, grid, rows, loss_out);
    return launch_status();
}

}  // extern "C"
