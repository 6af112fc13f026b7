// LeakyReLU + per-destination edge softmax (forward and backward) for gfx950.
//
// fp32, memory-bound: e is read, a written, both [E, H] in edge-id order and
// reached through the destination-major CSR's edge-id permutation.  A group of
// lanes (one lane per head) owns one destination row, so the H values of an
// edge are one contiguous read.  The forward pass keeps a running (max, sum)
// pair per lane (online softmax): two sweeps over the row instead of three.
#include "common.hpp"

namespace tango {

__device__ __forceinline__ float leaky(float v, float slope) { return v > 0.0f ? v : v * slope; }

__global__ __launch_bounds__(256) void edge_softmax_fwd_kernel(
    float* __restrict__ a, const float* __restrict__ e, const int64_t* __restrict__ indptr,
    const int64_t* __restrict__ eids, int64_t rows, int H, float slope) {
    const int64_t total = rows * H;
    const int64_t nthr = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += nthr) {
        const int64_t r = i / H;
        const int h = static_cast<int>(i - r * H);
        const int64_t p0 = indptr[r], p1 = indptr[r + 1];
        float mx = -INFINITY, sum = 0.0f;
        for (int64_t p = p0; p < p1; ++p) {
            const int64_t id = eids ? eids[p] : p;
            const float v = leaky(e[id * H + h], slope);
            if (v > mx) {
                sum = sum * __expf(mx - v) + 1.0f;
                mx = v;
            } else {
                sum += __expf(v - mx);
            }
        }
        const float inv = 1.0f / sum;
        for (int64_t p = p0; p < p1; ++p) {
            const int64_t id = eids ? eids[p] : p;
            a[id * H + h] = __expf(leaky(e[id * H + h], slope) - mx) * inv;
        }
    }
}

__global__ __launch_bounds__(256) void edge_softmax_bwd_kernel(
    float* __restrict__ de, const float* __restrict__ a, const float* __restrict__ da,
    const float* __restrict__ e, const int64_t* __restrict__ indptr,
    const int64_t* __restrict__ eids, int64_t rows, int H, float slope) {
    const int64_t total = rows * H;
    const int64_t nthr = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += nthr) {
        const int64_t r = i / H;
        const int h = static_cast<int>(i - r * H);
        const int64_t p0 = indptr[r], p1 = indptr[r + 1];
        float dot = 0.0f;
        for (int64_t p = p0; p < p1; ++p) {
            const int64_t id = eids ? eids[p] : p;
            dot += a[id * H + h] * da[id * H + h];
        }
        for (int64_t p = p0; p < p1; ++p) {
            const int64_t id = eids ? eids[p] : p;
            float g = a[id * H + h] * (da[id * H + h] - dot);
            if (!(e[id * H + h] > 0.0f)) g *= slope;
            de[id * H + h] = g;
        }
    }
}

}  // namespace tango

using namespace tango;

extern "C" {

int tango_edge_softmax_fwd(float* a, const float* e, const int64_t* indptr,
                           const int64_t* edge_ids, int64_t rows, int64_t H, float slope,
                           tango_stream_t stream) {
    if (rows < 0 || H < 0 || (rows > 0 && !indptr) || H >= (1LL << 31)) return TANGO_ERR_INVALID_ARG;
    if (rows * H == 0) return TANGO_OK;
    if (!a || !e) return TANGO_ERR_INVALID_ARG;
    hipLaunchKernelGGL(edge_softmax_fwd_kernel, dim3(grid_for(rows * H, 256, 16)), dim3(256), 0,
                       as_stream(stream), a, e, indptr, edge_ids, rows, static_cast<int>(H), slope);
    return launch_status();
}

int tango_edge_softmax_bwd(float* de, const float* a, const float* da, const float* e,
                           const int64_t* indptr, const int64_t* edge_ids, int64_t rows,
                           int64_t H, float slope, tango_stream_t stream) {
    if (rows < 0 || H < 0 || (rows > 0 && !indptr) || H >= (1LL << 31)) return TANGO_ERR_INVALID_ARG;
    if (rows * H == 0) return TANGO_OK;
    if (!de || !a || !da || !e) return TANGO_ERR_INVALID_ARG;
    hipLaunchKernelGGL(edge_softmax_bwd_kernel, dim3(grid_for(rows * H, 256, 16)), dim3(256), 0,
                       as_stream(stream), de, a, da, e, indptr, edge_ids, rows, static_cast<int>(H),
                       slope);
    return launch_status();
}

}  // extern "C"
