// LeakyReLU + per-destination edge softmax (forward and backward) for gfx950.
//
// fp32, memory-bound: e is read, a written, both [E, H] in edge-id order and
// reached through the destination-major CSR's edge-id permutation.  A wavefront
// owns one destination row; its lanes are (edge slot, head) pairs, so the H values
// of an edge are one contiguous read.  The forward pass keeps a running (max, sum)
// pair per lane (online softmax): two sweeps over the row instead of three.
// For H > 64 a thread-per-(row, head) fallback is used.
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
        float mx = -INFINITY;
        double sum = 0.0;  // long rows: keep the running sum's rounding error out of the result
        for (int64_t p = p0; p < p1; ++p) {
            const int64_t id = eids ? eids[p] : p;
            const float v = leaky(e[id * H + h], slope);
            if (v > mx) {
                sum = sum * static_cast<double>(expf(mx - v)) + 1.0;
                mx = v;
            } else {
                sum += static_cast<double>(expf(v - mx));
            }
        }
        const float inv = static_cast<float>(1.0 / sum);
        for (int64_t p = p0; p < p1; ++p) {
            const int64_t id = eids ? eids[p] : p;
            a[id * H + h] = expf(leaky(e[id * H + h], slope) - mx) * inv;
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
        double dsum = 0.0;
        for (int64_t p = p0; p < p1; ++p) {
            const int64_t id = eids ? eids[p] : p;
            dsum += static_cast<double>(a[id * H + h]) * static_cast<double>(da[id * H + h]);
        }
        const float dot = static_cast<float>(dsum);
        for (int64_t p = p0; p < p1; ++p) {
            const int64_t id = eids ? eids[p] : p;
            float g = a[id * H + h] * (da[id * H + h] - dot);
            if (!(e[id * H + h] > 0.0f)) g *= slope;
            de[id * H + h] = g;
        }
    }
}

// Wave-per-row kernels: lane = (edge slot es, head h) with Hp = H rounded up to a
// power of two, so one step of the wavefront covers 64 / Hp edges of the row and
// the per-head reduction is an xor-shuffle over the slot bits.  Used for H <= 64;
// a high-degree destination is walked by 64 lanes instead of one.
// Destinations with more in-edges than this are walked by a 1024-thread workgroup, not one wavefront.
constexpr int64_t kLongRow = 512;
constexpr int64_t kRowsPerLongBlock = 16;  // rows each long-row workgroup inspects

__device__ __forceinline__ void softmax_merge(float& m, double& s, float m2, double s2) {
    const float mx = fmaxf(m, m2);
    // exp(-inf - -inf) would be NaN: a side with no elements contributes nothing
    const double a = (m == -INFINITY) ? 0.0 : s * static_cast<double>(expf(m - mx));
    const double b = (m2 == -INFINITY) ? 0.0 : s2 * static_cast<double>(expf(m2 - mx));
    m = mx;
    s = a + b;
}

__global__ __launch_bounds__(256) void edge_softmax_fwd_wave_kernel(
    float* __restrict__ a, const float* __restrict__ e, const int64_t* __restrict__ indptr,
    const int64_t* __restrict__ eids, int64_t rows, int H, int hp_log2, float slope) {
    const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = lane_id();
    const int h = lane & ((1 << hp_log2) - 1);
    const int es = lane >> hp_log2;
    const int nes = kWave >> hp_log2;
    const int64_t p0 = indptr[row], p1 = indptr[row + 1];
    if (p1 - p0 > kLongRow) return;  // left to the workgroup-per-row kernel
    const bool hok = h < H;
    float mx = -INFINITY;
    double sum = 0.0;
    for (int64_t p = p0 + es; p < p1; p += 4 * nes) {  // four independent edges in flight per lane
        float v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t q = p + u * nes;
            v[u] = -INFINITY;
            if (hok && q < p1) v[u] = leaky(e[(eids ? eids[q] : q) * H + h], slope);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (v[u] != -INFINITY) softmax_merge(mx, sum, v[u], 1.0);
    }
    for (int off = 1 << hp_log2; off < kWave; off <<= 1) {
        const float m2 = __shfl_xor(mx, off, kWave);
        const double s2 = __shfl_xor(sum, off, kWave);
        softmax_merge(mx, sum, m2, s2);
    }
    const float inv = static_cast<float>(1.0 / sum);
    for (int64_t p = p0 + es; p < p1; p += 4 * nes) {
        int64_t id[4];
        float v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t q = p + u * nes;
            id[u] = -1;
            if (hok && q < p1) {
                id[u] = eids ? eids[q] : q;
                v[u] = e[id[u] * H + h];
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (id[u] >= 0) a[id[u] * H + h] = expf(leaky(v[u], slope) - mx) * inv;
    }
}

__global__ __launch_bounds__(256) void edge_softmax_bwd_wave_kernel(
    float* __restrict__ de, const float* __restrict__ a, const float* __restrict__ da,
    const float* __restrict__ e, const int64_t* __restrict__ indptr,
    const int64_t* __restrict__ eids, int64_t rows, int H, int hp_log2, float slope) {
    const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = lane_id();
    const int h = lane & ((1 << hp_log2) - 1);
    const int es = lane >> hp_log2;
    const int nes = kWave >> hp_log2;
    const int64_t p0 = indptr[row], p1 = indptr[row + 1];
    if (p1 - p0 > kLongRow) return;  // left to the workgroup-per-row kernel
    const bool hok = h < H;
    double dsum = 0.0;
    for (int64_t p = p0 + es; p < p1; p += 4 * nes) {
        float x[4], y[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t q = p + u * nes;
            x[u] = y[u] = 0.0f;
            if (hok && q < p1) {
                const int64_t id = eids ? eids[q] : q;
                x[u] = a[id * H + h];
                y[u] = da[id * H + h];
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) dsum += static_cast<double>(x[u]) * static_cast<double>(y[u]);
    }
    for (int off = 1 << hp_log2; off < kWave; off <<= 1) dsum += __shfl_xor(dsum, off, kWave);
    const float dot = static_cast<float>(dsum);
    for (int64_t p = p0 + es; p < p1; p += 4 * nes) {
        int64_t id[4];
        float x[4], y[4], z[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t q = p + u * nes;
            id[u] = -1;
            if (hok && q < p1) {
                id[u] = eids ? eids[q] : q;
                x[u] = a[id[u] * H + h];
                y[u] = da[id[u] * H + h];
                z[u] = e[id[u] * H + h];
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (id[u] >= 0) {
                float g = x[u] * (y[u] - dot);
                if (!(z[u] > 0.0f)) g *= slope;
                de[id[u] * H + h] = g;
            }
    }
}

// Workgroup-per-row kernels for hub destinations (in-degree > kLongRow): 1024 threads, thread =
// (edge slot, head), four independent edges per thread in flight, reduction through LDS.
// Each workgroup inspects every gridDim-th row and walks the long ones among them.
__global__ __launch_bounds__(1024) void edge_softmax_fwd_long_kernel(
    float* __restrict__ a, const float* __restrict__ e, const int64_t* __restrict__ indptr,
    const int64_t* __restrict__ eids, int64_t rows, int H, int hp_log2, float slope) {
    __shared__ float mred[1024];
    __shared__ double sred[1024];
    // strided assignment: neighbouring hub rows go to different workgroups
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const int64_t p0 = indptr[row], p1 = indptr[row + 1];
    if (p1 - p0 <= kLongRow) continue;  // uniform for the workgroup
    __syncthreads();                    // the previous long row's LDS values are consumed
    const int t = threadIdx.x;
    const int hp = 1 << hp_log2;
    const int h = t & (hp - 1);
    const int64_t es = t >> hp_log2, nes = 1024 >> hp_log2;
    const bool hok = h < H;
    float mx = -INFINITY;
    double sum = 0.0;
    for (int64_t p = p0 + es; p < p1; p += 4 * nes) {
        float v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t q = p + u * nes;
            v[u] = -INFINITY;
            if (hok && q < p1) v[u] = leaky(e[(eids ? eids[q] : q) * H + h], slope);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (v[u] != -INFINITY) softmax_merge(mx, sum, v[u], 1.0);
    }
    mred[t] = mx;
    sred[t] = sum;
    __syncthreads();
    for (int off = 512; off >= hp; off >>= 1) {
        if (t < off) {
            float m1 = mred[t];
            double s1 = sred[t];
            softmax_merge(m1, s1, mred[t + off], sred[t + off]);
            mred[t] = m1;
            sred[t] = s1;
        }
        __syncthreads();
    }
    mx = mred[h];
    const float inv = static_cast<float>(1.0 / sred[h]);
    for (int64_t p = p0 + es; p < p1; p += 4 * nes) {
        int64_t id[4];
        float v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t q = p + u * nes;
            id[u] = -1;
            if (hok && q < p1) {
                id[u] = eids ? eids[q] : q;
                v[u] = e[id[u] * H + h];
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (id[u] >= 0) a[id[u] * H + h] = expf(leaky(v[u], slope) - mx) * inv;
    }
    }
}

__global__ __launch_bounds__(1024) void edge_softmax_bwd_long_kernel(
    float* __restrict__ de, const float* __restrict__ a, const float* __restrict__ da,
    const float* __restrict__ e, const int64_t* __restrict__ indptr,
    const int64_t* __restrict__ eids, int64_t rows, int H, int hp_log2, float slope) {
    __shared__ double sred[1024];
    // strided assignment: neighbouring hub rows go to different workgroups
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const int64_t p0 = indptr[row], p1 = indptr[row + 1];
    if (p1 - p0 <= kLongRow) continue;
    __syncthreads();
    const int t = threadIdx.x;
    const int hp = 1 << hp_log2;
    const int h = t & (hp - 1);
    const int64_t es = t >> hp_log2, nes = 1024 >> hp_log2;
    const bool hok = h < H;
    double dsum = 0.0;
    for (int64_t p = p0 + es; p < p1; p += 4 * nes) {
        float x[4], y[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t q = p + u * nes;
            x[u] = y[u] = 0.0f;
            if (hok && q < p1) {
                const int64_t id = eids ? eids[q] : q;
                x[u] = a[id * H + h];
                y[u] = da[id * H + h];
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) dsum += static_cast<double>(x[u]) * static_cast<double>(y[u]);
    }
    sred[t] = dsum;
    __syncthreads();
    for (int off = 512; off >= hp; off >>= 1) {
        if (t < off) sred[t] += sred[t + off];
        __syncthreads();
    }
    const float dot = static_cast<float>(sred[h]);
    for (int64_t p = p0 + es; p < p1; p += 4 * nes) {
        int64_t id[4];
        float x[4], y[4], z[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t q = p + u * nes;
            id[u] = -1;
            if (hok && q < p1) {
                id[u] = eids ? eids[q] : q;
                x[u] = a[id[u] * H + h];
                y[u] = da[id[u] * H + h];
                z[u] = e[id[u] * H + h];
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (id[u] >= 0) {
                float g = x[u] * (y[u] - dot);
                if (!(z[u] > 0.0f)) g *= slope;
                de[id[u] * H + h] = g;
            }
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
    if (H <= 64 && rows <= INT32_MAX) {
        int hp = 0;
        while ((1 << hp) < H) ++hp;
        hipLaunchKernelGGL(edge_softmax_fwd_wave_kernel, dim3(static_cast<unsigned>(ceil_div(rows, 4))),
                           dim3(256), 0, as_stream(stream), a, e, indptr, edge_ids, rows,
                           static_cast<int>(H), hp, slope);
        hipLaunchKernelGGL(edge_softmax_fwd_long_kernel, dim3(static_cast<unsigned>(ceil_div(rows, kRowsPerLongBlock))),
                           dim3(1024), 0, as_stream(stream), a, e, indptr, edge_ids, rows, static_cast<int>(H), hp, slope);
        return launch_status();
    }
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
    if (H <= 64 && rows <= INT32_MAX) {
        int hp = 0;
        while ((1 << hp) < H) ++hp;
        hipLaunchKernelGGL(edge_softmax_bwd_wave_kernel, dim3(static_cast<unsigned>(ceil_div(rows, 4))),
                           dim3(256), 0, as_stream(stream), de, a, da, e, indptr, edge_ids, rows,
                           static_cast<int>(H), hp, slope);
        hipLaunchKernelGGL(edge_softmax_bwd_long_kernel, dim3(static_cast<unsigned>(ceil_div(rows, kRowsPerLongBlock))),
                           dim3(1024), 0, as_stream(stream), de, a, da, e, indptr, edge_ids, rows, static_cast<int>(H), hp, slope);
        return launch_status();
    }
    hipLaunchKernelGGL(edge_softmax_bwd_kernel, dim3(grid_for(rows * H, 256, 16)), dim3(256), 0,
                       as_stream(stream), de, a, da, e, indptr, edge_ids, rows, static_cast<int>(H),
                       slope);
    return launch_status();
}

}  // extern "C"
