// LeakyReLU + per-destination edge softmax (forward and backward) for gfx950.
//
// fp32, memory-bound: e is read, a written, both [E, H] in edge-id order and
// reached through the destination-major CSR's edge-id permutation.  Threads are
// (edge slot, head) pairs, so the H values of an edge are one contiguous read, and
// a destination is owned by a thread group sized to its in-degree (see the tiers
// below).  The forward pass keeps a running (max, sum) pair per thread (online
// softmax): two sweeps over a row instead of three, one for rows held in registers.
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

// Three tiers by in-degree, for H <= 64 (Hp = H rounded up to a power of two):
//   short  (<= kShortRow edges): a thread owns one (row, head) and keeps the row's values in
//          registers, one sweep over memory; a wavefront covers 64 / H rows, which is what
//          keeps enough bytes in flight when most destinations have a handful of in-edges;
//   medium (<= kMediumValues / Hp edges): a wavefront owns the row, lane = (edge slot, head),
//          four edges per lane in flight, reduction by xor-shuffles over the slot bits;
//   long   : a 1024-thread workgroup owns the row (a hub destination must not be walked by one
//          wavefront while the rest of the chip idles).
// The medium and long kernels find their rows themselves: a wavefront / workgroup inspects a
// strided set of rows at once (hubs with neighbouring ids spread out over the launch) and walks
// the ones of its tier; no list of rows is built in global memory.
constexpr int kShortRow = 16;
constexpr int kMediumValues = 2048;
// A hub: a destination with more than kHubValues / Hp in-edges.  One workgroup walking it alone
// would outlast the whole rest of the launch, so (when the caller passes a workspace) the long
// tier only records such rows and two further launches cut each into kHubChunks chunks: partial
// (max, sum) per chunk and head, then every chunk combines its row's partials and writes its part.
constexpr int kHubValues = 32768;
constexpr int kHubChunks = 32;
constexpr int kMaxHubs = 256;     // hubs beyond this stay with the long tier's single workgroup
constexpr int kHubGridY = 64;     // workgroup rows of the hub launches; each walks hubs y, y + 64, ...

// Workspace: [0] hub count (int), then kMaxHubs x (p0, p1) int64, then the partials
// [kMaxHubs][kHubChunks][Hp] of {float max; double sum} (backward: the double only).
struct HubPartial {
    double sum;
    float mx;
    float pad;
};
__host__ __device__ inline size_t hub_list_offset() { return 256; }
__host__ __device__ inline size_t hub_partial_offset() { return 256 + sizeof(int64_t) * 2 * kMaxHubs; }

__device__ __forceinline__ void softmax_merge(float& m, double& s, float m2, double s2) {
    const float mx = fmaxf(m, m2);
    // exp(-inf - -inf) would be NaN: a side with no elements contributes nothing
    const double a = (m == -INFINITY) ? 0.0 : s * static_cast<double>(expf(m - mx));
    const double b = (m2 == -INFINITY) ? 0.0 : s2 * static_cast<double>(expf(m2 - mx));
    m = mx;
    s = a + b;
}

// 0 = short, 1 = medium, 2 = long
__device__ __forceinline__ int row_tier(int64_t deg, int hp_log2) {
    if (deg <= kShortRow) return 0;
    return deg <= (kMediumValues >> hp_log2) ? 1 : 2;
}

__global__ __launch_bounds__(256) void edge_softmax_fwd_short_kernel(
    float* __restrict__ a, const float* __restrict__ e, const int64_t* __restrict__ indptr,
    const int64_t* __restrict__ eids, int64_t rows, int H, float slope) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= rows * H) return;
    const int64_t r = i / H;
    const int h = static_cast<int>(i - r * H);
    const int64_t p0 = indptr[r];
    const int64_t deg = indptr[r + 1] - p0;
    if (deg > kShortRow || deg == 0) return;
    int64_t id[kShortRow];
    float v[kShortRow];
#pragma unroll
    for (int u = 0; u < kShortRow; ++u) {
        v[u] = -INFINITY;
        id[u] = 0;
        if (u < deg) {
            id[u] = (eids ? eids[p0 + u] : p0 + u) * H + h;
            v[u] = leaky(e[id[u]], slope);
        }
    }
    float mx = v[0];
#pragma unroll
    for (int u = 1; u < kShortRow; ++u) mx = fmaxf(mx, v[u]);
    double sum = 0.0;
#pragma unroll
    for (int u = 0; u < kShortRow; ++u) {
        v[u] = u < deg ? expf(v[u] - mx) : 0.0f;
        sum += static_cast<double>(v[u]);
    }
    const float inv = static_cast<float>(1.0 / sum);
#pragma unroll
    for (int u = 0; u < kShortRow; ++u)
        if (u < deg) a[id[u]] = v[u] * inv;
}

__global__ __launch_bounds__(256) void edge_softmax_bwd_short_kernel(
    float* __restrict__ de, const float* __restrict__ a, const float* __restrict__ da,
    const float* __restrict__ e, const int64_t* __restrict__ indptr,
    const int64_t* __restrict__ eids, int64_t rows, int H, float slope) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= rows * H) return;
    const int64_t r = i / H;
    const int h = static_cast<int>(i - r * H);
    const int64_t p0 = indptr[r];
    const int64_t deg = indptr[r + 1] - p0;
    if (deg > kShortRow || deg == 0) return;
    int64_t id[kShortRow];
    float x[kShortRow], y[kShortRow], z[kShortRow];
    double dsum = 0.0;
#pragma unroll
    for (int u = 0; u < kShortRow; ++u) {
        x[u] = y[u] = z[u] = 0.0f;
        id[u] = 0;
        if (u < deg) {
            id[u] = (eids ? eids[p0 + u] : p0 + u) * H + h;
            x[u] = a[id[u]];
            y[u] = da[id[u]];
            z[u] = e[id[u]];
        }
    }
#pragma unroll
    for (int u = 0; u < kShortRow; ++u) dsum += static_cast<double>(x[u]) * static_cast<double>(y[u]);
    const float dot = static_cast<float>(dsum);
#pragma unroll
    for (int u = 0; u < kShortRow; ++u)
        if (u < deg) {
            float g = x[u] * (y[u] - dot);
            if (!(z[u] > 0.0f)) g *= slope;
            de[id[u]] = g;
        }
}

// `nthreads` threads (a wavefront or a workgroup) walk slots [p0, p1) of one row: thread t is
// (edge slot t >> hp_log2, head t & (Hp - 1)).  Returns this thread's running (max, sum).
template <int U>
__device__ __forceinline__ void fwd_partial(const float* __restrict__ e, const int64_t* __restrict__ eids,
                                            int64_t p0, int64_t p1, int t, int nthreads, int H, int hp_log2,
                                            float slope, float& mx, double& sum) {
    const int h = t & ((1 << hp_log2) - 1);
    const int64_t es = t >> hp_log2, nes = nthreads >> hp_log2;
    const bool hok = h < H;
    mx = -INFINITY;
    sum = 0.0;
    for (int64_t p = p0 + es; p < p1; p += U * nes) {  // U independent edges in flight per thread
        float v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t q = p + u * nes;
            v[u] = -INFINITY;
            if (hok && q < p1) v[u] = leaky(e[(eids ? eids[q] : q) * H + h], slope);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (v[u] == -INFINITY) continue;
            if (v[u] > mx) {  // one exp per element either way
                sum = sum * static_cast<double>(expf(mx - v[u])) + 1.0;  // exp(-inf) = 0 for the first element
                mx = v[u];
            } else {
                sum += static_cast<double>(expf(v[u] - mx));
            }
        }
    }
}

template <int U>
__device__ __forceinline__ void fwd_write(float* __restrict__ a, const float* __restrict__ e,
                                          const int64_t* __restrict__ eids, int64_t p0, int64_t p1, int t,
                                          int nthreads, int H, int hp_log2, float slope, float mx, float inv) {
    const int h = t & ((1 << hp_log2) - 1);
    const int64_t es = t >> hp_log2, nes = nthreads >> hp_log2;
    const bool hok = h < H;
    for (int64_t p = p0 + es; p < p1; p += U * nes) {
        int64_t id[U];
        float v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t q = p + u * nes;
            id[u] = -1;
            if (hok && q < p1) {
                id[u] = (eids ? eids[q] : q) * H + h;
                v[u] = e[id[u]];
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (id[u] >= 0) a[id[u]] = expf(leaky(v[u], slope) - mx) * inv;
    }
}

template <int U>
__device__ __forceinline__ double bwd_partial(const float* __restrict__ a, const float* __restrict__ da,
                                              const int64_t* __restrict__ eids, int64_t p0, int64_t p1, int t,
                                              int nthreads, int H, int hp_log2) {
    const int h = t & ((1 << hp_log2) - 1);
    const int64_t es = t >> hp_log2, nes = nthreads >> hp_log2;
    const bool hok = h < H;
    double dsum = 0.0;
    for (int64_t p = p0 + es; p < p1; p += U * nes) {
        float x[U], y[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t q = p + u * nes;
            x[u] = y[u] = 0.0f;
            if (hok && q < p1) {
                const int64_t id = (eids ? eids[q] : q) * H + h;
                x[u] = a[id];
                y[u] = da[id];
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) dsum += static_cast<double>(x[u]) * static_cast<double>(y[u]);
    }
    return dsum;
}

template <int U>
__device__ __forceinline__ void bwd_write(float* __restrict__ de, const float* __restrict__ a,
                                          const float* __restrict__ da, const float* __restrict__ e,
                                          const int64_t* __restrict__ eids, int64_t p0, int64_t p1, int t,
                                          int nthreads, int H, int hp_log2, float slope, float dot) {
    const int h = t & ((1 << hp_log2) - 1);
    const int64_t es = t >> hp_log2, nes = nthreads >> hp_log2;
    const bool hok = h < H;
    for (int64_t p = p0 + es; p < p1; p += U * nes) {
        int64_t id[U];
        float x[U], y[U], z[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t q = p + u * nes;
            id[u] = -1;
            if (hok && q < p1) {
                id[u] = (eids ? eids[q] : q) * H + h;
                x[u] = a[id[u]];
                y[u] = da[id[u]];
                z[u] = e[id[u]];
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (id[u] >= 0) {
                float g = x[u] * (y[u] - dot);
                if (!(z[u] > 0.0f)) g *= slope;
                de[id[u]] = g;
            }
    }
}

// Medium rows.  Wavefront w of the launch inspects rows w, w + W, w + 2W, ... (kRowsPerWave of
// them, W = number of wavefronts launched) and walks the medium ones in turn.
constexpr int kRowsPerWave = 8;
template <bool FWD>
__global__ __launch_bounds__(256) void edge_softmax_medium_kernel(
    float* __restrict__ out, const float* __restrict__ a, const float* __restrict__ da,
    const float* __restrict__ e, const int64_t* __restrict__ indptr, const int64_t* __restrict__ eids,
    int64_t rows, int H, int hp_log2, float slope) {
    const int lane = lane_id();
    const int64_t nwaves = static_cast<int64_t>(gridDim.x) * 4;
    const int64_t w = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    const int64_t mine = w + static_cast<int64_t>(lane) * nwaves;
    int64_t q0 = 0, q1 = 0;
    if (lane < kRowsPerWave && mine < rows) {
        q0 = indptr[mine];
        q1 = indptr[mine + 1];
    }
    uint64_t todo = __ballot(row_tier(q1 - q0, hp_log2) == 1);
    while (todo) {
        const int l = __builtin_ctzll(todo);
        todo &= todo - 1;
        const int64_t p0 = __shfl(q0, l, kWave), p1 = __shfl(q1, l, kWave);
        if (FWD) {
            float mx;
            double sum;
            fwd_partial<8>(e, eids, p0, p1, lane, kWave, H, hp_log2, slope, mx, sum);
            for (int off = 1 << hp_log2; off < kWave; off <<= 1) {
                const float m2 = __shfl_xor(mx, off, kWave);
                const double s2 = __shfl_xor(sum, off, kWave);
                softmax_merge(mx, sum, m2, s2);
            }
            fwd_write<8>(out, e, eids, p0, p1, lane, kWave, H, hp_log2, slope, mx, static_cast<float>(1.0 / sum));
        } else {
            double dsum = bwd_partial<8>(a, da, eids, p0, p1, lane, kWave, H, hp_log2);
            for (int off = 1 << hp_log2; off < kWave; off <<= 1) dsum += __shfl_xor(dsum, off, kWave);
            bwd_write<8>(out, a, da, e, eids, p0, p1, lane, kWave, H, hp_log2, slope, static_cast<float>(dsum));
        }
    }
}

// Long rows.  A fixed number of 1024-thread workgroups (G = gridDim.x) share the rows: thread t
// of workgroup b inspects row b + G * t (then b + G * (1024 + t), ...), the long ones are
// collected in LDS and walked in turn by all sixteen wavefronts: shuffles inside a wavefront,
// then one exchange of the sixteen partial results through LDS.
constexpr int kLongGrid = 512;

template <bool FWD>
__global__ __launch_bounds__(1024) void edge_softmax_long_kernel(
    float* __restrict__ out, const float* __restrict__ a, const float* __restrict__ da,
    const float* __restrict__ e, const int64_t* __restrict__ indptr, const int64_t* __restrict__ eids,
    int64_t rows, int H, int hp_log2, float slope, void* __restrict__ hub_ws) {
    __shared__ float mred[16][64];
    __shared__ double sred[16][64];
    __shared__ int64_t lp0[1024], lp1[1024];
    __shared__ int nlist;
    const int t = threadIdx.x;
    const int lane = lane_id();
    const int wave = t >> 6;
    const int hp = 1 << hp_log2;
    const int h = t & (hp - 1);
    const int64_t G = gridDim.x;
    for (int64_t first = blockIdx.x; first < rows; first += 1024 * G) {  // uniform trip count
        if (t == 0) nlist = 0;
        __syncthreads();
        const int64_t mine = first + G * t;
        if (mine < rows) {
            const int64_t q0 = indptr[mine], q1 = indptr[mine + 1];
            if (row_tier(q1 - q0, hp_log2) == 2) {
                int hub = -1;
                if (hub_ws && (q1 - q0) > (kHubValues >> hp_log2)) {
                    hub = atomicAdd(static_cast<int*>(hub_ws), 1);  // any order: rows are independent
                    if (hub < kMaxHubs) {
                        int64_t* hl = reinterpret_cast<int64_t*>(static_cast<char*>(hub_ws) + hub_list_offset());
                        hl[2 * hub] = q0;
                        hl[2 * hub + 1] = q1;
                    }
                }
                if (hub < 0 || hub >= kMaxHubs) {
                    const int k = atomicAdd(&nlist, 1);
                    lp0[k] = q0;
                    lp1[k] = q1;
                }
            }
        }
        __syncthreads();
        const int n = nlist;
        for (int k = 0; k < n; ++k) {
            const int64_t p0 = lp0[k], p1 = lp1[k];
            if (FWD) {
                float mx;
                double sum;
                fwd_partial<8>(e, eids, p0, p1, t, 1024, H, hp_log2, slope, mx, sum);
                for (int off = hp; off < kWave; off <<= 1) {
                    const float m2 = __shfl_xor(mx, off, kWave);
                    const double s2 = __shfl_xor(sum, off, kWave);
                    softmax_merge(mx, sum, m2, s2);
                }
                if (lane < hp) {
                    mred[wave][lane] = mx;
                    sred[wave][lane] = sum;
                }
                __syncthreads();
                mx = mred[0][h];
                sum = sred[0][h];
#pragma unroll
                for (int w = 1; w < 16; ++w) softmax_merge(mx, sum, mred[w][h], sred[w][h]);
                fwd_write<8>(out, e, eids, p0, p1, t, 1024, H, hp_log2, slope, mx, static_cast<float>(1.0 / sum));
            } else {
                double dsum = bwd_partial<8>(a, da, eids, p0, p1, t, 1024, H, hp_log2);
                for (int off = hp; off < kWave; off <<= 1) dsum += __shfl_xor(dsum, off, kWave);
                if (lane < hp) sred[wave][lane] = dsum;
                __syncthreads();
                dsum = 0.0;
#pragma unroll
                for (int w = 0; w < 16; ++w) dsum += sred[w][h];
                bwd_write<8>(out, a, da, e, eids, p0, p1, t, 1024, H, hp_log2, slope, static_cast<float>(dsum));
            }
            __syncthreads();  // the partial results are consumed before the next row overwrites them
        }
    }
}

// Hub launches.  blockDim.x = 256, grid = (kHubChunks, kHubGridY).  PHASE 0 writes the chunk's
// partials, PHASE 1 combines the kHubChunks partials of the row (every chunk does so for itself,
// in chunk order) and writes the chunk's outputs.
template <bool FWD, int PHASE>
__global__ __launch_bounds__(256) void edge_softmax_hub_kernel(
    float* __restrict__ out, const float* __restrict__ a, const float* __restrict__ da,
    const float* __restrict__ e, const int64_t* __restrict__ eids, int H, int hp_log2, float slope,
    void* __restrict__ hub_ws) {
    __shared__ float mred[4][64];
    __shared__ double sred[4][64];
    const int count = *static_cast<const int*>(hub_ws);
    const int nhubs = count < kMaxHubs ? count : kMaxHubs;
    const int64_t* hl = reinterpret_cast<const int64_t*>(static_cast<const char*>(hub_ws) + hub_list_offset());
    HubPartial* part = reinterpret_cast<HubPartial*>(static_cast<char*>(hub_ws) + hub_partial_offset());
    const int t = threadIdx.x, lane = lane_id(), wave = t >> 6;
    const int hp = 1 << hp_log2;
    const int h = t & (hp - 1);
    const int c = blockIdx.x;
    for (int hub = blockIdx.y; hub < nhubs; hub += gridDim.y) {
        const int64_t p0 = hl[2 * hub], p1 = hl[2 * hub + 1];
        const int64_t len = (p1 - p0 + kHubChunks - 1) / kHubChunks;
        const int64_t c0 = p0 + len * c < p1 ? p0 + len * c : p1;
        const int64_t c1 = c0 + len < p1 ? c0 + len : p1;
        HubPartial* row_part = part + (static_cast<int64_t>(hub) * kHubChunks << hp_log2);
        if (PHASE == 0) {
            float mx = -INFINITY;
            double sum = 0.0;
            if (FWD) {
                fwd_partial<8>(e, eids, c0, c1, t, 256, H, hp_log2, slope, mx, sum);
                for (int off = hp; off < kWave; off <<= 1) {
                    const float m2 = __shfl_xor(mx, off, kWave);
                    const double s2 = __shfl_xor(sum, off, kWave);
                    softmax_merge(mx, sum, m2, s2);
                }
            } else {
                sum = bwd_partial<8>(a, da, eids, c0, c1, t, 256, H, hp_log2);
                for (int off = hp; off < kWave; off <<= 1) sum += __shfl_xor(sum, off, kWave);
            }
            if (lane < hp) {
                mred[wave][lane] = mx;
                sred[wave][lane] = sum;
            }
            __syncthreads();
            if (t < hp) {
                mx = mred[0][t];
                sum = sred[0][t];
                for (int w = 1; w < 4; ++w) {
                    if (FWD) softmax_merge(mx, sum, mred[w][t], sred[w][t]);
                    else sum += sred[w][t];
                }
                row_part[(c << hp_log2) + t] = HubPartial{sum, mx, 0.0f};
            }
            __syncthreads();
        } else {
            float mx = -INFINITY;
            double sum = 0.0;
            for (int k = 0; k < kHubChunks; ++k) {
                const HubPartial q = row_part[(k << hp_log2) + h];
                if (FWD) softmax_merge(mx, sum, q.mx, q.sum);
                else sum += q.sum;
            }
            if (FWD) fwd_write<8>(out, e, eids, c0, c1, t, 256, H, hp_log2, slope, mx, static_cast<float>(1.0 / sum));
            else bwd_write<8>(out, a, da, e, eids, c0, c1, t, 256, H, hp_log2, slope, static_cast<float>(sum));
        }
    }
}

// Launches the tiers.  FWD: out = a; otherwise out = de.  hub_ws may be null.
template <bool FWD>
static void launch_tiers(float* out, const float* a, const float* da, const float* e, const int64_t* indptr,
                         const int64_t* eids, int64_t rows, int H, float slope, void* hub_ws, hipStream_t s) {
    int hp = 0;
    while ((1 << hp) < H) ++hp;
    const unsigned sgrid = static_cast<unsigned>(ceil_div(rows * H, 256));
    if (hub_ws) fill_u32(hub_ws, 0u, 1, s);  // the hub counter
    // the long tier first: its workgroups are the last to finish
    hipLaunchKernelGGL(edge_softmax_long_kernel<FWD>,
                       dim3(static_cast<unsigned>(rows < kLongGrid ? rows : kLongGrid)), dim3(1024), 0,
                       s, out, a, da, e, indptr, eids, rows, H, hp, slope, hub_ws);
    if (hub_ws) {
        const dim3 hgrid(kHubChunks, kHubGridY);
        hipLaunchKernelGGL((edge_softmax_hub_kernel<FWD, 0>), hgrid, dim3(256), 0, s, out, a, da, e, eids, H, hp, slope,
                           hub_ws);
        hipLaunchKernelGGL((edge_softmax_hub_kernel<FWD, 1>), hgrid, dim3(256), 0, s, out, a, da, e, eids, H, hp, slope,
                           hub_ws);
    }
    if (FWD)
        hipLaunchKernelGGL(edge_softmax_fwd_short_kernel, dim3(sgrid), dim3(256), 0, s, out, e, indptr, eids, rows, H,
                           slope);
    else
        hipLaunchKernelGGL(edge_softmax_bwd_short_kernel, dim3(sgrid), dim3(256), 0, s, out, a, da, e, indptr, eids,
                           rows, H, slope);
    hipLaunchKernelGGL(edge_softmax_medium_kernel<FWD>, dim3(static_cast<unsigned>(ceil_div(rows, 4 * kRowsPerWave))),
                       dim3(256), 0, s, out, a, da, e, indptr, eids, rows, H, hp, slope);
}

static size_t hub_workspace_bytes(int64_t H) {
    if (H <= 0 || H > 64) return 0;
    int hp = 0;
    while ((1 << hp) < H) ++hp;
    return hub_partial_offset() + (static_cast<size_t>(kMaxHubs) * kHubChunks << hp) * sizeof(HubPartial);
}

}  // namespace tango

using namespace tango;

extern "C" {

size_t tango_edge_softmax_workspace(int64_t H) { return hub_workspace_bytes(H); }

int tango_edge_softmax_fwd(float* a, const float* e, const int64_t* indptr,
                           const int64_t* edge_ids, int64_t rows, int64_t H, float slope,
                           void* workspace, size_t workspace_bytes, tango_stream_t stream) {
    if (rows < 0 || H < 0 || (rows > 0 && !indptr) || H >= (1LL << 31)) return TANGO_ERR_INVALID_ARG;
    if (rows * H == 0) return TANGO_OK;
    if (!a || !e) return TANGO_ERR_INVALID_ARG;
    if (H <= 64 && rows * H <= 256LL * INT32_MAX) {
        if (workspace && (workspace_bytes < hub_workspace_bytes(H) || (reinterpret_cast<uintptr_t>(workspace) & 15)))
            return TANGO_ERR_WORKSPACE;
        launch_tiers<true>(a, nullptr, nullptr, e, indptr, edge_ids, rows, static_cast<int>(H), slope, workspace,
                           as_stream(stream));
        return launch_status();
    }
    hipLaunchKernelGGL(edge_softmax_fwd_kernel, dim3(grid_for(rows * H, 256, 16)), dim3(256), 0,
                       as_stream(stream), a, e, indptr, edge_ids, rows, static_cast<int>(H), slope);
    return launch_status();
}

int tango_edge_softmax_bwd(float* de, const float* a, const float* da, const float* e,
                           const int64_t* indptr, const int64_t* edge_ids, int64_t rows,
                           int64_t H, float slope, void* workspace, size_t workspace_bytes,
                           tango_stream_t stream) {
    if (rows < 0 || H < 0 || (rows > 0 && !indptr) || H >= (1LL << 31)) return TANGO_ERR_INVALID_ARG;
    if (rows * H == 0) return TANGO_OK;
    if (!de || !a || !da || !e) return TANGO_ERR_INVALID_ARG;
    if (H <= 64 && rows * H <= 256LL * INT32_MAX) {
        if (workspace && (workspace_bytes < hub_workspace_bytes(H) || (reinterpret_cast<uintptr_t>(workspace) & 15)))
            return TANGO_ERR_WORKSPACE;
        launch_tiers<false>(de, a, da, e, indptr, edge_ids, rows, static_cast<int>(H), slope, workspace,
                            as_stream(stream));
        return launch_status();
    }
    hipLaunchKernelGGL(edge_softmax_bwd_kernel, dim3(grid_for(rows * H, 256, 16)), dim3(256), 0,
                       as_stream(stream), de, a, da, e, indptr, edge_ids, rows, static_cast<int>(H),
                       slope);
    return launch_status();
}

}  // extern "C"
