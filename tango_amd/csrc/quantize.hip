// Absmax scales and fp32 -> int8 quantization for gfx950.
//
// All three kernels are HBM-streaming: 4 B/element read for absmax, 5 B/element
// for quantize.  Each lane moves 16-byte vectors, a wavefront therefore covers
// 1 KiB per load instruction, and the grid is sized to keep every CU busy with
// several resident workgroups (the reference launches a fixed 960x128 grid,
// cuda/src/quantization.cu:39,87).
#include <type_traits>

#include "common.hpp"

namespace tango {

// ------------------------------------------------------------------ Philox
// Philox4x32-10, counter-based (Salmon et al., SC'11).  One call yields the
// noise of four consecutive elements.
struct Philox4 {
    uint32_t v[4];
};

__device__ __forceinline__ Philox4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2,
                                                 uint32_t c3, uint32_t k0, uint32_t k1) {
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        // one 32x32->64 multiply (v_mad_u64_u32) yields both halves; integer multiplies are quarter rate
        const uint64_t p0 = static_cast<uint64_t>(0xD2511F53u) * c0;
        const uint64_t p1 = static_cast<uint64_t>(0xCD9E8D57u) * c2;
        const uint32_t hi0 = static_cast<uint32_t>(p0 >> 32), lo0 = static_cast<uint32_t>(p0);
        const uint32_t hi1 = static_cast<uint32_t>(p1 >> 32), lo1 = static_cast<uint32_t>(p1);
        const uint32_t n0 = hi1 ^ c1 ^ k0;
        const uint32_t n2 = hi0 ^ c3 ^ k1;
        c0 = n0;
        c1 = lo1;
        c2 = n2;
        c3 = lo0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    return Philox4{{c0, c1, c2, c3}};
}

__device__ __forceinline__ float u01(uint32_t w) { return static_cast<float>(w >> 8) * 0x1.0p-24f; }

__device__ __forceinline__ float philox_uniform(uint64_t seed, uint64_t g) {
    const uint64_t blk = g >> 2;
    Philox4 r = philox4x32_10(static_cast<uint32_t>(blk), static_cast<uint32_t>(blk >> 32), 0u, 0u,
                              static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32));
    return u01(r.v[g & 3]);
}

// ------------------------------------------------------------------ absmax
__global__ __launch_bounds__(256) void absmax_kernel(const float* __restrict__ x, int64_t n,
                                                     int64_t head, float* __restrict__ out) {
    // [0, head) scalar, then n4 float4 vectors from an aligned base, then the tail
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int64_t nthr = static_cast<int64_t>(gridDim.x) * blockDim.x;
    float m = 0.0f;
    const int64_t n4 = (n - head) >> 2;
    const f32x4* x4 = reinterpret_cast<const f32x4*>(x + head);
    int64_t i = tid;
    for (; i + 3 * nthr < n4; i += 4 * nthr) {
        const f32x4 a = __builtin_nontemporal_load(x4 + i);
        const f32x4 b = __builtin_nontemporal_load(x4 + i + nthr);
        const f32x4 c = __builtin_nontemporal_load(x4 + i + 2 * nthr);
        const f32x4 d = __builtin_nontemporal_load(x4 + i + 3 * nthr);
        m = fmaxf(m, fmaxf(fmaxf(fabsf(a.x), fabsf(a.y)), fmaxf(fabsf(a.z), fabsf(a.w))));
        m = fmaxf(m, fmaxf(fmaxf(fabsf(b.x), fabsf(b.y)), fmaxf(fabsf(b.z), fabsf(b.w))));
        m = fmaxf(m, fmaxf(fmaxf(fabsf(c.x), fabsf(c.y)), fmaxf(fabsf(c.z), fabsf(c.w))));
        m = fmaxf(m, fmaxf(fmaxf(fabsf(d.x), fabsf(d.y)), fmaxf(fabsf(d.z), fabsf(d.w))));
    }
    for (; i < n4; i += nthr) {
        const f32x4 a = __builtin_nontemporal_load(x4 + i);
        m = fmaxf(m, fmaxf(fmaxf(fabsf(a.x), fabsf(a.y)), fmaxf(fabsf(a.z), fabsf(a.w))));
    }
    if (tid < head) m = fmaxf(m, fabsf(x[tid]));
    const int64_t tail0 = head + (n4 << 2);
    if (tail0 + tid < n) m = fmaxf(m, fabsf(x[tail0 + tid]));
    block_absmax_to_global(m / 127.0f, out);
}

// max |x[r, c] * row_mul[r]| / 127 of a dense matrix (no padding between rows) with an even number of columns,
// walked as a flat array of 16-byte vectors like absmax_kernel: rows whose length is not a multiple of four
// floats (602 columns) then cost no narrow loads.  A vector starts at an even column, so it lies in one row
// or has its second half in the next; the (row, column) of a lane's vector advances by a fixed step.
__global__ __launch_bounds__(256) void absmax_rowmul_dense_kernel(const float* __restrict__ x, int64_t n, int64_t cols,
                                                                  const float* __restrict__ row_mul,
                                                                  float* __restrict__ out) {
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int64_t nthr = static_cast<int64_t>(gridDim.x) * blockDim.x;
    const int64_t n4 = n >> 2;
    const f32x4* x4 = reinterpret_cast<const f32x4*>(x);
    int64_t row = (4 * tid) / cols, col = (4 * tid) % cols;
    const int64_t srow = (4 * nthr) / cols, scol = (4 * nthr) % cols;
    float m = 0.0f;
    // the two multipliers of a vector, then the step to the lane's next vector: index arithmetic and selects only,
    // so that the multiplier loads of a whole batch are in flight together with its vector loads
    auto multipliers = [&](float& r0, float& r1) {
        r0 = row_mul[row];
        r1 = row_mul[row + (col + 2 >= cols ? 1 : 0)];  // a vector whose second half is in the next row never ends the matrix
        row += srow;
        col += scol;
        const bool wrap = col >= cols;
        col -= wrap ? cols : 0;
        row += wrap ? 1 : 0;
    };
    auto take = [&](const f32x4 v, float r0, float r1) {
        m = fmaxf(m, fmaxf(fmaxf(fabsf(v.x * r0), fabsf(v.y * r0)), fmaxf(fabsf(v.z * r1), fabsf(v.w * r1))));
    };
    int64_t i = tid;
    for (; i + 7 * nthr < n4; i += 8 * nthr) {  // eight 16-byte loads in flight per lane
        f32x4 v[8];
        float r0[8], r1[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(x4 + i + u * nthr);
#pragma unroll
        for (int u = 0; u < 8; ++u) multipliers(r0[u], r1[u]);
#pragma unroll
        for (int u = 0; u < 8; ++u) take(v[u], r0[u], r1[u]);
    }
    for (; i < n4; i += nthr) {
        const f32x4 v = __builtin_nontemporal_load(x4 + i);
        float r0, r1;
        multipliers(r0, r1);
        take(v, r0, r1);
    }
    const int64_t t = (n4 << 2) + tid;  // at most two elements remain, in the last row
    if (t < n) m = fmaxf(m, fabsf(x[t] * row_mul[t / cols]));
    block_absmax_to_global(m / 127.0f, out);
}

// One workgroup, direct store: small tensors need no atomic and no pre-zeroing.
__global__ __launch_bounds__(1024) void absmax_small_kernel(const float* __restrict__ x, int64_t n,
                                                            float* __restrict__ out) {
    __shared__ float part[16];
    float m = 0.0f;
    if ((reinterpret_cast<uintptr_t>(x) & 15) == 0) {
        // four independent 16-byte loads in flight per thread: one workgroup is bound by load latency
        const f32x4* x4 = reinterpret_cast<const f32x4*>(x);
        const int64_t n4 = n >> 2;
        for (int64_t i = threadIdx.x; i < n4; i += 4 * blockDim.x) {
            f32x4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int64_t j = i + u * blockDim.x;
                v[u] = j < n4 ? x4[j] : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
                m = fmaxf(fmaxf(m, fmaxf(fabsf(v[u][0]), fabsf(v[u][1]))), fmaxf(fabsf(v[u][2]), fabsf(v[u][3])));
        }
        for (int64_t i = (n4 << 2) + threadIdx.x; i < n; i += blockDim.x) m = fmaxf(m, fabsf(x[i]));
    } else {
        for (int64_t i = threadIdx.x; i < n; i += blockDim.x) m = fmaxf(m, fabsf(x[i]));
    }
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x < 64) {
        float v = (threadIdx.x < (blockDim.x >> 6)) ? part[threadIdx.x] : 0.0f;
        v = wave_max(v);
        if (threadIdx.x == 0) out[0] = v / 127.0f;
    }
}

// One wavefront per row.
__global__ __launch_bounds__(256) void absmax_rows_kernel(const float* __restrict__ x,
                                                          int64_t rows, int64_t cols, int64_t ldx,
                                                          float* __restrict__ out) {
    const int64_t row = static_cast<int64_t>(blockIdx.x) * (blockDim.x / kWave) + threadIdx.x / kWave;
    if (row >= rows) return;
    const float* xr = x + row * ldx;
    float m = 0.0f;
    for (int64_t c = lane_id(); c < cols; c += kWave) m = fmaxf(m, fabsf(xr[c]));
    m = wave_max(m);
    if (lane_id() == 0) out[row] = m / 127.0f;
}

// ---------------------------------------------------------------- quantize
// Vector body: x is 16-byte aligned, q 4-byte aligned, n4 = n / 4 vectors.
template <int MODE>
__global__ __launch_bounds__(256) void quantize_vec_kernel(
    const float* __restrict__ x, int64_t n, const float* __restrict__ scale,
    int8_t* __restrict__ q, const float* __restrict__ noise, uint64_t seed, uint64_t offset_host,
    const uint64_t* __restrict__ offset_dev) {
    const uint64_t offset = offset_host + (offset_dev ? offset_dev[0] : 0);
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int64_t nthr = static_cast<int64_t>(gridDim.x) * blockDim.x;
    const float r = rscale_of(scale[0]);
    const int64_t n4 = n >> 2;
    const f32x4* x4 = reinterpret_cast<const f32x4*>(x);
    uint32_t* q4 = reinterpret_cast<uint32_t*>(q);
    const bool shared_block = (offset & 3) == 0;  // the 4 elements share one Philox block
    for (int64_t i = tid; i < n4; i += nthr) {
        const f32x4 v = __builtin_nontemporal_load(x4 + i);
        float u0 = 0.f, u1 = 0.f, u2 = 0.f, u3 = 0.f;
        if (MODE == TANGO_ROUND_STOCHASTIC) {
            if (noise) {
                // noise shares x's element index but not necessarily its alignment
                u0 = noise[4 * i];
                u1 = noise[4 * i + 1];
                u2 = noise[4 * i + 2];
                u3 = noise[4 * i + 3];
            } else if (shared_block) {
                const uint64_t blk = (offset + 4 * static_cast<uint64_t>(i)) >> 2;
                Philox4 p = philox4x32_10(static_cast<uint32_t>(blk), static_cast<uint32_t>(blk >> 32),
                                          0u, 0u, static_cast<uint32_t>(seed),
                                          static_cast<uint32_t>(seed >> 32));
                u0 = u01(p.v[0]);
                u1 = u01(p.v[1]);
                u2 = u01(p.v[2]);
                u3 = u01(p.v[3]);
            } else {
                const uint64_t g = offset + 4 * static_cast<uint64_t>(i);
                u0 = philox_uniform(seed, g);
                u1 = philox_uniform(seed, g + 1);
                u2 = philox_uniform(seed, g + 2);
                u3 = philox_uniform(seed, g + 3);
            }
        }
        const uint32_t w = pack4(quant_one<MODE>(v.x, r, u0), quant_one<MODE>(v.y, r, u1),
                                 quant_one<MODE>(v.z, r, u2), quant_one<MODE>(v.w, r, u3));
        __builtin_nontemporal_store(w, q4 + i);
    }
    const int64_t t = (n4 << 2) + tid;  // tail: at most 3 elements
    if (t < n) {
        float u = 0.f;
        if (MODE == TANGO_ROUND_STOCHASTIC) u = noise ? noise[t] : philox_uniform(seed, offset + t);
        q[t] = static_cast<int8_t>(quant_one<MODE>(x[t], r, u));
    }
}

// x under the mask value mk of a fused activation backward.  Mode 0 (ReLU): x where mk > 0, else 0.
// Mode 1 (ELU, mk = the activation's output): x where mk > 0, else x * (mk + 1), since
// d/dz (exp(z) - 1) = exp(z) = elu(z) + 1.
__device__ __forceinline__ float masked(float x, float mk, int mode) {
    if (mk > 0.0f) return x;
    return mode == 1 ? x * (mk + 1.0f) : 0.0f;
}

// Mode 2: the mask is one sign bit per element, bit c % 16 of the 16-bit word c / 16 of the row (what the
// aggregation's ReLU epilogue can write beside its output: 1/32 of the bytes of the fp32 output the other
// modes read).  mk[k] = 1 where the bit of column c0 + k is set, else 0; c0 is a multiple of four.
__device__ __forceinline__ void mask_bits4(float* mk, const uint16_t* __restrict__ words, int64_t c0) {
    const unsigned w = static_cast<unsigned>(words[c0 >> 4]) >> (c0 & 15);
#pragma unroll
    for (int k = 0; k < 4; ++k) mk[k] = ((w >> k) & 1u) ? 1.0f : 0.0f;
}

// quantize_rows_kernel's job on dense matrices whose rows hold a multiple of four columns (x, q and the
// mask all [rows, cols] without padding): the flat walk of quantize_vec_kernel, a lane's four elements
// never straddle a row, and the row index (for row_mul) advances by a fixed step per iteration.
template <int MODE, bool COLSUM = false>
__global__ __launch_bounds__(256) void quantize_dense_ex_kernel(
    const float* __restrict__ x, int64_t n4, int64_t cols, const float* __restrict__ scale,
    int8_t* __restrict__ q, const float* __restrict__ noise, uint64_t seed, uint64_t offset_host,
    const uint64_t* __restrict__ offset_dev,
    const float* __restrict__ row_mul, const float* __restrict__ mask, int mask_mode,
    float* __restrict__ colsum_partial /* null, or [gridDim.x, cols]: needs 256 % (cols / 4) == 0 */) {
    const uint64_t offset = offset_host + (offset_dev ? offset_dev[0] : 0);
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int64_t nthr = static_cast<int64_t>(gridDim.x) * blockDim.x;
    const float r = rscale_of(scale[0]);
    const f32x4* x4 = reinterpret_cast<const f32x4*>(x);
    const f32x4* m4 = reinterpret_cast<const f32x4*>(mask);
    uint32_t* q4 = reinterpret_cast<uint32_t*>(q);
    const bool shared_block = (offset & 3) == 0;
    int64_t row = (4 * tid) / cols, col = (4 * tid) % cols;
    const int64_t srow = (4 * nthr) / cols, scol = (4 * nthr) % cols;
    // column sums of the masked input (before the row multiplier): with a number of threads that is a multiple of
    // cols / 4 a lane meets the same four columns in every iteration
    float cs[4] = {0.f, 0.f, 0.f, 0.f};
    // The sign word and the row multiplier of a vector are asked for together with the vector, without a branch
    // around the loads (absent operands: some valid address, value unused): one memory round trip per iteration
    // instead of three in a row.
    const bool bits_mode = mask && mask_mode == 2;
    const uint16_t* words = bits_mode ? reinterpret_cast<const uint16_t*>(mask) : reinterpret_cast<const uint16_t*>(x);
    const float* rmp = row_mul ? row_mul : x;
    for (int64_t i = tid; i < n4; i += nthr) {
        const f32x4 v = __builtin_nontemporal_load(x4 + i);
        const unsigned word = words[(4 * i) >> 4];  // dense rows of a multiple of 16 columns: element e lies in word e / 16
        const float rm = rmp[row_mul ? row : 0];
        float f[4] = {v.x, v.y, v.z, v.w};
        if (bits_mode) {
            const unsigned w = word >> ((4 * i) & 15);
#pragma unroll
            for (int k = 0; k < 4; ++k) f[k] = ((w >> k) & 1u) ? f[k] : 0.0f;
        } else if (mask) {
            const f32x4 mk = __builtin_nontemporal_load(m4 + i);
            f[0] = masked(f[0], mk.x, mask_mode); f[1] = masked(f[1], mk.y, mask_mode);
            f[2] = masked(f[2], mk.z, mask_mode); f[3] = masked(f[3], mk.w, mask_mode);
        }
        if (COLSUM) {
#pragma unroll
            for (int k = 0; k < 4; ++k) cs[k] += f[k];
        }
        if (row_mul) {
#pragma unroll
            for (int k = 0; k < 4; ++k) f[k] = f[k] * rm;
            row += srow;
            col += scol;
            const bool wrap = col >= cols;
            col -= wrap ? cols : 0;
            row += wrap ? 1 : 0;
        }
        float u[4] = {0.f, 0.f, 0.f, 0.f};
        if (MODE == TANGO_ROUND_STOCHASTIC) {
            if (noise) {
#pragma unroll
                for (int k = 0; k < 4; ++k) u[k] = noise[4 * i + k];
            } else if (shared_block) {
                const uint64_t blk = (offset + 4 * static_cast<uint64_t>(i)) >> 2;
                const Philox4 p = philox4x32_10(static_cast<uint32_t>(blk), static_cast<uint32_t>(blk >> 32), 0u, 0u,
                                                static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32));
#pragma unroll
                for (int k = 0; k < 4; ++k) u[k] = u01(p.v[k]);
            } else {
                const uint64_t g = offset + 4 * static_cast<uint64_t>(i);
#pragma unroll
                for (int k = 0; k < 4; ++k) u[k] = philox_uniform(seed, g + k);
            }
        }
        __builtin_nontemporal_store(pack4(quant_one<MODE>(f[0], r, u[0]), quant_one<MODE>(f[1], r, u[1]),
                                          quant_one<MODE>(f[2], r, u[2]), quant_one<MODE>(f[3], r, u[3])), q4 + i);
    }
    if (COLSUM) {  // the lanes of a column quad are threadIdx.x = quad, quad + cols / 4, ...: added in that order
        __shared__ float red[256][4];
#pragma unroll
        for (int k = 0; k < 4; ++k) red[threadIdx.x][k] = cs[k];
        __syncthreads();
        const int quads = static_cast<int>(cols >> 2);
        if (static_cast<int>(threadIdx.x) < quads) {
            float a[4] = {0.f, 0.f, 0.f, 0.f};
            for (int t = threadIdx.x; t < 256; t += quads)
#pragma unroll
                for (int k = 0; k < 4; ++k) a[k] += red[t][k];
            float* prow = colsum_partial + static_cast<int64_t>(blockIdx.x) * cols + 4 * threadIdx.x;
#pragma unroll
            for (int k = 0; k < 4; ++k) prow[k] = a[k];
        }
    }
}

// The same flat walk for dense inputs whose rows do NOT hold a multiple of four columns (41): a lane's four
// consecutive elements may belong to two rows, so each carries its own (row, column); x is read with 16-byte loads
// and, with stochastic rounding, a lane computes one Philox block for its four elements (the row-strided kernel
// walks such rows with 4-byte loads and two Philox blocks per lane: 0.050 ms on [232965, 41] against 0.012 ms
// here).  The output rows are padded (ldq >= cols): the bytes go out one by one, and the lane that holds a row's
// last element also zeroes the row's padding.  n = rows * cols; the last n % 4 elements are done by the first lanes.
template <int MODE>
__global__ __launch_bounds__(256) void quantize_flat_rows_kernel(
    const float* __restrict__ x, int64_t n, int64_t cols, const float* __restrict__ scale,
    int8_t* __restrict__ q, int64_t ldq, const float* __restrict__ noise, uint64_t seed, uint64_t offset_host,
    const uint64_t* __restrict__ offset_dev, const float* __restrict__ row_mul) {
    const uint64_t offset = offset_host + (offset_dev ? offset_dev[0] : 0);
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int64_t nthr = static_cast<int64_t>(gridDim.x) * blockDim.x;
    const float r = rscale_of(scale[0]);
    const f32x4* x4 = reinterpret_cast<const f32x4*>(x);
    const bool shared_block = (offset & 3) == 0;
    const int64_t n4 = n >> 2;
    int64_t row = (4 * tid) / cols, col = (4 * tid) % cols;
    const int64_t srow = (4 * nthr) / cols, scol = (4 * nthr) % cols;
    auto one = [&](float f, int64_t e, int64_t rw, int64_t cl, float u) {
        if (row_mul) f = f * row_mul[rw];
        if (MODE == TANGO_ROUND_STOCHASTIC && noise) u = noise[e];
        int8_t* qr = q + rw * ldq;
        qr[cl] = static_cast<int8_t>(quant_one<MODE>(f, r, u));
        if (cl == cols - 1)
            for (int64_t c = cols; c < ldq; ++c) qr[c] = 0;
    };
    for (int64_t i = tid; i < n4; i += nthr) {
        const f32x4 v = __builtin_nontemporal_load(x4 + i);
        const float f[4] = {v.x, v.y, v.z, v.w};
        float u[4] = {0.f, 0.f, 0.f, 0.f};
        if (MODE == TANGO_ROUND_STOCHASTIC && !noise) {
            if (shared_block) {
                const uint64_t blk = (offset + 4 * static_cast<uint64_t>(i)) >> 2;
                const Philox4 ph = philox4x32_10(static_cast<uint32_t>(blk), static_cast<uint32_t>(blk >> 32), 0u, 0u,
                                                 static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32));
#pragma unroll
                for (int k = 0; k < 4; ++k) u[k] = u01(ph.v[k]);
            } else {
                const uint64_t g = offset + 4 * static_cast<uint64_t>(i);
#pragma unroll
                for (int k = 0; k < 4; ++k) u[k] = philox_uniform(seed, g + k);
            }
        }
        int64_t rw = row, cl = col;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            one(f[k], 4 * i + k, rw, cl, u[k]);
            if (++cl == cols) { cl = 0; ++rw; }
        }
        row += srow;
        col += scol;
        if (col >= cols) { col -= cols; ++row; }
    }
    const int64_t e = (n4 << 2) + tid;  // at most three elements remain, in the last row
    if (e < n) {
        float u = 0.f;
        if (MODE == TANGO_ROUND_STOCHASTIC && !noise) u = philox_uniform(seed, offset + e);
        one(x[e], e, e / cols, e % cols, u);
    }
}

// The same job for narrow rows (cols <= 128, not a multiple of four) into padded, 16-byte aligned output rows: a
// workgroup takes R consecutive rows (R a multiple of four with R * cols <= 1024, so that its dense elements start
// on a 16-byte boundary), every lane quantizes four consecutive dense elements exactly as the flat kernel above does
// (same Philox block per lane, so the same bytes), but the bytes meet in an LDS image of the R padded rows, which
// then leaves as one contiguous run of 16-byte stores: on [232965, 41] -> row pitch 64 the flat kernel's byte
// stores and per-row padding loops take 27 (half-even) to 41 us (stochastic) inside an epoch.
template <int MODE>
__global__ __launch_bounds__(256) void quantize_tile_rows_kernel(
    const float* __restrict__ x, int64_t rows, int cols, const float* __restrict__ scale, int8_t* __restrict__ q,
    int ldq, int R, const float* __restrict__ noise, uint64_t seed, uint64_t offset_host,
    const uint64_t* __restrict__ offset_dev, const float* __restrict__ row_mul) {
    extern __shared__ __attribute__((aligned(16))) uint8_t tile_rows[];  // [R][ldq]
    const uint64_t offset = offset_host + (offset_dev ? offset_dev[0] : 0);
    const bool shared_block = (offset & 3) == 0;
    const float r = rscale_of(scale[0]);
    const int tid = threadIdx.x;
    const int e0 = 4 * tid;
    // (row, column) inside the workgroup's rows of a lane's four elements: the same for every group of rows
    int rl[4], cl[4];
    rl[0] = e0 / cols;
    cl[0] = e0 - rl[0] * cols;
#pragma unroll
    for (int k = 1; k < 4; ++k) {
        const bool wrap = cl[k - 1] + 1 == cols;
        cl[k] = wrap ? 0 : cl[k - 1] + 1;
        rl[k] = rl[k - 1] + (wrap ? 1 : 0);
    }
    i32x4* tile16 = reinterpret_cast<i32x4*>(tile_rows);
    for (int64_t row0 = static_cast<int64_t>(blockIdx.x) * R; row0 < rows; row0 += static_cast<int64_t>(gridDim.x) * R) {
        const int rows_here = static_cast<int>(rows - row0 < R ? rows - row0 : R);
        const int nel = rows_here * cols;
        const int vecs = rows_here * (ldq >> 4);
        for (int i = tid; i < vecs; i += 256) tile16[i] = i32x4{0, 0, 0, 0};  // the padding of every row
        __syncthreads();
        if (e0 < nel) {
            const int64_t g0 = row0 * cols + e0;  // a multiple of four: R is
            float f[4], rm[4], u[4] = {0.f, 0.f, 0.f, 0.f};
            if (e0 + 4 <= nel) {
                const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(x + g0));
                f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
            } else {
#pragma unroll
                for (int k = 0; k < 4; ++k) f[k] = e0 + k < nel ? x[g0 + k] : 0.0f;
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int64_t rw = row0 + rl[k];
                rm[k] = row_mul ? row_mul[rw < rows ? rw : rows - 1] : 1.0f;
            }
            if (MODE == TANGO_ROUND_STOCHASTIC) {
                if (noise) {
#pragma unroll
                    for (int k = 0; k < 4; ++k) u[k] = e0 + k < nel ? noise[g0 + k] : 0.0f;
                } else if (shared_block) {
                    const uint64_t blk = (offset + static_cast<uint64_t>(g0)) >> 2;
                    const Philox4 ph = philox4x32_10(static_cast<uint32_t>(blk), static_cast<uint32_t>(blk >> 32), 0u, 0u,
                                                     static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32));
#pragma unroll
                    for (int k = 0; k < 4; ++k) u[k] = u01(ph.v[k]);
                } else {
#pragma unroll
                    for (int k = 0; k < 4; ++k) u[k] = philox_uniform(seed, offset + static_cast<uint64_t>(g0) + k);
                }
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float fv = row_mul ? f[k] * rm[k] : f[k];
                if (e0 + k < nel) tile_rows[rl[k] * ldq + cl[k]] = static_cast<uint8_t>(quant_one<MODE>(fv, r, u[k]));
            }
        }
        __syncthreads();
        i32x4* out16 = reinterpret_cast<i32x4*>(q + row0 * ldq);
        for (int i = tid; i < vecs; i += 256) __builtin_nontemporal_store(tile16[i], out16 + i);
        __syncthreads();  // the image is zeroed again for the next rows
    }
}

// Scalar fallback for misaligned views.
template <int MODE>
__global__ __launch_bounds__(256) void quantize_scalar_kernel(
    const float* __restrict__ x, int64_t n, const float* __restrict__ scale,
    int8_t* __restrict__ q, const float* __restrict__ noise, uint64_t seed, uint64_t offset_host,
    const uint64_t* __restrict__ offset_dev) {
    const uint64_t offset = offset_host + (offset_dev ? offset_dev[0] : 0);
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int64_t nthr = static_cast<int64_t>(gridDim.x) * blockDim.x;
    const float r = rscale_of(scale[0]);
    for (int64_t i = tid; i < n; i += nthr) {
        float u = 0.f;
        if (MODE == TANGO_ROUND_STOCHASTIC) u = noise ? noise[i] : philox_uniform(seed, offset + i);
        q[i] = static_cast<int8_t>(quant_one<MODE>(x[i], r, u));
    }
}

// Four consecutive floats of a row starting at column c0 (zero beyond `cols`), with the widest
// aligned access the row layout allows: XV = 4 (16-byte rows), 2 (8-byte) or 1.
template <int XV>
__device__ __forceinline__ void load4(float* f, const float* __restrict__ row, int64_t c0, int64_t cols) {
    f[0] = f[1] = f[2] = f[3] = 0.0f;
    if (XV == 4 && c0 + 4 <= cols) {
        const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(row + c0));
        f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
    } else if (XV == 2 && c0 + 4 <= cols) {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        const f32x2 v0 = __builtin_nontemporal_load(reinterpret_cast<const f32x2*>(row + c0));
        const f32x2 v1 = __builtin_nontemporal_load(reinterpret_cast<const f32x2*>(row + c0 + 2));
        f[0] = v0.x; f[1] = v0.y; f[2] = v1.x; f[3] = v1.y;
    } else {
#pragma unroll
        for (int k = 0; k < 4; ++k)
            if (c0 + k < cols) f[k] = row[c0 + k];
    }
}

// Row-strided: blockDim = (64, 4); each wavefront walks one row at a time, one lane per
// output dword (4 columns, padding included), so no per-thread index division is needed and
// a wavefront's loads and stores are contiguous.  XV = floats per aligned load (4, 2 or 1).
template <int MODE, int XV>
__global__ __launch_bounds__(256) void quantize_rows_kernel(
    const float* __restrict__ x, int64_t rows, int64_t cols, int64_t ldx,
    const float* __restrict__ scale, int per_row, int8_t* __restrict__ q, int64_t ldq,
    const float* __restrict__ noise, uint64_t seed, uint64_t offset_host, const uint64_t* __restrict__ offset_dev,
    const float* __restrict__ row_mul, const float* __restrict__ mask, int64_t ldm, int gpr_log2,
    int mask_mode) {
    const uint64_t offset = offset_host + (offset_dev ? offset_dev[0] : 0);
    // the mask may use x's vector width when its rows are laid out and aligned like x's
    const bool mask_vec = mask && ldm == ldx &&
                          ((reinterpret_cast<uintptr_t>(mask) ^ reinterpret_cast<uintptr_t>(x)) & 15) == 0;
    const int64_t groups = (ldq + 3) >> 2;  // dword groups per row
    const bool quad_aligned = (cols & 3) == 0 && (offset & 3) == 0;  // every lane's quad starts a Philox block
    const bool dword_ok = (ldq & 3) == 0 && (reinterpret_cast<uintptr_t>(q) & 3) == 0;
    // narrow rows: a wavefront takes 64 / gpr rows at once (gpr = groups rounded up to a power of two)
    const int gpr = 1 << gpr_log2;
    const int rpw = kWave >> gpr_log2;
    const int sub = static_cast<int>(threadIdx.x) >> gpr_log2;
    const int64_t row_step = static_cast<int64_t>(gridDim.x) * blockDim.y * rpw;
    for (int64_t row = (static_cast<int64_t>(blockIdx.x) * blockDim.y + threadIdx.y) * rpw + sub; row < rows;
         row += row_step) {
        const float r = rscale_of(scale[per_row ? row : 0]);
        const float* xr = x + row * ldx;
        int8_t* qr = q + row * ldq;
        for (int64_t gi = threadIdx.x & (gpr - 1); gi < groups; gi += gpr) {
            const int64_t c0 = gi << 2;
            float f[4];
            load4<XV>(f, xr, c0, cols);
            if (mask) {  // the activation's backward first (as the absmax pass does), then the row multiplier
                float mk[4];
                if (mask_mode == 2) mask_bits4(mk, reinterpret_cast<const uint16_t*>(mask) + row * ldm, c0);
                else if (mask_vec) load4<XV>(mk, mask + row * ldm, c0, cols);
                else load4<1>(mk, mask + row * ldm, c0, cols);
#pragma unroll
                for (int k = 0; k < 4; ++k) f[k] = masked(f[k], mk[k], mask_mode);
            }
            if (row_mul) {  // x * row_mul[row], one rounding, before quantization
                const float rm = row_mul[row];
#pragma unroll
                for (int k = 0; k < 4; ++k) f[k] = f[k] * rm;
            }
            int v[4];
            const uint64_t lin = static_cast<uint64_t>(row) * cols + c0;
            float u[4] = {0.f, 0.f, 0.f, 0.f};
            if (MODE == TANGO_ROUND_STOCHASTIC) {
                if (noise) {
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        if (c0 + k < cols) u[k] = noise[lin + k];
                } else {
                    const uint64_t g0 = offset + lin;
                    const uint64_t b0 = g0 >> 2;
                    const Philox4 p0 = philox4x32_10(static_cast<uint32_t>(b0), static_cast<uint32_t>(b0 >> 32), 0u, 0u,
                                                     static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32));
                    if (quad_aligned) {  // uniform: a lane's four elements are exactly one Philox block
#pragma unroll
                        for (int k = 0; k < 4; ++k) u[k] = u01(p0.v[k]);
                    } else {
                    // the four elements touch two Philox blocks
                    Philox4 p1 = p0;
                    if (g0 & 3)
                        p1 = philox4x32_10(static_cast<uint32_t>(b0 + 1), static_cast<uint32_t>((b0 + 1) >> 32), 0u, 0u,
                                           static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32));
                    // words shift .. shift + 3 of the eight, picked with selects (a register array indexed
                    // by a run-time value would live in scratch memory)
                    const int shift = static_cast<int>(g0 & 3);
                    const uint32_t w[8] = {p0.v[0], p0.v[1], p0.v[2], p0.v[3], p1.v[0], p1.v[1], p1.v[2], p1.v[3]};
                    uint32_t h[6];
#pragma unroll
                    for (int i = 0; i < 6; ++i) h[i] = (shift & 1) ? w[i + 1] : w[i];
#pragma unroll
                    for (int k = 0; k < 4; ++k) u[k] = u01((shift & 2) ? h[k + 2] : h[k]);
                    }
                }
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] = (c0 + k < cols) ? quant_one<MODE>(f[k], r, u[k]) : 0;
            if (dword_ok) {
                __builtin_nontemporal_store(pack4(v[0], v[1], v[2], v[3]), reinterpret_cast<uint32_t*>(qr + c0));
            } else {
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    if (c0 + k < ldq) qr[c0 + k] = static_cast<int8_t>(v[k]);
            }
        }
    }
}

// --------------------------------------------------------- transpose_quant
// x[nrow, ncol] fp32 -> out[ncol, nrow] int8.  One thread owns four
// consecutive rows, so for every column the wavefront stores 256 contiguous
// bytes; the reads of a wavefront cover one contiguous 1 KiB * ncol span.
__global__ __launch_bounds__(256) void transpose_quant_kernel(const float* __restrict__ x,
                                                              int64_t nrow, int64_t ncol,
                                                              const float* __restrict__ scale,
                                                              int8_t* __restrict__ out) {
    const float r = rscale_of(scale[0]);
    const int64_t groups = (nrow + 3) >> 2;
    const int64_t nthr = static_cast<int64_t>(gridDim.x) * blockDim.x;
    const bool dword_ok = (nrow & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 3) == 0;
    for (int64_t g = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; g < groups;
         g += nthr) {
        const int64_t r0 = g << 2;
        for (int64_t c = 0; c < ncol; ++c) {
            int v[4];
#pragma unroll
            for (int k = 0; k < 4; ++k)
                v[k] = (r0 + k < nrow) ? quant_one<TANGO_ROUND_RNE>(x[(r0 + k) * ncol + c], r, 0.f) : 0;
            int8_t* o = out + c * nrow + r0;
            if (dword_ok) {
                *reinterpret_cast<uint32_t*>(o) = pack4(v[0], v[1], v[2], v[3]);
            } else {
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    if (r0 + k < nrow) o[k] = static_cast<int8_t>(v[k]);
            }
        }
    }
}

// max |x[r,c] * row_mul[r]| over unmasked elements, and optionally the column sums of the
// unmasked x (not multiplied): the two reductions of a fused "mask, sum for the bias gradient,
// scale rows, quantize" backward step in one read of x.  blockDim = (64, 4), a wavefront walks
// rows; lane l owns columns 4 l .. 4 l + 3 (+ 256 t).  Column sums are written as one partial
// row per wavefront and reduced in a fixed order afterwards, so they are deterministic.
template <int T, int XV, int MK /* 0 no mask, 1 fp32 mask, 2 sign-bit words */>
__global__ __launch_bounds__(256) void absmax_ex_kernel(
    const float* __restrict__ x, int64_t rows, int64_t cols, int64_t ldx,
    const float* __restrict__ row_mul, const float* __restrict__ mask, int64_t ldm,
    float* __restrict__ scale_out, float* __restrict__ partial /* [gridDim.x, cols] or null */,
    int gpr_log2, int mask_mode) {
    __shared__ float red[3][T * 256];
    const bool mask_vec = mask && ldm == ldx &&
                          ((reinterpret_cast<uintptr_t>(mask) ^ reinterpret_cast<uintptr_t>(x)) & 15) == 0;
    const bool whole_quads = (cols & 3) == 0 && rows > 0;
    float m = 0.0f;
    float cs[T][4];
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
        for (int k = 0; k < 4; ++k) cs[t][k] = 0.0f;
    // narrow rows (T == 1): a wavefront takes 64 / gpr rows at once, lane = (row in wave, column group)
    const int gpr = 1 << gpr_log2;
    const int rpw = kWave >> gpr_log2;
    const int sub = static_cast<int>(threadIdx.x) >> gpr_log2;
    const int gl = static_cast<int>(threadIdx.x) & (gpr - 1);
    const int64_t row_step = static_cast<int64_t>(gridDim.x) * blockDim.y * rpw;
    constexpr int RU = 4;  // rows in flight per lane: the loads of four rows are issued before any is used
    for (int64_t row0 = (static_cast<int64_t>(blockIdx.x) * blockDim.y + threadIdx.y) * rpw + sub; row0 < rows;
         row0 += RU * row_step) {
        float v[RU][T][4];
        float mk[MK == 1 ? RU : 1][T][4];  // fp32 mask values
        unsigned wb[MK == 2 ? RU : 1][T];  // the four sign bits of the lane's columns (bit set = keep)
        // the rows' multipliers, asked for with the rows themselves (without a multiplier: some valid address, and
        // the value is not used); a load in the loop that consumes the rows would wait for each row in turn
        float rmv[RU];
        {
            const float* rmp = row_mul ? row_mul : x;
#pragma unroll
            for (int u = 0; u < RU; ++u) {
                const int64_t row = row0 + u * row_step;
                rmv[u] = rmp[row_mul ? (row < rows ? row : rows - 1) : 0];
            }
        }
        if (XV == 4 && whole_quads && (MK != 1 || mask_vec)) {
            // No lane has a partial quad: every load is issued unconditionally from a clamped address and the
            // lanes outside the matrix discard theirs.  Without branches between them the loads of all RU rows
            // are in flight together (with the guarded form below the compiler waits between rows).
#pragma unroll
            for (int u = 0; u < RU; ++u) {
                const int64_t row = row0 + u * row_step;
#pragma unroll
                for (int t = 0; t < T; ++t) {
                    const int64_t c0 = (static_cast<int64_t>(gl) + 64 * t) << 2;
                    const bool in = row < rows && c0 < cols;
                    // lanes outside re-read a nearby vector (one fixed address for all of them would be a hot spot)
                    const int64_t rr = row < rows ? row : rows - 1, cc = c0 < cols ? c0 : cols - 4;
                    const f32x4 a = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(x + rr * ldx + cc));
#pragma unroll
                    for (int k = 0; k < 4; ++k) v[u][t][k] = in ? a[k] : 0.0f;
                    if (MK == 1) {
                        const f32x4 b = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(mask + rr * ldm + cc));
#pragma unroll
                        for (int k = 0; k < 4; ++k) mk[u][t][k] = in ? b[k] : 1.0f;
                    }
                    if (MK == 2) {
                        const unsigned w = (reinterpret_cast<const uint16_t*>(mask) + rr * ldm)[cc >> 4];
                        wb[u][t] = in ? (w >> (cc & 15)) : 0xFu;
                    }
                }
            }
        } else {
            // Rows with a partial last quad, or without 16-byte alignment: the same unconditional loads from
            // clamped addresses, as wide as the layout allows (a quad of a padded row lies inside its pitch).
#pragma unroll
            for (int u = 0; u < RU; ++u) {
                const int64_t row = row0 + u * row_step;
                const int64_t rr = row < rows ? row : rows - 1;
                const float* xr = x + rr * ldx;
#pragma unroll
                for (int t = 0; t < T; ++t) {
                    const int64_t c0 = (static_cast<int64_t>(gl) + 64 * t) << 2;
                    const bool in0 = row < rows && c0 < cols;
                    if (XV == 4) {
                        const int64_t cc = c0 < cols ? c0 : ((cols - 1) & ~static_cast<int64_t>(3));
                        const f32x4 a = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(xr + cc));
#pragma unroll
                        for (int k = 0; k < 4; ++k) v[u][t][k] = (in0 && c0 + k < cols) ? a[k] : 0.0f;
                    } else if (XV == 2) {  // even columns and pitch: a pair lies inside the row or outside
                        typedef float f32x2 __attribute__((ext_vector_type(2)));
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            const int64_t c = c0 + 2 * h;
                            const f32x2 a = __builtin_nontemporal_load(reinterpret_cast<const f32x2*>(xr + (c < cols ? c : cols - 2)));
                            v[u][t][2 * h] = (row < rows && c < cols) ? a[0] : 0.0f;
                            v[u][t][2 * h + 1] = (row < rows && c + 1 < cols) ? a[1] : 0.0f;
                        }
                    } else {
                        const int cl = static_cast<int>(cols), cb = static_cast<int>(c0);  // cols <= 1024: 32-bit column math
                        const bool rin = row < rows;
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            const int c = cb + k;
                            const float a = xr[c < cl ? c : cl - 1];
                            v[u][t][k] = (rin && c < cl) ? a : 0.0f;
                        }
                    }
                    if (MK == 1) {
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            const int64_t c = c0 + k;
                            const float b = mask[rr * ldm + (c < cols ? c : cols - 1)];
                            mk[u][t][k] = (row < rows && c < cols) ? b : 1.0f;
                        }
                    }
                    if (MK == 2) {  // cols is a multiple of 16 here (checked by the caller)
                        const int64_t cc = c0 < cols ? c0 : cols - 4;
                        const unsigned w = (reinterpret_cast<const uint16_t*>(mask) + rr * ldm)[cc >> 4];
                        wb[u][t] = in0 ? (w >> (cc & 15)) : 0xFu;
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < RU; ++u) {  // rows are added in the order a one-row-at-a-time loop would take them
            const float rm = rmv[u];
#pragma unroll
            for (int t = 0; t < T; ++t)
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    float e = v[u][t][k];
                    if (MK == 1) e = masked(e, mk[u][t][k], mask_mode);
                    if (MK == 2) e = ((wb[u][t] >> k) & 1u) ? e : 0.0f;
                    cs[t][k] += e;
                    m = fmaxf(m, fabsf(row_mul ? e * rm : e));
                }
        }
    }
    if (partial) {  // fold the block's four wavefronts in a fixed order, one partial row per block
        // first the rows a wavefront handled side by side (lanes that differ only in `sub`)
        for (int off = gpr; off < kWave; off <<= 1) {
#pragma unroll
            for (int t = 0; t < T; ++t)
#pragma unroll
                for (int k = 0; k < 4; ++k) cs[t][k] += __shfl_xor(cs[t][k], off, kWave);
        }
        if (threadIdx.y > 0) {
#pragma unroll
            for (int t = 0; t < T; ++t)
#pragma unroll
                for (int k = 0; k < 4; ++k) red[threadIdx.y - 1][(t * 4 + k) * 64 + threadIdx.x] = cs[t][k];
        }
        __syncthreads();
        if (threadIdx.y == 0) {
            float* prow = partial + static_cast<int64_t>(blockIdx.x) * cols;
#pragma unroll
            for (int t = 0; t < T; ++t) {
                const int64_t c0 = (static_cast<int64_t>(threadIdx.x) + 64 * t) << 2;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int i = (t * 4 + k) * 64 + threadIdx.x;
                    const float v = ((cs[t][k] + red[0][i]) + red[1][i]) + red[2][i];
                    if (c0 + k < cols) prow[c0 + k] = v;
                }
            }
        }
    }
    block_absmax_to_global(m / 127.0f, scale_out);
}

// blockDim = (16, 64): 16 columns per block; thread (x, y) sums partial rows y, y + 64, ... with four loads in
// flight (a thousand lanes per block: the partial rows are few, and each step is one memory round trip); the
// sixty-four sums of a column are then added in a fixed order.
__global__ __launch_bounds__(1024) void colsum_finish_kernel(const float* __restrict__ partial,
                                                             int64_t nrows, int64_t cols,
                                                             float* __restrict__ out) {
    constexpr int RY = 64;
    __shared__ float red[RY][16];
    const int64_t c = static_cast<int64_t>(blockIdx.x) * 16 + threadIdx.x;
    float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
    if (c < cols) {
        int64_t r = threadIdx.y;
        for (; r + 3 * RY < nrows; r += 4 * RY) {
            a0 += partial[r * cols + c];
            a1 += partial[(r + RY) * cols + c];
            a2 += partial[(r + 2 * RY) * cols + c];
            a3 += partial[(r + 3 * RY) * cols + c];
        }
        for (; r < nrows; r += RY) a0 += partial[r * cols + c];
    }
    red[threadIdx.y][threadIdx.x] = (a0 + a1) + (a2 + a3);
    __syncthreads();
    if (threadIdx.y == 0 && c < cols) {
        float s = 0.0f;
#pragma unroll
        for (int y = 0; y < RY; ++y) s += red[y][threadIdx.x];
        out[c] = s;
    }
}

template <typename F>
static int dispatch_mode(int mode, F&& f) {
    switch (mode) {
        case TANGO_ROUND_RNE: f(std::integral_constant<int, TANGO_ROUND_RNE>{}); return TANGO_OK;
        case TANGO_ROUND_TRUNC: f(std::integral_constant<int, TANGO_ROUND_TRUNC>{}); return TANGO_OK;
        case TANGO_ROUND_STOCHASTIC:
            f(std::integral_constant<int, TANGO_ROUND_STOCHASTIC>{});
            return TANGO_OK;
        default: return TANGO_ERR_UNSUPPORTED;
    }
}

}  // namespace tango

using namespace tango;

extern "C" {

const char* tango_status_string(int status) {
    switch (status) {
        case TANGO_OK: return "ok";
        case TANGO_ERR_INVALID_ARG: return "invalid argument";
        case TANGO_ERR_UNSUPPORTED: return "unsupported op, mode or shape";
        case TANGO_ERR_LAUNCH: return "kernel launch failed";
        case TANGO_ERR_WORKSPACE: return "workspace missing or too small";
        case TANGO_ERR_STATIC_LIMIT: return "input too large for the fixed scratch of the entry point that allocates nothing";
        default: return "unknown status";
    }
}

int tango_abi_version(void) { return 3; }

int tango_absmax_f32(const float* x, int64_t n, float* scale_out, tango_stream_t stream) {
    if (!scale_out || n < 0 || (n > 0 && !x)) return TANGO_ERR_INVALID_ARG;
    if ((reinterpret_cast<uintptr_t>(x) & 3) != 0) return TANGO_ERR_INVALID_ARG;
    hipStream_t s = as_stream(stream);
    if (n <= (1 << 16)) {
        hipLaunchKernelGGL(absmax_small_kernel, dim3(1), dim3(1024), 0, s, x, n, scale_out);
        return launch_status();
    }
    fill_u32(scale_out, 0u, 1, s);
    const int64_t head = ((16 - (reinterpret_cast<uintptr_t>(x) & 15)) & 15) >> 2;
    // two workgroups per CU: every workgroup ends with one atomic on the same address, and those
    // serialise (561 MB: 98 us with eight per CU, 81 us with two; 87 MB: 33 -> 17 us)
    const int grid = grid_for(n / 16, 256, 2);
    hipLaunchKernelGGL(absmax_kernel, dim3(grid), dim3(256), 0, s, x, n, head, scale_out);
    return launch_status();
}

int tango_absmax_acc_f32(const float* x, int64_t n, float* scale_acc, tango_stream_t stream) {
    if (!scale_acc || n < 0 || (n > 0 && !x)) return TANGO_ERR_INVALID_ARG;
    if ((reinterpret_cast<uintptr_t>(x) & 3) != 0) return TANGO_ERR_INVALID_ARG;
    if (n == 0) return TANGO_OK;
    int64_t head = ((16 - (reinterpret_cast<uintptr_t>(x) & 15)) & 15) >> 2;
    if (head > n) head = n;
    const int grid = grid_for(n / 16 + 1, 256, 2);
    hipLaunchKernelGGL(absmax_kernel, dim3(grid), dim3(256), 0, as_stream(stream), x, n, head, scale_acc);
    return launch_status();
}

int tango_absmax_rows_f32(const float* x, int64_t rows, int64_t cols, int64_t ldx,
                          float* scale_out, tango_stream_t stream) {
    if (rows < 0 || cols < 0 || ldx < cols || (rows > 0 && (!x || !scale_out)))
        return TANGO_ERR_INVALID_ARG;
    if (rows == 0) return TANGO_OK;
    const int64_t blocks = ceil_div(rows, 4);
    if (blocks > INT32_MAX) return TANGO_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(absmax_rows_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       as_stream(stream), x, rows, cols, ldx, scale_out);
    return launch_status();
}

static int absmax_ex_grid(int64_t rows) {
    const int64_t blocks = ceil_div(rows, 4);
    return static_cast<int>(blocks < 1024 ? (blocks < 1 ? 1 : blocks) : 1024);
}

size_t tango_absmax_ex_workspace(int64_t rows, int64_t cols, int want_colsum) {
    if (!want_colsum || rows <= 0 || cols <= 0) return 0;
    return static_cast<size_t>(absmax_ex_grid(rows)) * static_cast<size_t>(cols) * sizeof(float);
}

int tango_absmax_ex_f32(const float* x, int64_t rows, int64_t cols, int64_t ldx, const float* row_mul,
                        const void* mask_, int64_t ldm, int mask_mode, float* scale_out, int accumulate,
                        float* colsum_out, void* workspace, size_t workspace_bytes, tango_stream_t stream) {
    const float* mask = static_cast<const float*>(mask_);  // 16-bit words in mode 2
    if (rows < 0 || cols < 0 || ldx < cols || !scale_out || (rows * cols > 0 && !x) ||
        (mask && ldm < (mask_mode == 2 ? cols / 16 : cols)))
        return TANGO_ERR_INVALID_ARG;
    if (cols > 1024 || mask_mode < 0 || mask_mode > 2 || (mask && mask_mode == 2 && (cols & 15) != 0))
        return TANGO_ERR_UNSUPPORTED;
    hipStream_t s = as_stream(stream);
    if (!accumulate) fill_u32(scale_out, 0u, 1, s);
    const int grid = absmax_ex_grid(rows);
    float* partial = nullptr;
    if (colsum_out) {
        const size_t need = tango_absmax_ex_workspace(rows > 0 ? rows : 1, cols, 1);
        if (cols > 0 && (!workspace || workspace_bytes < need)) return TANGO_ERR_WORKSPACE;
        partial = static_cast<float*>(workspace);
    }
    if (cols == 0) return launch_status();
    if (row_mul && !mask && !colsum_out && ldx == cols && (cols & 1) == 0 && (cols & 3) != 0 &&
        (reinterpret_cast<uintptr_t>(x) & 15) == 0 && rows * cols >= (1 << 16)) {
        // rows of 8-byte alignment only: the flat walk reads them with 16-byte loads all the same
        const int64_t n = rows * cols;
        hipLaunchKernelGGL(absmax_rowmul_dense_kernel, dim3(grid_for(n / 16, 256, 2)), dim3(256), 0, s, x, n, cols,
                           row_mul, scale_out);
        return launch_status();
    }
    const dim3 block(64, 4);
    const int T = static_cast<int>(ceil_div(cols, 256));
    int gpr_log2 = 6;
    const int64_t cgroups = ceil_div(cols, 4);
    while (gpr_log2 > 0 && (1LL << (gpr_log2 - 1)) >= cgroups) --gpr_log2;
    const uintptr_t xa = reinterpret_cast<uintptr_t>(x);
    const int xv = ((xa & 15) == 0 && (ldx & 3) == 0) ? 4 : ((xa & 7) == 0 && (ldx & 1) == 0) ? 2 : 1;
#define TANGO_AEX_M(T_, V_, M_)                                                                             \
    hipLaunchKernelGGL((absmax_ex_kernel<T_, V_, M_>), dim3(grid), block, 0, s, x, rows, cols, ldx, row_mul, \
                       mask, ldm, scale_out, partial, gpr_log2, mask_mode)
#define TANGO_AEX(T_, V_)                                                                   \
    do {                                                                                    \
        if (!mask) TANGO_AEX_M(T_, V_, 0); else if (mask_mode == 2) TANGO_AEX_M(T_, V_, 2); \
        else TANGO_AEX_M(T_, V_, 1);                                                        \
    } while (0)
#define TANGO_AEX_T(T_)                                                              \
    do {                                                                             \
        if (xv == 4) TANGO_AEX(T_, 4); else if (xv == 2) TANGO_AEX(T_, 2); else TANGO_AEX(T_, 1); \
    } while (0)
    if (T <= 1) TANGO_AEX_T(1); else if (T == 2) TANGO_AEX_T(2); else if (T == 3) TANGO_AEX_T(3); else TANGO_AEX_T(4);
#undef TANGO_AEX_T
#undef TANGO_AEX
#undef TANGO_AEX_M
    if (colsum_out)
        hipLaunchKernelGGL(colsum_finish_kernel, dim3(static_cast<unsigned>(ceil_div(cols, 16))), dim3(16, 64), 0,
                           s, partial, static_cast<int64_t>(grid), cols, colsum_out);
    return launch_status();
}

// counter[0] += inc, one thread (a kernel rather than a host-side update, so that a captured graph advances the
// stream of random numbers on every replay)
static __global__ void counter_add_kernel(uint64_t* counter, uint64_t inc) { counter[0] += inc; }

int tango_counter_add_u64(uint64_t* counter, uint64_t inc, tango_stream_t stream) {
    if (!counter || (reinterpret_cast<uintptr_t>(counter) & 7) != 0) return TANGO_ERR_INVALID_ARG;
    hipLaunchKernelGGL(counter_add_kernel, dim3(1), dim3(1), 0, as_stream(stream), counter, inc);
    return launch_status();
}

int tango_quantize_f32_i8(const float* x, int64_t n, const float* scale, int8_t* q,
                          int round_mode, const float* noise, uint64_t seed, uint64_t offset,
                          const uint64_t* offset_dev, tango_stream_t stream) {
    if (n < 0 || !scale || (n > 0 && (!x || !q))) return TANGO_ERR_INVALID_ARG;
    if (n == 0) return (round_mode >= 0 && round_mode <= 2) ? TANGO_OK : TANGO_ERR_UNSUPPORTED;
    hipStream_t s = as_stream(stream);
    const bool vec = (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(q) & 3) == 0;
    int rc = dispatch_mode(round_mode, [&](auto mode) {
        constexpr int M = decltype(mode)::value;
        if (vec) {
            hipLaunchKernelGGL(quantize_vec_kernel<M>, dim3(grid_for(ceil_div(n, 4), 256)), dim3(256),
                               0, s, x, n, scale, q, noise, seed, offset, offset_dev);
        } else {
            hipLaunchKernelGGL(quantize_scalar_kernel<M>, dim3(grid_for(n, 256)), dim3(256), 0, s, x,
                               n, scale, q, noise, seed, offset, offset_dev);
        }
    });
    return rc != TANGO_OK ? rc : launch_status();
}

int tango_quantize_rows_f32_i8(const float* x, int64_t rows, int64_t cols, int64_t ldx,
                               const float* scale, int per_row, int8_t* q, int64_t ldq,
                               int round_mode, const float* noise, uint64_t seed,
                               uint64_t offset, tango_stream_t stream) {
    return tango_quantize_rows_ex_f32_i8(x, rows, cols, ldx, nullptr, nullptr, 0, 0, scale, per_row, q, ldq,
                                         round_mode, noise, seed, offset, nullptr, stream);
}

int tango_quantize_rows_ex_f32_i8(const float* x, int64_t rows, int64_t cols, int64_t ldx,
                                  const float* row_mul, const void* mask_, int64_t ldm, int mask_mode,
                                  const float* scale, int per_row, int8_t* q, int64_t ldq,
                                  int round_mode, const float* noise, uint64_t seed,
                                  uint64_t offset, const uint64_t* offset_dev, tango_stream_t stream) {
    const float* mask = static_cast<const float*>(mask_);  // 16-bit words in mode 2
    if (mask && ldm < (mask_mode == 2 ? cols / 16 : cols)) return TANGO_ERR_INVALID_ARG;
    if (mask_mode < 0 || mask_mode > 2 || (mask && mask_mode == 2 && (cols & 15) != 0)) return TANGO_ERR_UNSUPPORTED;
    if (rows < 0 || cols < 0 || ldx < cols || ldq < cols || !scale ||
        (rows * cols > 0 && (!x || !q)))
        return TANGO_ERR_INVALID_ARG;
    if (rows == 0 || ldq == 0) return (round_mode >= 0 && round_mode <= 2) ? TANGO_OK : TANGO_ERR_UNSUPPORTED;
    hipStream_t s = as_stream(stream);
    if ((row_mul || mask) && !per_row && cols > 0 && (cols & 3) == 0 && ldx == cols && ldq == cols &&
        (!mask || ldm == (mask_mode == 2 ? cols / 16 : cols)) && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
        (reinterpret_cast<uintptr_t>(mask) & (mask_mode == 2 ? 1 : 15)) == 0 && (reinterpret_cast<uintptr_t>(q) & 3) == 0) {
        const int64_t n4 = rows * (cols >> 2);
        int rc = dispatch_mode(round_mode, [&](auto mode) {
            constexpr int M = decltype(mode)::value;
            hipLaunchKernelGGL(quantize_dense_ex_kernel<M>, dim3(grid_for(n4, 256)), dim3(256), 0, s, x, n4, cols, scale,
                               q, noise, seed, offset, offset_dev, row_mul, mask, mask_mode, static_cast<float*>(nullptr));
        });
        return rc != TANGO_OK ? rc : launch_status();
    }
    if (!mask && !per_row && (cols & 3) != 0 && cols <= 128 && ldx == cols && rows * cols >= (1 << 16) &&
        (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (ldq & 15) == 0 && (reinterpret_cast<uintptr_t>(q) & 15) == 0 &&
        4 * (256 / cols) * ldq <= 32768) {
        const int R = 4 * (256 / static_cast<int>(cols));  // rows per workgroup: R * cols <= 1024 dense elements
        const size_t lds = static_cast<size_t>(R) * static_cast<size_t>(ldq);
        int rc = dispatch_mode(round_mode, [&](auto mode) {
            constexpr int M = decltype(mode)::value;
            hipLaunchKernelGGL(quantize_tile_rows_kernel<M>, dim3(grid_for(ceil_div(rows, R), 1, 16)), dim3(256), lds, s, x,
                               rows, static_cast<int>(cols), scale, q, static_cast<int>(ldq), R, noise, seed, offset,
                               offset_dev, row_mul);
        });
        return rc != TANGO_OK ? rc : launch_status();
    }
    if (!mask && !per_row && (cols & 3) != 0 && ldx == cols && rows * cols >= (1 << 16) &&
        (reinterpret_cast<uintptr_t>(x) & 15) == 0) {
        const int64_t n = rows * cols;
        int rc = dispatch_mode(round_mode, [&](auto mode) {
            constexpr int M = decltype(mode)::value;
            hipLaunchKernelGGL(quantize_flat_rows_kernel<M>, dim3(grid_for(n >> 2, 256)), dim3(256), 0, s, x, n, cols,
                               scale, q, ldq, noise, seed, offset, offset_dev, row_mul);
        });
        return rc != TANGO_OK ? rc : launch_status();
    }
    const int64_t groups = (ldq + 3) >> 2;
    int gpr_log2 = 6;
    while (gpr_log2 > 0 && (1LL << (gpr_log2 - 1)) >= groups) --gpr_log2;
    const int64_t blocks = ceil_div(rows, 4 * (64 >> gpr_log2));
    const dim3 grid(static_cast<unsigned>(blocks < 256 * 16 ? (blocks < 1 ? 1 : blocks) : 256 * 16)), block(64, 4);
    const uintptr_t xa = reinterpret_cast<uintptr_t>(x);
    const int xv = ((xa & 15) == 0 && (ldx & 3) == 0) ? 4 : ((xa & 7) == 0 && (ldx & 1) == 0) ? 2 : 1;
    int rc = dispatch_mode(round_mode, [&](auto mode) {
        constexpr int M = decltype(mode)::value;
        if (xv == 4)
            hipLaunchKernelGGL((quantize_rows_kernel<M, 4>), grid, block, 0, s, x, rows, cols, ldx, scale,
                               per_row, q, ldq, noise, seed, offset, offset_dev, row_mul, mask, ldm, gpr_log2, mask_mode);
        else if (xv == 2)
            hipLaunchKernelGGL((quantize_rows_kernel<M, 2>), grid, block, 0, s, x, rows, cols, ldx, scale,
                               per_row, q, ldq, noise, seed, offset, offset_dev, row_mul, mask, ldm, gpr_log2, mask_mode);
        else
            hipLaunchKernelGGL((quantize_rows_kernel<M, 1>), grid, block, 0, s, x, rows, cols, ldx, scale,
                               per_row, q, ldq, noise, seed, offset, offset_dev, row_mul, mask, ldm, gpr_log2, mask_mode);
    });
    return rc != TANGO_OK ? rc : launch_status();
}

size_t tango_quantize_rows_colsum_workspace(int64_t rows, int64_t cols) {
    if (rows <= 0 || cols <= 0) return 0;
    return static_cast<size_t>(grid_for(rows * (cols >> 2), 256)) * static_cast<size_t>(cols) * sizeof(float);
}

int tango_quantize_rows_colsum_f32_i8(const float* x, int64_t rows, int64_t cols, const float* row_mul,
                                      const void* mask_, int mask_mode, const float* scale, int8_t* q,
                                      int round_mode, const float* noise, uint64_t seed, uint64_t offset,
                                      const uint64_t* offset_dev, float* colsum_out, void* workspace,
                                      size_t workspace_bytes, tango_stream_t stream) {
    const float* mask = static_cast<const float*>(mask_);  // 16-bit words in mode 2
    if (rows < 0 || cols < 0 || !scale || !colsum_out || (rows * cols > 0 && (!x || !q))) return TANGO_ERR_INVALID_ARG;
    if (mask_mode < 0 || mask_mode > 2 || round_mode < 0 || round_mode > 2) return TANGO_ERR_UNSUPPORTED;
    // dense rows of 4, 8, ..., 1024 columns whose quads divide a workgroup's 256 lanes; sign words need whole words
    const int64_t quads = cols >> 2;
    if (rows == 0 || cols == 0 || (cols & 3) != 0 || quads > 256 || 256 % quads != 0 ||
        (mask && mask_mode == 2 && (cols & 15) != 0) || (reinterpret_cast<uintptr_t>(x) & 15) != 0 ||
        (reinterpret_cast<uintptr_t>(mask) & (mask_mode == 2 ? 1 : 15)) != 0 || (reinterpret_cast<uintptr_t>(q) & 3) != 0)
        return TANGO_ERR_UNSUPPORTED;
    const size_t need = tango_quantize_rows_colsum_workspace(rows, cols);
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 3) != 0) return TANGO_ERR_WORKSPACE;
    hipStream_t s = as_stream(stream);
    const int64_t n4 = rows * quads;
    const int grid = grid_for(n4, 256);
    float* partial = static_cast<float*>(workspace);
    int rc = dispatch_mode(round_mode, [&](auto mode) {
        constexpr int M = decltype(mode)::value;
        hipLaunchKernelGGL((quantize_dense_ex_kernel<M, true>), dim3(grid), dim3(256), 0, s, x, n4, cols, scale, q, noise,
                           seed, offset, offset_dev, row_mul, mask, mask_mode, partial);
    });
    if (rc != TANGO_OK) return rc;
    hipLaunchKernelGGL(colsum_finish_kernel, dim3(static_cast<unsigned>(ceil_div(cols, 16))), dim3(16, 64), 0, s,
                       partial, static_cast<int64_t>(grid), cols, colsum_out);
    return launch_status();
}

int tango_transpose_quant_f32_i8(const float* x, int64_t nrow, int64_t ncol, const float* scale,
                                 int8_t* out, tango_stream_t stream) {
    if (nrow < 0 || ncol < 0 || !scale || (nrow * ncol > 0 && (!x || !out)))
        return TANGO_ERR_INVALID_ARG;
    if (nrow * ncol == 0) return TANGO_OK;
    hipLaunchKernelGGL(transpose_quant_kernel, dim3(grid_for(ceil_div(nrow, 4), 256)), dim3(256), 0,
                       as_stream(stream), x, nrow, ncol, scale, out);
    return launch_status();
}

}  // extern "C"
