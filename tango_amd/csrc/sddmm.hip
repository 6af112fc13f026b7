// Quantized SDDMM for gfx950: per-edge dot products and element-wise ops on
// int8 node features gathered by (src, dst).
//
// Edge-parallel and memory-bound (two gathered rows + 16 index bytes in, H or
// T floats out per edge); no MFMA.  One lane owns one (edge, head) pair of the
// dot product, so the lanes of an edge read consecutive D-byte chunks of the
// two rows and write consecutive floats; the reduction over D runs inside the
// lane with v_dot4 on 16-, 4- or 1-byte loads and needs no cross-lane step
// (the reference spends a 32-lane shuffle tree per head on byte loads,
// cuda/src/SDDMM.cu:25-34).
#include "common.hpp"

namespace tango {

template <int VEC, bool REDUCE>
__global__ __launch_bounds__(256) void sddmm_dot_kernel(
    float* __restrict__ out, float* __restrict__ scale_out, const int64_t* __restrict__ src,
    const int64_t* __restrict__ dst, const int8_t* __restrict__ U, const int8_t* __restrict__ V,
    const float* __restrict__ sU, const float* __restrict__ sV, int64_t E, int H, int D) {
    const float s = sU[0] * sV[0];
    const int64_t total = E * H;
    const int64_t nthr = static_cast<int64_t>(gridDim.x) * blockDim.x;
    float m = 0.0f;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += nthr) {
        const int64_t e = i / H;
        const int h = static_cast<int>(i - e * H);
        const int8_t* u = U + (src[e] * H + h) * D;
        const int8_t* v = V + (dst[e] * H + h) * D;
        int acc = 0;
        if (VEC == 16) {
            for (int d = 0; d < D; d += 16) {
                const u32x4 a = *reinterpret_cast<const u32x4*>(u + d);
                const u32x4 b = *reinterpret_cast<const u32x4*>(v + d);
                acc = __builtin_amdgcn_sdot4(a.x, b.x, acc, false);
                acc = __builtin_amdgcn_sdot4(a.y, b.y, acc, false);
                acc = __builtin_amdgcn_sdot4(a.z, b.z, acc, false);
                acc = __builtin_amdgcn_sdot4(a.w, b.w, acc, false);
            }
        } else if (VEC == 4) {
            for (int d = 0; d < D; d += 4)
                acc = __builtin_amdgcn_sdot4(*reinterpret_cast<const int*>(u + d),
                                             *reinterpret_cast<const int*>(v + d), acc, false);
        } else {
            for (int d = 0; d < D; ++d) acc += static_cast<int>(u[d]) * static_cast<int>(v[d]);
        }
        const float y = static_cast<float>(acc) * s;
        __builtin_nontemporal_store(y, out + i);
        if (REDUCE) m = fmaxf(m, fabsf(y));
    }
    if (REDUCE) block_absmax_to_global(m / 127.0f, scale_out);
}

// The dot product when an edge's H * D bytes are a power of two of at most 1 KB (D = 16 * LPH): the 64 lanes of a
// wavefront hold 64 / (H * LPH) whole edges, a lane's place inside its edge never changes, and the edge index is
// wave-uniform arithmetic, so the loop carries no division (the kernels below divide a 64-bit index by a run-time
// value per element, which costs more instructions than the dot product itself).  Four groups of edges per
// iteration: the index loads of all four, then the eight row loads, are in flight together.  Every load is
// unconditional (edges past the end read the last edge again and store nothing).
template <int LPH, bool REDUCE>
__global__ __launch_bounds__(256) void sddmm_dot_wave_kernel(
    float* __restrict__ out, float* __restrict__ scale_out, const int64_t* __restrict__ src,
    const int64_t* __restrict__ dst, const int8_t* __restrict__ U, const int8_t* __restrict__ V,
    const float* __restrict__ sU, const float* __restrict__ sV, int64_t E, int H, int shift) {
    constexpr int UNR = 8;
    const float s = sU[0] * sV[0];
    const int lane = threadIdx.x & (kWave - 1);
    const int per = 1 << shift;            // lanes per edge = H * LPH
    const int epw = kWave >> shift;        // edges per wavefront and group
    const int sub = lane >> shift;         // the lane's edge inside a group
    const int r = lane & (per - 1);        // the lane's 16-byte piece of the edge's row
    const bool writer = (r & (LPH - 1)) == 0;
    const int head = r / LPH;
    const int64_t wave = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) >> 6;
    const int64_t waves = (static_cast<int64_t>(gridDim.x) * blockDim.x) >> 6;
    const int64_t step = static_cast<int64_t>(epw) * UNR;
    float m = 0.0f;
    for (int64_t base = wave * step; base < E; base += waves * step) {
        int64_t e[UNR], su[UNR], dv[UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            e[u] = base + u * epw + sub;
            const int64_t ec = e[u] < E ? e[u] : E - 1;
            su[u] = src[ec];
            dv[u] = dst[ec];
        }
        u32x4 a[UNR], b[UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            a[u] = *reinterpret_cast<const u32x4*>(U + (((su[u] << shift) + r) << 4));
            b[u] = *reinterpret_cast<const u32x4*>(V + (((dv[u] << shift) + r) << 4));
        }
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            int acc = __builtin_amdgcn_sdot4(a[u].x, b[u].x, 0, false);
            acc = __builtin_amdgcn_sdot4(a[u].y, b[u].y, acc, false);
            acc = __builtin_amdgcn_sdot4(a[u].z, b[u].z, acc, false);
            acc = __builtin_amdgcn_sdot4(a[u].w, b[u].w, acc, false);
#pragma unroll
            for (int off = 1; off < LPH; off <<= 1) acc += __shfl_xor(acc, off, kWave);
            if (writer && e[u] < E) {
                const float y = static_cast<float>(acc) * s;
                __builtin_nontemporal_store(y, out + e[u] * H + head);
                if (REDUCE) m = fmaxf(m, fabsf(y));
            }
        }
    }
    if (REDUCE) block_absmax_to_global(m / 127.0f, scale_out);
}

// Heads wider than 16 bytes (D = 16 * LPH, LPH a power of two): LPH consecutive lanes share one
// (edge, head) pair, each with 16 bytes of it, so the lanes of an edge read its two rows as
// contiguous runs; the partial dot products meet with xor-shuffles.  (With one lane per head and
// D = 64, the lanes of a wavefront would read 64 separate 16-byte pieces per load instruction.)
template <int LPH, bool REDUCE>
__global__ __launch_bounds__(256) void sddmm_dot_split_kernel(
    float* __restrict__ out, float* __restrict__ scale_out, const int64_t* __restrict__ src,
    const int64_t* __restrict__ dst, const int8_t* __restrict__ U, const int8_t* __restrict__ V,
    const float* __restrict__ sU, const float* __restrict__ sV, int64_t E, int H) {
    const float s = sU[0] * sV[0];
    const int64_t per = static_cast<int64_t>(H) * LPH;  // lanes per edge; the row is per * 16 bytes
    const int64_t total = E * per;
    const int64_t nthr = static_cast<int64_t>(gridDim.x) * blockDim.x;
    float m = 0.0f;
    // every lane of a wavefront takes part in the shuffles: the loop bound is rounded up to whole wavefronts
    const int64_t total_up = (total + kWave - 1) & ~static_cast<int64_t>(kWave - 1);
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total_up; i += nthr) {
        int acc = 0;
        const bool ok = i < total;
        const int64_t e = ok ? i / per : 0;
        const int64_t r = ok ? i - e * per : 0;  // 16-byte piece of the row
        if (ok) {
            const u32x4 a = *reinterpret_cast<const u32x4*>(U + (src[e] * per + r) * 16);
            const u32x4 b = *reinterpret_cast<const u32x4*>(V + (dst[e] * per + r) * 16);
            acc = __builtin_amdgcn_sdot4(a.x, b.x, acc, false);
            acc = __builtin_amdgcn_sdot4(a.y, b.y, acc, false);
            acc = __builtin_amdgcn_sdot4(a.z, b.z, acc, false);
            acc = __builtin_amdgcn_sdot4(a.w, b.w, acc, false);
        }
#pragma unroll
        for (int off = 1; off < LPH; off <<= 1) acc += __shfl_xor(acc, off, kWave);
        if (ok && (r & (LPH - 1)) == 0) {
            const float y = static_cast<float>(acc) * s;
            __builtin_nontemporal_store(y, out + e * H + r / LPH);
            if (REDUCE) m = fmaxf(m, fabsf(y));
        }
    }
    if (REDUCE) block_absmax_to_global(m / 127.0f, scale_out);
}

template <int OP>
__device__ __forceinline__ float apply_op(float a, float b) {
    if (OP == TANGO_OP_ADD) return a + b;
    if (OP == TANGO_OP_SUB) return a - b;
    if (OP == TANGO_OP_MUL) return a * b;
    return a / b;
}

// One lane owns VEC consecutive outputs of one edge.
template <int OP, int VEC, bool REDUCE>
__global__ __launch_bounds__(256) void sddmm_ewise_kernel(
    float* __restrict__ out, float* __restrict__ scale_out, const int64_t* __restrict__ src,
    const int64_t* __restrict__ dst, const int8_t* __restrict__ U, const int8_t* __restrict__ V,
    const float* __restrict__ sU, const float* __restrict__ sV, int64_t E, int64_t T) {
    const float su = sU[0], sv = sV[0];
    const int64_t per = T / VEC;  // VEC divides T
    const int64_t total = E * per;
    const int64_t nthr = static_cast<int64_t>(gridDim.x) * blockDim.x;
    float m = 0.0f;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += nthr) {
        const int64_t e = i / per;
        const int64_t t = (i - e * per) * VEC;
        const int8_t* u = U + src[e] * T + t;
        const int8_t* v = V + dst[e] * T + t;
        if (VEC == 4) {
            const int a = *reinterpret_cast<const int*>(u);
            const int b = *reinterpret_cast<const int*>(v);
            f32x4 y;
            y.x = apply_op<OP>(static_cast<float>(static_cast<int8_t>(a)) * su,
                               static_cast<float>(static_cast<int8_t>(b)) * sv);
            y.y = apply_op<OP>(static_cast<float>(static_cast<int8_t>(a >> 8)) * su,
                               static_cast<float>(static_cast<int8_t>(b >> 8)) * sv);
            y.z = apply_op<OP>(static_cast<float>(static_cast<int8_t>(a >> 16)) * su,
                               static_cast<float>(static_cast<int8_t>(b >> 16)) * sv);
            y.w = apply_op<OP>(static_cast<float>(a >> 24) * su, static_cast<float>(b >> 24) * sv);
            __builtin_nontemporal_store(y, reinterpret_cast<f32x4*>(out + e * T + t));
            if (REDUCE) m = fmaxf(m, fmaxf(fmaxf(fabsf(y.x), fabsf(y.y)), fmaxf(fabsf(y.z), fabsf(y.w))));
        } else {
            const float y = apply_op<OP>(static_cast<float>(u[0]) * su, static_cast<float>(v[0]) * sv);
            out[e * T + t] = y;
            if (REDUCE) m = fmaxf(m, fabsf(y));
        }
    }
    if (REDUCE) block_absmax_to_global(m / 127.0f, scale_out);
}

// As sddmm_ewise_kernel with fp32 operands quantized as they are loaded (round to nearest even or
// truncation with the given scales): the same int8 values a separate quantize pass would have stored, so
// the same result, without that pass and its int8 copies.
template <int OP, int VEC, int MODE>
__global__ __launch_bounds__(256) void sddmm_ewise_f32q_kernel(
    float* __restrict__ out, const int64_t* __restrict__ src, const int64_t* __restrict__ dst,
    const float* __restrict__ U, const float* __restrict__ V, const float* __restrict__ sU,
    const float* __restrict__ sV, int64_t E, int64_t T) {
    const float su = sU[0], sv = sV[0];
    const float ru = rscale_of(su), rv = rscale_of(sv);
    const int64_t per = T / VEC;  // VEC divides T
    const int64_t total = E * per;
    const int64_t nthr = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += nthr) {
        const int64_t e = i / per;
        const int64_t t = (i - e * per) * VEC;
        const float* u = U + src[e] * T + t;
        const float* v = V + dst[e] * T + t;
        if (VEC == 4) {
            const f32x4 a = *reinterpret_cast<const f32x4*>(u);
            const f32x4 b = *reinterpret_cast<const f32x4*>(v);
            f32x4 y;
#pragma unroll
            for (int k = 0; k < 4; ++k)
                y[k] = apply_op<OP>(static_cast<float>(quant_one<MODE>(a[k], ru, 0.0f)) * su,
                                    static_cast<float>(quant_one<MODE>(b[k], rv, 0.0f)) * sv);
            __builtin_nontemporal_store(y, reinterpret_cast<f32x4*>(out + e * T + t));
        } else {
            out[e * T + t] = apply_op<OP>(static_cast<float>(quant_one<MODE>(u[0], ru, 0.0f)) * su,
                                          static_cast<float>(quant_one<MODE>(v[0], rv, 0.0f)) * sv);
        }
    }
}

}  // namespace tango

using namespace tango;

extern "C" {

int tango_sddmm_dot_i8(float* out, float* scale_out, const int64_t* src, const int64_t* dst,
                       const int8_t* U, const int8_t* V, const float* sU, const float* sV,
                       int64_t num_edges, int64_t H, int64_t D, tango_stream_t stream) {
    if (num_edges < 0 || H < 0 || D < 0 || !sU || !sV ||
        (num_edges * H > 0 && (!out || !src || !dst || !U || !V)))
        return TANGO_ERR_INVALID_ARG;
    if (H >= (1LL << 31) || D >= (1LL << 31)) return TANGO_ERR_UNSUPPORTED;
    hipStream_t s = as_stream(stream);
    if (scale_out) fill_u32(scale_out, 0u, 1, s);
    const int64_t total = num_edges * H;
    if (total == 0) return launch_status();
    const uintptr_t al = reinterpret_cast<uintptr_t>(U) | reinterpret_cast<uintptr_t>(V);
    const int vec = ((D & 15) == 0 && (al & 15) == 0) ? 16 : ((D & 3) == 0 && (al & 3) == 0) ? 4 : 1;
    const int64_t lph = D / 16;
    const int64_t per = H * lph;  // lanes per edge with 16 bytes per lane
    if (vec == 16 && lph >= 1 && lph <= 16 && (lph & (lph - 1)) == 0 && per <= 64 && (per & (per - 1)) == 0 &&
        D == 16 * lph) {
        int shift = 0;
        while ((1 << shift) < per) ++shift;
        const int64_t groups = ceil_div(num_edges, (64 / per) * 8);  // wavefront iterations of four edge groups
        const dim3 wgrid(grid_for(groups * 64, 256, 16)), wblock(256);
#define TANGO_DOT_WAVE(L_)                                                                                    \
    do {                                                                                                      \
        if (scale_out)                                                                                        \
            hipLaunchKernelGGL((sddmm_dot_wave_kernel<L_, true>), wgrid, wblock, 0, s, out, scale_out, src,   \
                               dst, U, V, sU, sV, num_edges, static_cast<int>(H), shift);                     \
        else                                                                                                  \
            hipLaunchKernelGGL((sddmm_dot_wave_kernel<L_, false>), wgrid, wblock, 0, s, out, scale_out, src,  \
                               dst, U, V, sU, sV, num_edges, static_cast<int>(H), shift);                     \
    } while (0)
        if (lph == 1) TANGO_DOT_WAVE(1);
        else if (lph == 2) TANGO_DOT_WAVE(2);
        else if (lph == 4) TANGO_DOT_WAVE(4);
        else if (lph == 8) TANGO_DOT_WAVE(8);
        else TANGO_DOT_WAVE(16);
#undef TANGO_DOT_WAVE
        return launch_status();
    }
    if (vec == 16 && lph >= 2 && lph <= 16 && (lph & (lph - 1)) == 0) {
        const dim3 sgrid(grid_for(total * lph, 256, 16)), sblock(256);
#define TANGO_DOT_SPLIT(L_)                                                                                   \
    do {                                                                                                      \
        if (scale_out)                                                                                        \
            hipLaunchKernelGGL((sddmm_dot_split_kernel<L_, true>), sgrid, sblock, 0, s, out, scale_out, src,  \
                               dst, U, V, sU, sV, num_edges, static_cast<int>(H));                            \
        else                                                                                                  \
            hipLaunchKernelGGL((sddmm_dot_split_kernel<L_, false>), sgrid, sblock, 0, s, out, scale_out, src, \
                               dst, U, V, sU, sV, num_edges, static_cast<int>(H));                            \
    } while (0)
        if (lph == 2) TANGO_DOT_SPLIT(2);
        else if (lph == 4) TANGO_DOT_SPLIT(4);
        else if (lph == 8) TANGO_DOT_SPLIT(8);
        else TANGO_DOT_SPLIT(16);
#undef TANGO_DOT_SPLIT
        return launch_status();
    }
    const dim3 grid(grid_for(total, 256, 16)), block(256);
#define TANGO_DOT(V_, R_)                                                                         \
    hipLaunchKernelGGL((sddmm_dot_kernel<V_, R_>), grid, block, 0, s, out, scale_out, src, dst, U, \
                       V, sU, sV, num_edges, static_cast<int>(H), static_cast<int>(D))
    if (scale_out) {
        if (vec == 16) TANGO_DOT(16, true); else if (vec == 4) TANGO_DOT(4, true); else TANGO_DOT(1, true);
    } else {
        if (vec == 16) TANGO_DOT(16, false); else if (vec == 4) TANGO_DOT(4, false); else TANGO_DOT(1, false);
    }
#undef TANGO_DOT
    return launch_status();
}

int tango_sddmm_ewise_i8(int op, float* out, float* scale_out, const int64_t* src,
                         const int64_t* dst, const int8_t* U, const int8_t* V, const float* sU,
                         const float* sV, int64_t num_edges, int64_t T, tango_stream_t stream) {
    if (op < TANGO_OP_ADD || op > TANGO_OP_DIV) return TANGO_ERR_UNSUPPORTED;
    if (num_edges < 0 || T < 0 || !sU || !sV ||
        (num_edges * T > 0 && (!out || !src || !dst || !U || !V)))
        return TANGO_ERR_INVALID_ARG;
    hipStream_t s = as_stream(stream);
    if (scale_out) fill_u32(scale_out, 0u, 1, s);
    if (num_edges * T == 0) return launch_status();
    const uintptr_t al = reinterpret_cast<uintptr_t>(U) | reinterpret_cast<uintptr_t>(V);
    const bool v4 = (T & 3) == 0 && (al & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
    const dim3 grid(grid_for(num_edges * (v4 ? T / 4 : T), 256, 16)), block(256);
#define TANGO_EW(OP_, V_, R_)                                                                    \
    hipLaunchKernelGGL((sddmm_ewise_kernel<OP_, V_, R_>), grid, block, 0, s, out, scale_out, src, \
                       dst, U, V, sU, sV, num_edges, T)
#define TANGO_EW_OP(OP_)                                                  \
    do {                                                                  \
        if (scale_out) {                                                  \
            if (v4) TANGO_EW(OP_, 4, true); else TANGO_EW(OP_, 1, true);  \
        } else {                                                          \
            if (v4) TANGO_EW(OP_, 4, false); else TANGO_EW(OP_, 1, false);\
        }                                                                 \
    } while (0)
    switch (op) {
        case TANGO_OP_ADD: TANGO_EW_OP(TANGO_OP_ADD); break;
        case TANGO_OP_SUB: TANGO_EW_OP(TANGO_OP_SUB); break;
        case TANGO_OP_MUL: TANGO_EW_OP(TANGO_OP_MUL); break;
        default: TANGO_EW_OP(TANGO_OP_DIV); break;
    }
#undef TANGO_EW_OP
#undef TANGO_EW
    return launch_status();
}

int tango_sddmm_ewise_f32q(int op, float* out, const int64_t* src, const int64_t* dst, const float* U,
                           const float* V, const float* sU, const float* sV, int64_t num_edges, int64_t T,
                           int round_mode, tango_stream_t stream) {
    if (op < TANGO_OP_ADD || op > TANGO_OP_DIV) return TANGO_ERR_UNSUPPORTED;
    if (round_mode != TANGO_ROUND_RNE && round_mode != TANGO_ROUND_TRUNC) return TANGO_ERR_UNSUPPORTED;
    if (num_edges < 0 || T < 0 || !sU || !sV || (num_edges * T > 0 && (!out || !src || !dst || !U || !V)))
        return TANGO_ERR_INVALID_ARG;
    if (num_edges * T == 0) return TANGO_OK;
    const uintptr_t al = reinterpret_cast<uintptr_t>(U) | reinterpret_cast<uintptr_t>(V) |
                         reinterpret_cast<uintptr_t>(out);
    const bool v4 = (T & 3) == 0 && (al & 15) == 0;
    const dim3 grid(grid_for(num_edges * (v4 ? T / 4 : T), 256, 16)), block(256);
    hipStream_t s = as_stream(stream);
#define TANGO_EWQ(OP_, V_, M_)                                                                              \
    hipLaunchKernelGGL((sddmm_ewise_f32q_kernel<OP_, V_, M_>), grid, block, 0, s, out, src, dst, U, V, sU, \
                       sV, num_edges, T)
#define TANGO_EWQ_OP(OP_)                                                      \
    do {                                                                       \
        if (round_mode == TANGO_ROUND_RNE) {                                   \
            if (v4) TANGO_EWQ(OP_, 4, TANGO_ROUND_RNE);                        \
            else TANGO_EWQ(OP_, 1, TANGO_ROUND_RNE);                           \
        } else {                                                               \
            if (v4) TANGO_EWQ(OP_, 4, TANGO_ROUND_TRUNC);                      \
            else TANGO_EWQ(OP_, 1, TANGO_ROUND_TRUNC);                         \
        }                                                                      \
    } while (0)
    switch (op) {
        case TANGO_OP_ADD: TANGO_EWQ_OP(TANGO_OP_ADD); break;
        case TANGO_OP_SUB: TANGO_EWQ_OP(TANGO_OP_SUB); break;
        case TANGO_OP_MUL: TANGO_EWQ_OP(TANGO_OP_MUL); break;
        default: TANGO_EWQ_OP(TANGO_OP_DIV); break;
    }
#undef TANGO_EWQ_OP
#undef TANGO_EWQ
    return launch_status();
}

}  // extern "C"
