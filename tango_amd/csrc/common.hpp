// Shared device/host helpers for the gfx950 kernels of libtango_hip.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/tango_hip.h"

namespace tango {

constexpr int kWave = 64;

// Native vector types (the nontemporal builtins and MFMA operands need these,
// not HIP's float4/int4 structs).
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

inline hipStream_t as_stream(tango_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// Status of the launch just issued (configuration errors surface here; kernel
// faults surface at the caller's next synchronisation, as with any HIP code).
inline int launch_status() {
    return hipGetLastError() == hipSuccess ? TANGO_OK : TANGO_ERR_LAUNCH;
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Number of workgroups for a grid-stride kernel: enough to give every one of
// the 256 CUs several resident groups, never more than the work needs.
inline int grid_for(int64_t work_items, int threads, int groups_per_cu = 8) {
    int64_t need = ceil_div(work_items, threads);
    int64_t cap = 256LL * groups_per_cu;
    if (need < 1) need = 1;
    return static_cast<int>(need < cap ? need : cap);
}

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// Workgroup-wide maximum of non-negative floats followed by one integer
// atomicMax on the float's bit pattern (order-preserving for values >= 0).
// *out must hold 0 (or an earlier partial maximum) before the first arrival.
// Every thread of the workgroup must call this.
__device__ __forceinline__ void block_absmax_to_global(float v, float* out) {
    __shared__ float part[16];
    v = wave_max(v);
    const int nw = (blockDim.x * blockDim.y + kWave - 1) / kWave;
    const int tid = threadIdx.y * blockDim.x + threadIdx.x;
    const int w = tid / kWave;
    if ((tid & (kWave - 1)) == 0) part[w] = v;
    __syncthreads();
    if (w == 0) {
        float m = (tid < nw) ? part[tid] : 0.0f;
        m = wave_max(m);
        // Fire and forget.  Atomics on one address are served one at a time (some 15 ns each), in the
        // background of the kernel; reading the slot first to skip the atomic was tried, at the end of a
        // workgroup and at its start, and either way the coherent load of that hot address stalls the
        // workgroup for longer than the atomic costs.
        if (tid == 0) atomicMax(reinterpret_cast<int*>(out), __float_as_int(m));
    }
}

// 1/s with the convention that an all-zero tensor (s == 0) quantizes to zeros.
__device__ __forceinline__ float rscale_of(float s) { return s > 0.0f ? 1.0f / s : 0.0f; }

// fp32 -> int8 rounding shared by the quantize kernels and the GEMM's fused quantize.
// The rounded value goes through v_cvt_i32_f32 (toward zero, saturating, NaN -> 0: what the float-domain clamp and
// the NaN test before a C cast spelled out in four more instructions) and is clamped as an integer: three VALU
// instructions per element for truncation, four for half-to-even.
template <int MODE>
__device__ __forceinline__ int quant_one(float x, float r, float u) {
    const float p = x * r;
    float v;
    if (MODE == TANGO_ROUND_RNE)
        v = rintf(p);
    else if (MODE == TANGO_ROUND_TRUNC)
        v = p;  // the conversion below truncates
    else
        v = floorf(p + u);
    int q;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(q) : "v"(v));
    return q < -127 ? -127 : (q > 127 ? 127 : q);
}

// bytes (a, b, c, d) of four ints in [-128, 127] as one dword, three v_perm_b32
__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
    const uint32_t lo = __builtin_amdgcn_perm(static_cast<uint32_t>(b), static_cast<uint32_t>(a), 0x0c0c0400u);
    const uint32_t hi = __builtin_amdgcn_perm(static_cast<uint32_t>(d), static_cast<uint32_t>(c), 0x0c0c0400u);
    return __builtin_amdgcn_perm(hi, lo, 0x05040100u);
}

// 4x4 byte transpose with v_perm_b32: rows r0..r3 (one dword each) -> c[j] = bytes (r0[j], r1[j], r2[j], r3[j]).
__device__ __forceinline__ void transpose4x4(uint32_t r0, uint32_t r1, uint32_t r2, uint32_t r3,
                                             uint32_t* c) {
    const uint32_t t0 = __builtin_amdgcn_perm(r1, r0, 0x05010400u);
    const uint32_t t1 = __builtin_amdgcn_perm(r1, r0, 0x07030602u);
    const uint32_t t2 = __builtin_amdgcn_perm(r3, r2, 0x05010400u);
    const uint32_t t3 = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
    c[0] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
    c[1] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
    c[2] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
    c[3] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
}

// largest r in [0, rows) with indptr[r] <= key (indptr[0] = 0 <= key): 64 probes per round
__device__ __forceinline__ int64_t row_of_slot_wave(const int64_t* __restrict__ indptr, int64_t rows, int64_t key,
                                                    int lane) {
    int64_t lo = 0, hi = rows;  // the answer lies in [lo, hi)
    while (hi - lo > 1) {
        const int64_t step = (hi - lo + kWave - 1) >> 6;
        const int64_t probe = lo + lane * step;
        const bool ok = probe < hi && indptr[probe] <= key;
        const int cnt = __popcll(__ballot(ok));  // lane 0 always holds
        lo += (cnt - 1) * step;
        hi = lo + step < hi ? lo + step : hi;
    }
    return lo;
}

// Sets a handful of 32-bit words.  Used instead of hipMemsetAsync so that a
// caller may capture any entry point into a HIP graph.
static __global__ void fill_u32_kernel(uint32_t* p, uint32_t v, int n) {
    if (static_cast<int>(threadIdx.x) < n) p[threadIdx.x] = v;
}

inline void fill_u32(void* p, uint32_t v, int n, hipStream_t s) {
    hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(64), 0, s, static_cast<uint32_t*>(p), v, n);
}

}  // namespace tango
