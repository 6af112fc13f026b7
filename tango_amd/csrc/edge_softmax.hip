// LeakyReLU + per-destination edge softmax (forward and backward) for gfx950.
//
// fp32, memory-bound: e is read, a written, both [E, H] in edge-id order and
// reached through the destination-major CSR's edge-id permutation.  The work is cut
// by edge slots, not by rows: a wavefront owns a span of 256 consecutive slots of the
// destination-major order whatever rows they belong to, so a hub destination and a
// million destinations with three in-edges cost the same per edge.  Rows that lie
// inside one span are finished in one sweep (values stay in registers between the
// reduction and the write); a row cut by a span boundary leaves per-span partial
// results that a small second launch combines and a third writes out.  Without a
// workspace a thread-per-(row, head) kernel is used.
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

// ---------------------------------------------------------------------------------------------
// Span kernels.  Wavefront w owns slots [w * kSpan, (w + 1) * kSpan), lane l of step u holds slot
// base + 64 u + l with HB heads of it (head block blockIdx.y).  Per step, a segmented scan over
// the lanes (segments = rows) gives every lane its row's (max, sum of exp) within the step; rows
// running over a step boundary chain through a wave-uniform carry, and the lanes of their earlier
// steps pick the finished result up from `fin`.  Three kinds of row:
//   inside : starts and ends within the span -> written by this launch;
//   head   : started in an earlier span      -> partial result in piece 0 of the span's record;
//   tail   : runs on into the next span      -> partial result in piece 1.
// span_fix_kernel merges a row's pieces (the tail of the span it starts in and the heads of the
// spans that follow) and stores the row's result back into every piece; span_rest_kernel then
// writes the head and tail slots.  No atomics: results do not depend on scheduling.
constexpr int kSteps = 4;
constexpr int kSpan = kWave * kSteps;
constexpr int kWin = kSpan + kWave;  // row pointers staged per wavefront: 64 empty rows of slack

struct SpanMeta {
    int64_t head_end;    // slots [base, head_end) belong to a row that started before the span
    int64_t tail_start;  // slots [tail_start, end) belong to a row that runs on after the span
    int64_t head_open;   // the head row also runs on after the span (then there is no tail)
};

__host__ __device__ inline size_t span_vals_offset(int64_t nspans) {
    return (static_cast<size_t>(nspans) * sizeof(SpanMeta) + 255) & ~static_cast<size_t>(255);
}
// vals[span][piece][component][H]: component 0 = max, 1 = sum (backward: only the sum)
__device__ __forceinline__ float* span_vals(void* ws, int64_t nspans, int64_t w, int piece, int comp, int H) {
    return reinterpret_cast<float*>(static_cast<char*>(ws) + span_vals_offset(nspans)) +
           ((w * 2 + piece) * 2 + comp) * static_cast<int64_t>(H);
}

__device__ __forceinline__ float rl_f(float v, int l) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l));
}

// inclusive scans over lanes [lo, lane] (lo = first lane of this lane's segment)
__device__ __forceinline__ float seg_scan_max(float x, int lane, int lo) {
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const float t = __shfl_up(x, off, kWave);
        if (lane - off >= lo) x = fmaxf(x, t);
    }
    return x;
}
__device__ __forceinline__ float seg_scan_add(float x, int lane, int lo) {
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const float t = __shfl_up(x, off, kWave);
        if (lane - off >= lo) x += t;
    }
    return x;
}

template <int HB, bool VEC>
__device__ __forceinline__ void load_heads(float (&v)[HB], const float* __restrict__ p, int nh) {
    if (VEC && HB == 8) {
        const float4 x = *reinterpret_cast<const float4*>(p), y = *reinterpret_cast<const float4*>(p + 4);
        v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
        v[4 % HB] = y.x; v[5 % HB] = y.y; v[6 % HB] = y.z; v[7 % HB] = y.w;
    } else if (VEC && HB == 4) {
        const float4 x = *reinterpret_cast<const float4*>(p);
        v[0] = x.x; v[1 % HB] = x.y; v[2 % HB] = x.z; v[3 % HB] = x.w;
    } else if (VEC && HB == 2) {
        const float2 x = *reinterpret_cast<const float2*>(p);
        v[0] = x.x; v[1 % HB] = x.y;
    } else {
#pragma unroll
        for (int i = 0; i < HB; ++i) v[i] = i < nh ? p[i] : 0.0f;
    }
}

template <int HB, bool VEC>
__device__ __forceinline__ void store_heads(float* __restrict__ p, const float (&v)[HB], int nh) {
    if (VEC && HB == 8) {
        *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1 % HB], v[2 % HB], v[3 % HB]);
        *reinterpret_cast<float4*>(p + 4) = make_float4(v[4 % HB], v[5 % HB], v[6 % HB], v[7 % HB]);
    } else if (VEC && HB == 4) {
        *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1 % HB], v[2 % HB], v[3 % HB]);
    } else if (VEC && HB == 2) {
        *reinterpret_cast<float2*>(p) = make_float2(v[0], v[1 % HB]);
    } else {
#pragma unroll
        for (int i = 0; i < HB; ++i)
            if (i < nh) p[i] = v[i];
    }
}

// blockDim.x = 256 (four spans per workgroup), grid = (ceil(nspans / 4), ceil(H / HB)).
// VEC: H is a multiple of HB, so the HB heads of an edge are one aligned vector.
template <int HB, bool VEC, bool FWD>
__global__ __launch_bounds__(256) void span_kernel(
    float* __restrict__ out, const float* __restrict__ a, const float* __restrict__ da,
    const float* __restrict__ e, const int64_t* __restrict__ indptr, const int64_t* __restrict__ eids,
    int64_t rows, int64_t nnz, int H, float slope, void* __restrict__ ws) {
    __shared__ int64_t win_all[4][kWin];
    const int lane = lane_id();
    const int wave = static_cast<int>(threadIdx.x) >> 6;
    const int64_t nspans = (nnz + kSpan - 1) / kSpan;
    const int64_t w = static_cast<int64_t>(blockIdx.x) * 4 + wave;
    if (w >= nspans) return;  // the whole wavefront leaves; no workgroup barrier below
    int64_t* win = win_all[wave];
    const int h0 = static_cast<int>(blockIdx.y) * HB;
    const int nh = H - h0 < HB ? H - h0 : HB;
    const int64_t base = w * kSpan;
    const int endl = static_cast<int>((nnz - base < kSpan) ? nnz - base : kSpan);  // slots in this span
    const int64_t end = base + endl;

    // ---- which row does each of my slots belong to
    const int64_t r0 = row_of_slot_wave(indptr, rows, base, lane);
#pragma unroll
    for (int k = 0; k < kWin / kWave; ++k) {
        const int64_t r = r0 + lane + kWave * k;
        win[lane + kWave * k] = r <= rows ? indptr[r] : INT64_MAX;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const bool staged = win[kWin - 1] >= end;  // every row of the span has both pointers in the window
    int rsl[kSteps], rel[kSteps];  // my row's first slot and end slot relative to base: -1 = before, kSpan + 1 = after
#pragma unroll
    for (int u = 0; u < kSteps; ++u) {
        int64_t s = base + kWave * u + lane;
        s = s < end ? s : end - 1;
        int64_t rs, re;
        if (staged) {
            int pos = 0;
#pragma unroll
            for (int step = 256; step > 0; step >>= 1)
                if (pos + step < kWin && win[pos + step] <= s) pos += step;
            rs = win[pos];
            re = win[pos + 1];
        } else {  // a long run of empty rows inside the span: search the array itself
            int64_t lo = r0, hi = rows;
            while (hi - lo > 1) {
                const int64_t mid = lo + ((hi - lo) >> 1);
                if (indptr[mid] <= s) lo = mid; else hi = mid;
            }
            rs = indptr[lo];
            re = indptr[lo + 1];
        }
        rsl[u] = rs < base ? -1 : static_cast<int>(rs - base);
        rel[u] = re > end ? kSpan + 1 : static_cast<int>(re - base);
    }

    // ---- values
    int64_t id[kSteps];
    float x[kSteps][HB];   // forward: leaky(e); backward: a
    float y[kSteps][HB];   // backward: da
#pragma unroll
    for (int u = 0; u < kSteps; ++u) {
        const int64_t s = base + kWave * u + lane;
        const bool valid = kWave * u + lane < endl;
        id[u] = -1;
#pragma unroll
        for (int i = 0; i < HB; ++i) x[u][i] = FWD ? -INFINITY : 0.0f, y[u][i] = 0.0f;
        if (valid) {
            id[u] = (eids ? eids[s] : s) * H + h0;
            if (FWD) {
                load_heads<HB, VEC>(x[u], e + id[u], nh);
#pragma unroll
                for (int i = 0; i < HB; ++i) x[u][i] = leaky(x[u][i], slope);
            } else {
                load_heads<HB, VEC>(x[u], a + id[u], nh);
                load_heads<HB, VEC>(y[u], da + id[u], nh);
            }
        }
    }

    // ---- per step: my row's result within the span so far
    float tm[kSteps][HB], ts[kSteps][HB];
    float fm[kSteps - 1][HB], fs[kSteps - 1][HB];  // wave-uniform: the row crossing the boundary after step b
    float cm[HB], cs[HB];                          // wave-uniform carry of the row open at the end of the last step
#pragma unroll
    for (int i = 0; i < HB; ++i) cm[i] = -INFINITY, cs[i] = 0.0f;
#pragma unroll
    for (int b = 0; b < kSteps - 1; ++b)
#pragma unroll
        for (int i = 0; i < HB; ++i) fm[b][i] = 0.0f, fs[b][i] = 1.0f;
#pragma unroll
    for (int u = 0; u < kSteps; ++u) {
        const int sbl = kWave * u;
        const int sel = sbl + kWave < endl ? sbl + kWave : endl;
        if (sbl >= endl) break;  // uniform
        const int lo = rsl[u] > sbl ? rsl[u] - sbl : 0;
        const int hi = (rel[u] < sel ? rel[u] : sel) - 1 - sbl;
        const bool cont_in = rsl[u] < sbl;  // my row began in an earlier step (or span)
#pragma unroll
        for (int i = 0; i < HB; ++i) {
            if (FWD) {
                float m = seg_scan_max(x[u][i], lane, lo);
                m = __shfl(m, hi, kWave);
                if (cont_in) m = fmaxf(m, cm[i]);
                const float ex = (kWave * u + lane < endl) ? expf(x[u][i] - m) : 0.0f;
                float s = seg_scan_add(ex, lane, lo);
                s = __shfl(s, hi, kWave);
                if (cont_in) s += cs[i] * expf(cm[i] - m);  // an empty carry is (-inf, 0)
                tm[u][i] = m;
                ts[u][i] = s;
            } else {
                float s = seg_scan_add(x[u][i] * y[u][i], lane, lo);
                s = __shfl(s, hi, kWave);
                if (cont_in) s += cs[i];
                tm[u][i] = 0.0f;
                ts[u][i] = s;
            }
        }
        // the row of lane 0 ends in this step and began in an earlier step of this span: its result
        // goes to the boundaries it crossed
        const int rs0 = __builtin_amdgcn_readfirstlane(rsl[u]);
        const int re0 = __builtin_amdgcn_readfirstlane(rel[u]);
        if (rs0 >= 0 && rs0 < sbl && re0 <= sel) {
#pragma unroll
            for (int b = 0; b < kSteps - 1; ++b)
                if (b < u && b >= (rs0 >> 6)) {
#pragma unroll
                    for (int i = 0; i < HB; ++i) fm[b][i] = rl_f(tm[u][i], 0), fs[b][i] = rl_f(ts[u][i], 0);
                }
        }
        // carry: the row of the last lane, if it runs on
        const bool open = __builtin_amdgcn_readlane(rel[u], kWave - 1) > sel;
#pragma unroll
        for (int i = 0; i < HB; ++i) {
            cm[i] = open ? rl_f(tm[u][i], kWave - 1) : -INFINITY;
            cs[i] = open ? rl_f(ts[u][i], kWave - 1) : 0.0f;
        }
        // partial results of the head row (at its last slot in the span) and of the tail row (at the span's last slot)
        const int ls = sbl + lane;  // my slot, relative
        if (ls < endl) {
            const bool last_of_row = ls == (rel[u] < endl ? rel[u] : endl) - 1;
            if (last_of_row && rsl[u] < 0) {
                store_heads<HB, false>(span_vals(ws, nspans, w, 0, 0, H) + h0, tm[u], nh);
                store_heads<HB, false>(span_vals(ws, nspans, w, 0, 1, H) + h0, ts[u], nh);
            }
            if (last_of_row && rsl[u] >= 0 && rel[u] > endl) {
                store_heads<HB, false>(span_vals(ws, nspans, w, 1, 0, H) + h0, tm[u], nh);
                store_heads<HB, false>(span_vals(ws, nspans, w, 1, 1, H) + h0, ts[u], nh);
            }
            if (blockIdx.y == 0) {
                SpanMeta* meta = static_cast<SpanMeta*>(ws) + w;
                if (ls == 0) {
                    meta->head_end = rsl[u] < 0 ? base + (rel[u] < endl ? rel[u] : endl) : base;
                    meta->head_open = (rsl[u] < 0 && rel[u] > endl) ? 1 : 0;
                }
                if (ls == endl - 1) meta->tail_start = (rsl[u] >= 0 && rel[u] > endl) ? base + rsl[u] : end;
            }
        }
    }

    // ---- rows inside the span: write
#pragma unroll
    for (int u = 0; u < kSteps; ++u) {
        const int sbl = kWave * u;
        const int sel = sbl + kWave < endl ? sbl + kWave : endl;
        if (id[u] < 0 || rsl[u] < 0 || rel[u] > endl) continue;
        const bool later = rel[u] > sel;  // my row ends in a later step
        float o[HB];
        if (FWD) {
#pragma unroll
            for (int i = 0; i < HB; ++i) {
                const float m = (later && u < kSteps - 1) ? fm[u < kSteps - 1 ? u : 0][i] : tm[u][i];
                const float s = (later && u < kSteps - 1) ? fs[u < kSteps - 1 ? u : 0][i] : ts[u][i];
                o[i] = expf(x[u][i] - m) * (1.0f / s);
            }
        } else {
            float z[HB];
            load_heads<HB, VEC>(z, e + id[u], nh);
#pragma unroll
            for (int i = 0; i < HB; ++i) {
                const float dot = (later && u < kSteps - 1) ? fs[u < kSteps - 1 ? u : 0][i] : ts[u][i];
                float g = x[u][i] * (y[u][i] - dot);
                if (!(z[i] > 0.0f)) g *= slope;
                o[i] = g;
            }
        }
        store_heads<HB, VEC>(out + id[u], o, nh);
    }
}

// One wavefront per span that holds the start of a cut row: merges the row's pieces and stores the
// result into each of them.  blockDim.x = 256, grid = ceil(nspans / 4).
template <bool FWD>
__global__ __launch_bounds__(256) void span_fix_kernel(int64_t nnz, int H, void* __restrict__ ws) {
    const int lane = lane_id();
    const int64_t nspans = (nnz + kSpan - 1) / kSpan;
    const int64_t w = static_cast<int64_t>(blockIdx.x) * 4 + (static_cast<int>(threadIdx.x) >> 6);
    if (w >= nspans) return;
    const SpanMeta* meta = static_cast<const SpanMeta*>(ws);
    const int64_t end = (w + 1) * kSpan < nnz ? (w + 1) * kSpan : nnz;
    if (meta[w].tail_start >= end) return;  // no row starts here and runs on
    // the pieces: tail of w, then heads of w + 1 .. last, where last is the first span whose head is closed
    int64_t last = w + 1;
    for (;; last += kWave) {
        const int64_t j = last + lane;
        const bool closed = j >= nspans || meta[j].head_open == 0;
        const uint64_t m = __ballot(closed);
        if (m) {
            last += __builtin_ctzll(m);
            break;
        }
    }
    if (last >= nspans) last = nspans - 1;
    for (int h = 0; h < H; ++h) {
        float m = -INFINITY, s = 0.0f;
        for (int64_t j = w + 1 + lane; j <= last; j += kWave) {
            const float s2 = *(span_vals(ws, nspans, j, 0, 1, H) + h);
            if (FWD) {
                const float m2 = *(span_vals(ws, nspans, j, 0, 0, H) + h);
                const float mx = fmaxf(m, m2);
                s = (m == -INFINITY ? 0.0f : s * expf(m - mx)) + s2 * expf(m2 - mx);
                m = mx;
            } else {
                s += s2;
            }
        }
        if (lane == 0) {  // the tail piece joins on lane 0
            const float s2 = *(span_vals(ws, nspans, w, 1, 1, H) + h);
            if (FWD) {
                const float m2 = *(span_vals(ws, nspans, w, 1, 0, H) + h);
                const float mx = fmaxf(m, m2);
                s = (m == -INFINITY ? 0.0f : s * expf(m - mx)) + s2 * expf(m2 - mx);
                m = mx;
            } else {
                s += s2;
            }
        }
        if (FWD) {
            const float mx = wave_max(m);
            s = (m == -INFINITY) ? 0.0f : s * expf(m - mx);
            m = mx;
        }
        s = wave_sum(s);
        for (int64_t j = w + 1 + lane; j <= last; j += kWave) {
            *(span_vals(ws, nspans, j, 0, 0, H) + h) = m;
            *(span_vals(ws, nspans, j, 0, 1, H) + h) = s;
        }
        if (lane == 0) {
            *(span_vals(ws, nspans, w, 1, 0, H) + h) = m;
            *(span_vals(ws, nspans, w, 1, 1, H) + h) = s;
        }
    }
}

// Writes the head and tail slots of every span from the merged results.  Launched like span_kernel.
template <int HB, bool VEC, bool FWD>
__global__ __launch_bounds__(256) void span_rest_kernel(
    float* __restrict__ out, const float* __restrict__ a, const float* __restrict__ da,
    const float* __restrict__ e, const int64_t* __restrict__ eids, int64_t nnz, int H, float slope,
    void* __restrict__ ws) {
    const int lane = lane_id();
    const int64_t nspans = (nnz + kSpan - 1) / kSpan;
    const int64_t w = static_cast<int64_t>(blockIdx.x) * 4 + (static_cast<int>(threadIdx.x) >> 6);
    if (w >= nspans) return;
    const SpanMeta mt = static_cast<const SpanMeta*>(ws)[w];
    const int64_t base = w * kSpan;
    const int64_t end = base + kSpan < nnz ? base + kSpan : nnz;
    if (mt.head_end <= base && mt.tail_start >= end) return;
    const int h0 = static_cast<int>(blockIdx.y) * HB;
    const int nh = H - h0 < HB ? H - h0 : HB;
    float rm[2][HB], rs[2][HB];
#pragma unroll
    for (int piece = 0; piece < 2; ++piece) {
        const bool have = piece == 0 ? mt.head_end > base : mt.tail_start < end;
#pragma unroll
        for (int i = 0; i < HB; ++i) {
            rm[piece][i] = (have && i < nh) ? *(span_vals(ws, nspans, w, piece, 0, H) + h0 + i) : 0.0f;
            rs[piece][i] = (have && i < nh) ? *(span_vals(ws, nspans, w, piece, 1, H) + h0 + i) : 1.0f;
        }
    }
#pragma unroll
    for (int u = 0; u < kSteps; ++u) {
        const int64_t s = base + kWave * u + lane;
        const bool inhead = s < mt.head_end;
        const bool intail = s >= mt.tail_start && s < end;
        if (!inhead && !intail) continue;
        const int piece = inhead ? 0 : 1;
        const int64_t id = (eids ? eids[s] : s) * H + h0;
        float o[HB], z[HB];
        load_heads<HB, VEC>(z, e + id, nh);
        if (FWD) {
#pragma unroll
            for (int i = 0; i < HB; ++i)
                o[i] = expf(leaky(z[i], slope) - (piece ? rm[1][i] : rm[0][i])) * (1.0f / (piece ? rs[1][i] : rs[0][i]));
        } else {
            float x[HB], y[HB];
            load_heads<HB, VEC>(x, a + id, nh);
            load_heads<HB, VEC>(y, da + id, nh);
#pragma unroll
            for (int i = 0; i < HB; ++i) {
                float g = x[i] * (y[i] - (piece ? rs[1][i] : rs[0][i]));
                if (!(z[i] > 0.0f)) g *= slope;
                o[i] = g;
            }
        }
        store_heads<HB, VEC>(out + id, o, nh);
    }
}

template <int HB, bool VEC, bool FWD>
static void launch_spans_hb(float* out, const float* a, const float* da, const float* e, const int64_t* indptr,
                            const int64_t* eids, int64_t rows, int64_t nnz, int H, float slope, void* ws,
                            hipStream_t s) {
    const int64_t nspans = ceil_div(nnz, kSpan);
    const dim3 grid(static_cast<unsigned>(ceil_div(nspans, 4)), static_cast<unsigned>(ceil_div(H, HB)));
    hipLaunchKernelGGL((span_kernel<HB, VEC, FWD>), grid, dim3(256), 0, s, out, a, da, e, indptr, eids, rows, nnz, H,
                       slope, ws);
    hipLaunchKernelGGL(span_fix_kernel<FWD>, dim3(grid.x), dim3(256), 0, s, nnz, H, ws);
    hipLaunchKernelGGL((span_rest_kernel<HB, VEC, FWD>), grid, dim3(256), 0, s, out, a, da, e, eids, nnz, H, slope,
                       ws);
}

template <bool FWD>
static void launch_spans(float* out, const float* a, const float* da, const float* e, const int64_t* indptr,
                         const int64_t* eids, int64_t rows, int64_t nnz, int H, float slope, void* ws,
                         hipStream_t s) {
#define TANGO_SPANS(HB, VEC) launch_spans_hb<HB, VEC, FWD>(out, a, da, e, indptr, eids, rows, nnz, H, slope, ws, s)
    if (H % 8 == 0) TANGO_SPANS(8, true);
    else if (H % 4 == 0) TANGO_SPANS(4, true);
    else if (H == 2) TANGO_SPANS(2, true);
    else if (H == 1) TANGO_SPANS(1, false);
    else if (H < 4) TANGO_SPANS(4, false);
    else TANGO_SPANS(8, false);
#undef TANGO_SPANS
}

static size_t span_workspace_bytes(int64_t nnz, int64_t H) {
    if (nnz <= 0 || H <= 0) return 0;
    const int64_t nspans = ceil_div(nnz, kSpan);
    return span_vals_offset(nspans) + static_cast<size_t>(nspans) * 4 * static_cast<size_t>(H) * sizeof(float);
}

}  // namespace tango

using namespace tango;

extern "C" {

size_t tango_edge_softmax_workspace(int64_t nnz, int64_t H) { return span_workspace_bytes(nnz, H); }

int tango_edge_softmax_fwd(float* a, const float* e, const int64_t* indptr,
                           const int64_t* edge_ids, int64_t rows, int64_t nnz, int64_t H, float slope,
                           void* workspace, size_t workspace_bytes, tango_stream_t stream) {
    if (rows < 0 || nnz < 0 || H < 0 || (rows > 0 && !indptr) || H >= (1LL << 31)) return TANGO_ERR_INVALID_ARG;
    if (rows * H == 0 || nnz == 0) return TANGO_OK;
    if (!a || !e) return TANGO_ERR_INVALID_ARG;
    if (workspace && ceil_div(nnz, 4 * kSpan) <= INT32_MAX && ceil_div(H, 8) <= 65535) {
        if (workspace_bytes < span_workspace_bytes(nnz, H) || (reinterpret_cast<uintptr_t>(workspace) & 15))
            return TANGO_ERR_WORKSPACE;
        launch_spans<true>(a, nullptr, nullptr, e, indptr, edge_ids, rows, nnz, static_cast<int>(H), slope,
                           workspace, as_stream(stream));
        return launch_status();
    }
    hipLaunchKernelGGL(edge_softmax_fwd_kernel, dim3(grid_for(rows * H, 256, 16)), dim3(256), 0,
                       as_stream(stream), a, e, indptr, edge_ids, rows, static_cast<int>(H), slope);
    return launch_status();
}

int tango_edge_softmax_bwd(float* de, const float* a, const float* da, const float* e,
                           const int64_t* indptr, const int64_t* edge_ids, int64_t rows, int64_t nnz,
                           int64_t H, float slope, void* workspace, size_t workspace_bytes,
                           tango_stream_t stream) {
    if (rows < 0 || nnz < 0 || H < 0 || (rows > 0 && !indptr) || H >= (1LL << 31)) return TANGO_ERR_INVALID_ARG;
    if (rows * H == 0 || nnz == 0) return TANGO_OK;
    if (!de || !a || !da || !e) return TANGO_ERR_INVALID_ARG;
    if (workspace && ceil_div(nnz, 4 * kSpan) <= INT32_MAX && ceil_div(H, 8) <= 65535) {
        if (workspace_bytes < span_workspace_bytes(nnz, H) || (reinterpret_cast<uintptr_t>(workspace) & 15))
            return TANGO_ERR_WORKSPACE;
        launch_spans<false>(de, a, da, e, indptr, edge_ids, rows, nnz, static_cast<int>(H), slope, workspace,
                            as_stream(stream));
        return launch_status();
    }
    hipLaunchKernelGGL(edge_softmax_bwd_kernel, dim3(grid_for(rows * H, 256, 16)), dim3(256), 0,
                       as_stream(stream), de, a, da, e, indptr, edge_ids, rows, static_cast<int>(H),
                       slope);
    return launch_status();
}

}  // extern "C"
