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

#include <mutex>

namespace tango {

// Scratch of the entry point that allocates nothing (tango_edge_softmax_fwd_static): the per-span partial
// (max, sum) records that the span kernels otherwise keep in the caller's workspace.  One copy per device,
// held until the process ends.  In host code this name is only a handle for hipGetSymbolAddress; kernels
// receive the device address that call returns.
static __device__ __align__(256) unsigned char scratch[TANGO_EDGE_SOFTMAX_STATIC_BYTES];

constexpr int kMaxDevices = 64;
static std::mutex scratch_mutex;
// Per device: the device address of `scratch` (looked up once), and what orders calls that arrive on different
// streams: the stream of the last call and an event recorded behind its kernels.  A call on another stream waits
// for that event first, so that it does not overwrite records the earlier call's kernels still read.
struct StaticScratch {
    void* address;
    hipEvent_t done;
    hipStream_t last_stream;
    bool recorded;
};
static StaticScratch static_scratch[kMaxDevices];

// Set-up of the current device's entry (address of `scratch`, the event), once per device; nullptr on failure.
// Call with scratch_mutex held.
static StaticScratch* scratch_of_current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    StaticScratch& sc = static_scratch[dev];
    if (!sc.address) {
        void* p = nullptr;
        hipEvent_t ev = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess ||
            hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        sc.done = ev;
        sc.address = p;
    }
    return &sc;
}

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
            if (e && !(e[id * H + h] > 0.0f)) g *= slope;  // e may be absent for slope 1
            de[id * H + h] = g;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Span kernels.  Wavefront w owns SPAN consecutive slots (64 to 256, by the number of heads a
// wavefront covers).  The lanes are (group g, head h) pairs, HB heads (head block blockIdx.y) by
// G = 64 / HB groups, and a lane holds the K consecutive slots [g K, g K + K) of its head in
// registers: a row's reduction is a serial sweep over the lane's own values, and only one
// aggregate per lane crosses lanes (a segmented scan over the G groups, then one fetch from the
// group the row ends in): about 1.5 cross-lane steps per value instead of the 14 a lane-per-slot
// layout needs.  Row starts are the bits of a mask in LDS, built from the row pointers that
// follow the span's first row (a 64-ary search finds that row).  Three kinds of row:
//   inside : starts and ends within the span -> written by this launch;
//   head   : started in an earlier span      -> partial result in piece 0 of the span's record;
//   tail   : runs on into the next span      -> partial result in piece 1.
// span_fix_kernel merges a row's pieces (the tail of the span it starts in and the heads of the
// spans that follow) and stores the row's result back into every piece; span_rest_kernel then
// writes the head and tail slots.  No atomics on results: they do not depend on scheduling.
constexpr int kWin = 256 + kWave;  // row pointers inspected per span: 64 empty rows of slack

// What the neighbours of the softmax in an attention layer fold into these kernels (all optional):
//   el, er ..: the logits are formed here, e[edge, h] = q(el[src, h]) s_el + q(er[dst, h]) s_er with q the
//              half-to-even int8 rounding of the two scales (what the quantize-on-load element-wise SDDMM
//              writes out, same operations in the same order), instead of being read from memory;
//   sign_out : forward, bit h % 8 of byte [slot, h / 8] = (e > 0), all the backward pass needs of e;
//   sign_in  : backward, those bytes in place of e;
//   scale_out: receives max|result| / 127, the scale the next quantizer needs, so that no separate pass over the
//              result looks for it: every wavefront leaves the maximum of what it wrote in `part` (one word per
//              wavefront of the two writing launches, plain stores: thousands of atomics on one word would be
//              served one at a time) and a one-workgroup launch folds those.
struct AttnFuse {
    const float* el;
    const float* er;
    const float* s_el;
    const float* s_er;
    const int64_t* src;  // edge-id order
    const int64_t* dst;
    uint8_t* sign_out;
    const uint8_t* sign_in;
    float* scale_out;
    float* part;  // [2][head blocks][spans] in the workspace
};

__device__ __forceinline__ float fused_logit(const AttnFuse& fz, int64_t edge, int H, int h, float r_el, float r_er,
                                             float s_el, float s_er) {
    const float u = static_cast<float>(quant_one<TANGO_ROUND_RNE>(fz.el[fz.src[edge] * H + h], r_el, 0.0f)) * s_el;
    const float v = static_cast<float>(quant_one<TANGO_ROUND_RNE>(fz.er[fz.dst[edge] * H + h], r_er, 0.0f)) * s_er;
    return u + v;
}

// the wavefront's maximum into its word of the partial results
__device__ __forceinline__ void wave_part_out(float m, float* slot) {
    m = wave_max(m);
    if (lane_id() == 0) *slot = m;
}

// scale_out[0] = max(part[0 .. count)) / 127.  One workgroup of 1024.
__global__ __launch_bounds__(1024) void scale_reduce_kernel(const float* __restrict__ part, int64_t count,
                                                            float* __restrict__ scale_out) {
    __shared__ float wm[16];
    float m = 0.0f;
    for (int64_t i = threadIdx.x; i < count; i += 1024) m = fmaxf(m, part[i]);
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) wm[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x < 64) {
        m = threadIdx.x < 16 ? wm[threadIdx.x] : 0.0f;
        m = wave_max(m);
        if (threadIdx.x == 0) scale_out[0] = m / 127.0f;
    }
}

struct SpanMeta {
    int64_t head_end;    // slots [base, head_end) belong to a row that started before the span
    int64_t tail_start;  // slots [tail_start, end) belong to a row that runs on after the span
    int64_t head_open;   // the head row also runs on after the span (then there is no tail)
};

__host__ __device__ inline size_t span_vals_offset(int64_t nspans) {
    return (static_cast<size_t>(nspans) * sizeof(SpanMeta) + 255) & ~static_cast<size_t>(255);
}
// after the records' values: one word per wavefront of the two launches that write results (see AttnFuse::part)
__host__ __device__ inline size_t span_parts_offset(int64_t nspans, int64_t H) {
    return span_vals_offset(nspans) + static_cast<size_t>(nspans) * 4 * static_cast<size_t>(H) * sizeof(float);
}
// vals[span][piece][component][H]: component 0 = max, 1 = sum (backward: only the sum)
__device__ __forceinline__ float* span_vals(void* ws, int64_t nspans, int64_t w, int piece, int comp, int H) {
    return reinterpret_cast<float*>(static_cast<char*>(ws) + span_vals_offset(nspans)) +
           ((w * 2 + piece) * 2 + comp) * static_cast<int64_t>(H);
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

// Where a row's aggregate comes from, per lane: everything the cross-group step needs.
struct GroupLinks {
    int g;        // my group
    int seg0;     // first group of the run of groups my last segment's row spans so far (scan bound)
    int next;     // lane (same head) of the next group that holds a row start, or -1
    int last;     // lane (same head) of the last group with slots of this span
};

// F = aggregate of my slots before my first row start (all of them if I have none), L = of my slots
// from my last row start on.  Returns TF = the whole (within the span) of the row that ends at my
// first row start and X = of the row my last slots belong to.
template <int HB, bool MAX>
__device__ __forceinline__ void cross_groups(float F, float L, const GroupLinks& k, float& TF, float& X) {
    constexpr int G = kWave / HB;
    float S = L;  // inclusive scan over the groups back to the one my row starts in
#pragma unroll
    for (int d = 1; d < G; d <<= 1) {
        const float t = __shfl_up(S, d * HB, kWave);
        if (k.g - d >= k.seg0) S = MAX ? fmaxf(S, t) : S + t;
    }
    float PF = __shfl_up(S, HB, kWave);
    if (k.g == 0) PF = MAX ? -INFINITY : 0.0f;
    TF = MAX ? fmaxf(PF, F) : PF + F;
    const float xn = __shfl(TF, k.next < 0 ? 0 : k.next, kWave);
    const float xe = __shfl(S, k.last, kWave);
    X = k.next < 0 ? xe : xn;
}

// In-lane pass over the lane's K values: v[] becomes, slot by slot, the aggregate of the slot's
// row within the span.  `sub` has bit k set when slot k starts a row.
template <int HB, int K, bool MAX>
__device__ __forceinline__ void row_aggregates(float (&v)[K], unsigned sub, const GroupLinks& lk, float& TF, float& X) {
    const float ident = MAX ? -INFINITY : 0.0f;
    float run = ident, F = ident;
    bool seen = false;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        if ((sub >> k) & 1u) {
            if (!seen) F = run;
            seen = true;
            run = ident;
        }
        run = MAX ? fmaxf(run, v[k]) : run + v[k];
        v[k] = run;  // prefix within the row's slots of this lane
    }
    if (!seen) F = run;
    cross_groups<HB, MAX>(F, run, lk, TF, X);
    // backwards: the last slots take X, rows inside the lane their own prefix at their last slot, the first slots TF
    const int kf = sub ? __builtin_ctz(sub) : K;
    float cur = X;
#pragma unroll
    for (int k = K - 1; k >= 0; --k) {
        const float prev = k > 0 ? v[k - 1] : ident;
        v[k] = cur;
        if ((sub >> k) & 1u) cur = (k == kf) ? TF : prev;
    }
}

// blockDim.x = 256 (four spans per workgroup), grid = (ceil(nspans / 4), ceil(H / HB)).
template <int HB, int K, bool FWD>
__global__ __launch_bounds__(256) void span_kernel(
    float* __restrict__ out, const float* __restrict__ a, const float* __restrict__ da,
    const float* __restrict__ e, const int64_t* __restrict__ indptr, const int64_t* __restrict__ eids,
    int64_t rows, int64_t nnz, int H, float slope, void* __restrict__ ws, const AttnFuse fz) {
    constexpr int G = kWave / HB;
    constexpr int SPAN = G * K;
    static_assert(SPAN <= 256 && (32 % K) == 0, "a lane's row-start bits must sit in one mask word");
    __shared__ unsigned maskw_all[4][12];
    const int lane = lane_id();
    const int wave = static_cast<int>(threadIdx.x) >> 6;
    const int64_t nspans = (nnz + SPAN - 1) / SPAN;
    const int64_t w = static_cast<int64_t>(blockIdx.x) * 4 + wave;
    if (w >= nspans) return;  // the whole wavefront leaves; no workgroup barrier below
    unsigned* maskw = maskw_all[wave];
    const int g = lane / HB, h = lane % HB;
    const int h0 = static_cast<int>(blockIdx.y) * HB;
    const bool hok = h0 + h < H;
    const int64_t base = w * SPAN;
    const int endl = static_cast<int>((nnz - base < SPAN) ? nnz - base : SPAN);  // slots in this span
    const int64_t end = base + endl;

    // ---- values first: their loads are in flight while the row structure is worked out
    int64_t id[K];
    float x[K], y[K];
    unsigned posbits = 0u;  // bit k: the logit of slot k is positive (LeakyReLU's derivative is 1)
    const int nhb = (H + 7) >> 3;  // sign bytes per slot
    float s_el = 0.0f, s_er = 0.0f, r_el = 0.0f, r_er = 0.0f;
    if (FWD && fz.el) {
        s_el = fz.s_el[0], s_er = fz.s_er[0];
        r_el = rscale_of(s_el), r_er = rscale_of(s_er);
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const int j = g * K + k;
        id[k] = -1;
        x[k] = FWD ? -INFINITY : 0.0f;
        y[k] = 0.0f;
        if (j < endl && hok) {
            const int64_t edge = eids ? eids[base + j] : base + j;
            id[k] = edge * H + h0 + h;
            if (FWD) {
                const float ev = fz.el ? fused_logit(fz, edge, H, h0 + h, r_el, r_er, s_el, s_er) : e[id[k]];
                posbits |= (ev > 0.0f ? 1u : 0u) << k;
                x[k] = leaky(ev, slope);
            } else {
                x[k] = a[id[k]];
                y[k] = da[id[k]];
                bool pos = true;
                if (fz.sign_in) pos = (fz.sign_in[(base + j) * nhb + ((h0 + h) >> 3)] >> ((h0 + h) & 7)) & 1;
                else if (e) pos = e[id[k]] > 0.0f;
                posbits |= (pos ? 1u : 0u) << k;
            }
        }
    }
    if (FWD && fz.sign_out) {
        // A lane group holds HB <= 8 heads of a slot, and head blocks narrower than eight only occur when they
        // hold every head (H <= HB), so each sign byte is written whole by one lane.
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const uint64_t bal = __ballot((posbits >> k) & 1u);
            const int j = g * K + k;
            if (h == 0 && j < endl)
                fz.sign_out[(base + j) * nhb + (h0 >> 3)] = static_cast<uint8_t>((bal >> (g * HB)) & ((1u << HB) - 1u));
        }
    }

    // ---- row starts inside the span
    const int64_t r0 = row_of_slot_wave(indptr, rows, base, lane);
    if (lane < 12) maskw[lane] = 0u;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    bool covered = false;  // the inspected row pointers reach the span's end
#pragma unroll
    for (int k = 0; k < kWin / kWave; ++k) {
        const int64_t r = r0 + lane + kWave * k;
        const int64_t pv = r <= rows ? indptr[r] : INT64_MAX;
        if (pv >= base && pv < end) {
            const int sl = static_cast<int>(pv - base);
            atomicOr(&maskw[sl >> 5], 1u << (sl & 31));
        }
        if (pv == end) atomicOr(&maskw[8], 1u);  // a row ends exactly at the span's end
        if (k == kWin / kWave - 1) covered = __builtin_amdgcn_readlane(static_cast<int>(pv >= end), kWave - 1) != 0;
    }
    if (!covered) {  // more than 64 empty rows inside the span: search the array per slot
        for (int sl = lane; sl < endl; sl += kWave) {
            const int64_t s = base + sl;
            int64_t lo = r0, hi = rows;
            while (hi - lo > 1) {
                const int64_t mid = lo + ((hi - lo) >> 1);
                if (indptr[mid] <= s) lo = mid; else hi = mid;
            }
            if (indptr[lo] == s) atomicOr(&maskw[sl >> 5], 1u << (sl & 31));
            if (sl == endl - 1 && indptr[lo + 1] == end) atomicOr(&maskw[8], 1u);
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const unsigned sub = (maskw[(g * K) >> 5] >> ((g * K) & 31)) & (K == 32 ? 0xFFFFFFFFu : (1u << (K & 31)) - 1u);
    const bool last_open = (maskw[8] & 1u) == 0u;  // the row of the last slot runs on into the next span
    const bool head = (maskw[0] & 1u) == 0u;       // the row of the first slot began before the span
    const uint64_t bm = __ballot(sub != 0u);       // lanes of groups that hold a row start
    GroupLinks lk;
    lk.g = g;
    {
        const uint64_t upto = bm & ((2ull << (g * HB + HB - 1)) - 1ull);  // 2 << 63 wraps to 0: all bits kept
        lk.seg0 = upto ? (63 - __builtin_clzll(upto)) / HB : 0;
        const int sh = (g + 1) * HB;
        const uint64_t after = sh < kWave ? bm >> sh : 0ull;
        lk.next = after ? (g + 1 + __builtin_ctzll(after) / HB) * HB + h : -1;
        lk.last = ((endl - 1) / K) * HB + h;
    }
    // first and last row start of the span, as slots (wave-uniform)
    const int kf = sub ? __builtin_ctz(sub) : K;
    const int kl = sub ? 31 - __builtin_clz(sub) : 0;
    const int gfirst = bm ? __builtin_ctzll(bm) / HB : 0, glast = bm ? (63 - __builtin_clzll(bm)) / HB : 0;
    const int ffpos = __shfl(g * K + kf, gfirst * HB, kWave), lfpos = __shfl(g * K + kl, glast * HB, kWave);
    const int hpos = !head ? 0 : (bm ? ffpos : endl);                // slots before hpos: the head row
    const int tpos = (last_open && bm) ? lfpos : endl;               // slots from tpos on: the tail row

    float rm[K], rs[K];  // per slot: the row's max and sum within the span
    float tfm = 0.0f, xm = 0.0f, tfs, xs;
    if (FWD) {
#pragma unroll
        for (int k = 0; k < K; ++k) rm[k] = x[k];
        row_aggregates<HB, K, true>(rm, sub, lk, tfm, xm);
#pragma unroll
        for (int k = 0; k < K; ++k) {
            x[k] = id[k] >= 0 ? expf(x[k] - rm[k]) : 0.0f;
            rs[k] = x[k];
        }
    } else {
#pragma unroll
        for (int k = 0; k < K; ++k) rs[k] = x[k] * y[k], rm[k] = 0.0f;
    }
    row_aggregates<HB, K, false>(rs, sub, lk, tfs, xs);

    // ---- partial results of the head row and of the tail row, the span's record
    float* vals_hm = span_vals(ws, nspans, w, 0, 0, H) + h0 + h;
    float* vals_hs = span_vals(ws, nspans, w, 0, 1, H) + h0 + h;
    if (head && hok) {
        if (bm && g == gfirst) {
            *vals_hm = tfm;
            *vals_hs = tfs;
        }
        if (!bm && lane == lk.last) {  // no row starts in the span: it is all head
            *vals_hm = xm;
            *vals_hs = xs;
        }
    }
    if (last_open && bm && lane == lk.last && hok) {
        *(span_vals(ws, nspans, w, 1, 0, H) + h0 + h) = xm;
        *(span_vals(ws, nspans, w, 1, 1, H) + h0 + h) = xs;
    }
    if (lane == 0 && blockIdx.y == 0) {
        SpanMeta* meta = static_cast<SpanMeta*>(ws) + w;
        meta->head_end = base + hpos;
        meta->tail_start = base + tpos;
        meta->head_open = (head && !bm && last_open) ? 1 : 0;
    }

    // ---- rows inside the span: write
    float amax = 0.0f;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const int j = g * K + k;
        if (id[k] < 0 || j < hpos || j >= tpos) continue;
        float o;
        if (FWD) {
            o = x[k] * __builtin_amdgcn_rcpf(rs[k]);  // 1 ulp: an IEEE divide is ten instructions per value
        } else {
            o = x[k] * (y[k] - rs[k]);
            if (!((posbits >> k) & 1u)) o *= slope;
        }
        out[id[k]] = o;
        amax = fmaxf(amax, fabsf(o));
    }
    if (fz.scale_out) wave_part_out(amax, fz.part + static_cast<int64_t>(blockIdx.y) * nspans + w);
}

__device__ __forceinline__ void merge_max_sum(float& m, float& s, float m2, float s2) {
    const float mx = fmaxf(m, m2);
    // exp(-inf - -inf) would be NaN: a side with no elements contributes nothing
    const float u = (m == -INFINITY) ? 0.0f : s * expf(m - mx);
    const float v = (m2 == -INFINITY) ? 0.0f : s2 * expf(m2 - mx);
    m = mx;
    s = u + v;
}

// One wavefront per span that holds the start of a cut row: merges the row's pieces (the tail piece
// of this span, the head pieces of the following ones) and stores the result into each of them.
// Lanes are (chunk, head) pairs: a lane folds every 64/Hp-th piece of its head, the chunks are
// folded with xor-shuffles.  blockDim.x = 256, grid = ceil(nspans / 4).
template <bool FWD>
__global__ __launch_bounds__(256) void span_fix_kernel(int64_t nnz, int span, int H, void* __restrict__ ws) {
    const int lane = lane_id();
    const int64_t nspans = (nnz + span - 1) / span;
    const int64_t w = static_cast<int64_t>(blockIdx.x) * 4 + (static_cast<int>(threadIdx.x) >> 6);
    if (w >= nspans) return;
    const SpanMeta* meta = static_cast<const SpanMeta*>(ws);
    const int64_t end = (w + 1) * span < nnz ? (w + 1) * span : nnz;
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
    int hp = 1;
    while (hp < H && hp < kWave) hp <<= 1;
    const int chunks = kWave / hp, c = lane / hp;
    for (int hb = 0; hb < H; hb += hp) {
        const int h = hb + lane % hp;
        const bool ok = h < H;
        float m = -INFINITY, s = 0.0f;
        if (ok) {
            for (int64_t j = w + 1 + c; j <= last; j += chunks) {
                const float s2 = *(span_vals(ws, nspans, j, 0, 1, H) + h);
                if (FWD) merge_max_sum(m, s, *(span_vals(ws, nspans, j, 0, 0, H) + h), s2);
                else s += s2;
            }
            if (c == 0) {  // the tail piece joins on chunk 0
                const float s2 = *(span_vals(ws, nspans, w, 1, 1, H) + h);
                if (FWD) merge_max_sum(m, s, *(span_vals(ws, nspans, w, 1, 0, H) + h), s2);
                else s += s2;
            }
        }
        for (int off = hp; off < kWave; off <<= 1) {
            const float m2 = __shfl_xor(m, off, kWave), s2 = __shfl_xor(s, off, kWave);
            if (FWD) merge_max_sum(m, s, m2, s2);
            else s += s2;
        }
        if (ok) {
            for (int64_t j = w + 1 + c; j <= last; j += chunks) {
                *(span_vals(ws, nspans, j, 0, 0, H) + h) = m;
                *(span_vals(ws, nspans, j, 0, 1, H) + h) = s;
            }
            if (c == 0) {
                *(span_vals(ws, nspans, w, 1, 0, H) + h) = m;
                *(span_vals(ws, nspans, w, 1, 1, H) + h) = s;
            }
        }
    }
}

// Writes the head and tail slots of every span from the merged results.  Launched like span_kernel.
template <int HB, bool VEC, bool FWD>
__global__ __launch_bounds__(256) void span_rest_kernel(
    float* __restrict__ out, const float* __restrict__ a, const float* __restrict__ da,
    const float* __restrict__ e, const int64_t* __restrict__ eids, int64_t nnz, int span, int H, float slope,
    void* __restrict__ ws, const AttnFuse fz) {
    const int lane = lane_id();
    const int64_t nspans = (nnz + span - 1) / span;
    const int64_t w = static_cast<int64_t>(blockIdx.x) * 4 + (static_cast<int>(threadIdx.x) >> 6);
    if (w >= nspans) return;
    const SpanMeta mt = static_cast<const SpanMeta*>(ws)[w];
    const int64_t base = static_cast<int64_t>(w) * span;
    const int64_t end = base + span < nnz ? base + span : nnz;
    float* const my_part = fz.part + (static_cast<int64_t>(gridDim.y) + blockIdx.y) * nspans + w;
    if (mt.head_end <= base && mt.tail_start >= end) {
        if (fz.scale_out && lane == 0) *my_part = 0.0f;
        return;
    }
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
    const int nhb = (H + 7) >> 3;
    float s_el = 0.0f, s_er = 0.0f, r_el = 0.0f, r_er = 0.0f;
    if (FWD && fz.el) {
        s_el = fz.s_el[0], s_er = fz.s_er[0];
        r_el = rscale_of(s_el), r_er = rscale_of(s_er);
    }
    float amax = 0.0f;
    for (int u = 0; u < span / kWave; ++u) {
        const int64_t s = base + kWave * u + lane;
        const bool inhead = s < mt.head_end;
        const bool intail = s >= mt.tail_start && s < end;
        if (!inhead && !intail) continue;
        const int piece = inhead ? 0 : 1;
        const int64_t edge = eids ? eids[s] : s;
        const int64_t id = edge * H + h0;
        float o[HB], z[HB];
        if (FWD && fz.el) {
#pragma unroll
            for (int i = 0; i < HB; ++i) z[i] = i < nh ? fused_logit(fz, edge, H, h0 + i, r_el, r_er, s_el, s_er) : 0.0f;
        } else if (!FWD && fz.sign_in) {
            const unsigned bits = fz.sign_in[s * nhb + (h0 >> 3)] >> (h0 & 7);
#pragma unroll
            for (int i = 0; i < HB; ++i) z[i] = ((bits >> i) & 1u) ? 1.0f : -1.0f;
        } else if (e) {
            load_heads<HB, VEC>(z, e + id, nh);
        } else {
#pragma unroll
            for (int i = 0; i < HB; ++i) z[i] = 1.0f;
        }
        if (FWD) {
#pragma unroll
            for (int i = 0; i < HB; ++i)
                o[i] = expf(leaky(z[i], slope) - (piece ? rm[1][i] : rm[0][i])) * __builtin_amdgcn_rcpf(piece ? rs[1][i] : rs[0][i]);
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
#pragma unroll
        for (int i = 0; i < HB; ++i)
            if (i < nh) amax = fmaxf(amax, fabsf(o[i]));
    }
    if (fz.scale_out) wave_part_out(amax, my_part);
}

// slots per span by head count: lanes are (group, head) pairs, K slots per lane
static int span_slots(int H) { return H % 8 == 0 || H > 4 ? 128 : 256; }

template <int HB, int K, bool VEC, bool FWD>
static void launch_spans_hb(float* out, const float* a, const float* da, const float* e, const int64_t* indptr,
                            const int64_t* eids, int64_t rows, int64_t nnz, int H, float slope, void* ws,
                            hipStream_t s, const AttnFuse& fz_) {
    constexpr int SPAN = (kWave / HB) * K;
    const int64_t nspans = ceil_div(nnz, SPAN);
    const dim3 grid(static_cast<unsigned>(ceil_div(nspans, 4)), static_cast<unsigned>(ceil_div(H, HB)));
    AttnFuse fz = fz_;
    fz.part = reinterpret_cast<float*>(static_cast<char*>(ws) + span_parts_offset(nspans, H));
    hipLaunchKernelGGL((span_kernel<HB, K, FWD>), grid, dim3(256), 0, s, out, a, da, e, indptr, eids, rows, nnz, H,
                       slope, ws, fz);
    hipLaunchKernelGGL(span_fix_kernel<FWD>, dim3(grid.x), dim3(256), 0, s, nnz, SPAN, H, ws);
    hipLaunchKernelGGL((span_rest_kernel<HB, VEC, FWD>), grid, dim3(256), 0, s, out, a, da, e, eids, nnz, SPAN, H,
                       slope, ws, fz);
    if (fz.scale_out)
        hipLaunchKernelGGL(scale_reduce_kernel, dim3(1), dim3(1024), 0, s, fz.part, 2 * static_cast<int64_t>(grid.y) * nspans,
                           fz.scale_out);
}

template <bool FWD>
static void launch_spans(float* out, const float* a, const float* da, const float* e, const int64_t* indptr,
                         const int64_t* eids, int64_t rows, int64_t nnz, int H, float slope, void* ws,
                         hipStream_t s, const AttnFuse& fz = AttnFuse{}) {
#define TANGO_SPANS(HB, K, VEC) launch_spans_hb<HB, K, VEC, FWD>(out, a, da, e, indptr, eids, rows, nnz, H, slope, ws, s, fz)
    if (H % 8 == 0) TANGO_SPANS(8, 16, true);
    else if (H > 4) TANGO_SPANS(8, 16, false);
    else if (H == 4) TANGO_SPANS(4, 16, true);
    else if (H == 3) TANGO_SPANS(4, 16, false);
    else if (H == 2) TANGO_SPANS(2, 8, true);
    else TANGO_SPANS(1, 4, false);
#undef TANGO_SPANS
}

static size_t span_workspace_bytes(int64_t nnz, int64_t H) {
    if (nnz <= 0 || H <= 0) return 0;
    const int64_t nspans = ceil_div(nnz, span_slots(static_cast<int>(H < 64 ? H : 64)));
    // head blocks are min(H, 8) heads wide: one for H <= 8, else ceil(H / 8)
    const int64_t blocks = H <= 8 ? 1 : ceil_div(H, 8);
    return span_parts_offset(nspans, H) + static_cast<size_t>(2 * blocks * nspans) * sizeof(float);
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
    if (workspace && ceil_div(nnz, 4 * 128) <= INT32_MAX && ceil_div(H, 8) <= 65535) {
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

int tango_edge_softmax_fwd_static(float* a, const float* e, const int64_t* indptr, const int64_t* edge_ids,
                                  int64_t rows, int64_t nnz, int64_t H, float slope, tango_stream_t stream) {
    if (rows < 0 || nnz < 0 || H < 0 || (rows > 0 && !indptr) || H >= (1LL << 31)) return TANGO_ERR_INVALID_ARG;
    if (rows * H == 0 || nnz == 0) return TANGO_OK;
    if (!a || !e) return TANGO_ERR_INVALID_ARG;
    if (ceil_div(nnz, 4 * 128) > INT32_MAX || ceil_div(H, 8) > 65535) return TANGO_ERR_UNSUPPORTED;
    if (span_workspace_bytes(nnz, H) > TANGO_EDGE_SOFTMAX_STATIC_BYTES) return TANGO_ERR_STATIC_LIMIT;
    hipStream_t s = as_stream(stream);
    std::lock_guard<std::mutex> lock(scratch_mutex);
    StaticScratch* sc = scratch_of_current_device();
    if (!sc) return TANGO_ERR_LAUNCH;
    // Calls on one stream are ordered by the stream.  A call on another stream than the last one first waits for
    // the last call's kernels.  Not under stream capture: there the graph's own dependencies order the nodes, and
    // an event recorded outside the capture must not be waited for inside it.
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &capture) != hipSuccess) {
        (void)hipGetLastError();
        capture = hipStreamCaptureStatusActive;  // the legacy stream while another stream captures: no event calls
    }
    const bool eager = capture == hipStreamCaptureStatusNone;
    if (eager && sc->recorded && sc->last_stream != s && hipStreamWaitEvent(s, sc->done, 0) != hipSuccess) {
        (void)hipGetLastError();
        return TANGO_ERR_LAUNCH;
    }
    // The span kernels write every record of the scratch they later read, so nothing has to be cleared.
    launch_spans<true>(a, nullptr, nullptr, e, indptr, edge_ids, rows, nnz, static_cast<int>(H), slope, sc->address, s);
    const int rc = launch_status();
    if (eager && rc == TANGO_OK) {
        if (hipEventRecord(sc->done, s) != hipSuccess) {
            (void)hipGetLastError();
            return TANGO_ERR_LAUNCH;
        }
        sc->last_stream = s;
        sc->recorded = true;
    }
    return rc;
}

int tango_edge_softmax_fwd_ex(float* a, float* scale_a, uint8_t* sign_out, const float* e, const float* el,
                              const float* er, const float* s_el, const float* s_er, const int64_t* src,
                              const int64_t* dst, const int64_t* indptr, const int64_t* edge_ids, int64_t rows,
                              int64_t nnz, int64_t H, float slope, void* workspace, size_t workspace_bytes,
                              tango_stream_t stream) {
    if (rows < 0 || nnz < 0 || H < 0 || (rows > 0 && !indptr) || H >= (1LL << 31)) return TANGO_ERR_INVALID_ARG;
    if (rows * H == 0 || nnz == 0) return TANGO_OK;
    if (!a) return TANGO_ERR_INVALID_ARG;
    const bool fused = el != nullptr;
    if (fused ? (!er || !s_el || !s_er || !src || !dst) : !e) return TANGO_ERR_INVALID_ARG;
    if (!workspace) return TANGO_ERR_WORKSPACE;  // only the slot-span kernels carry the fused forms
    if (ceil_div(nnz, 4 * 128) > INT32_MAX || ceil_div(H, 8) > 65535) return TANGO_ERR_UNSUPPORTED;
    if (workspace_bytes < span_workspace_bytes(nnz, H) || (reinterpret_cast<uintptr_t>(workspace) & 15))
        return TANGO_ERR_WORKSPACE;
    hipStream_t s = as_stream(stream);
    AttnFuse fz{};
    fz.el = el; fz.er = er; fz.s_el = s_el; fz.s_er = s_er; fz.src = src; fz.dst = dst;
    fz.sign_out = sign_out; fz.scale_out = scale_a;
    launch_spans<true>(a, nullptr, nullptr, e, indptr, edge_ids, rows, nnz, static_cast<int>(H), slope, workspace, s,
                       fz);
    return launch_status();
}

int tango_edge_softmax_bwd_ex(float* de, float* scale_de, const float* a, const float* da, const float* e,
                              const uint8_t* sign_in, const int64_t* indptr, const int64_t* edge_ids, int64_t rows,
                              int64_t nnz, int64_t H, float slope, void* workspace, size_t workspace_bytes,
                              tango_stream_t stream) {
    if (rows < 0 || nnz < 0 || H < 0 || (rows > 0 && !indptr) || H >= (1LL << 31)) return TANGO_ERR_INVALID_ARG;
    if (rows * H == 0 || nnz == 0) return TANGO_OK;
    if (!de || !a || !da) return TANGO_ERR_INVALID_ARG;
    if (!e && !sign_in && slope != 1.0f) return TANGO_ERR_INVALID_ARG;  // LeakyReLU's derivative needs one of them
    if (!workspace) return TANGO_ERR_WORKSPACE;
    if (ceil_div(nnz, 4 * 128) > INT32_MAX || ceil_div(H, 8) > 65535) return TANGO_ERR_UNSUPPORTED;
    if (workspace_bytes < span_workspace_bytes(nnz, H) || (reinterpret_cast<uintptr_t>(workspace) & 15))
        return TANGO_ERR_WORKSPACE;
    AttnFuse fz{};
    fz.sign_in = sign_in; fz.scale_out = scale_de;
    launch_spans<false>(de, a, da, e, indptr, edge_ids, rows, nnz, static_cast<int>(H), slope, workspace,
                        as_stream(stream), fz);
    return launch_status();
}

int tango_edge_softmax_bwd(float* de, const float* a, const float* da, const float* e,
                           const int64_t* indptr, const int64_t* edge_ids, int64_t rows, int64_t nnz,
                           int64_t H, float slope, void* workspace, size_t workspace_bytes,
                           tango_stream_t stream) {
    if (rows < 0 || nnz < 0 || H < 0 || (rows > 0 && !indptr) || H >= (1LL << 31)) return TANGO_ERR_INVALID_ARG;
    if (rows * H == 0 || nnz == 0) return TANGO_OK;
    if (!de || !a || !da || (!e && slope != 1.0f)) return TANGO_ERR_INVALID_ARG;
    if (workspace && ceil_div(nnz, 4 * 128) <= INT32_MAX && ceil_div(H, 8) <= 65535) {
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
