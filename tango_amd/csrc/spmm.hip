// Quantized SpMM family for gfx950: copy_u (CSR), u_mul_e (CSR, int8 edge
// values, optional fused edge-id permutation) and copy_e (sorted incidence COO).
//
// These are gather kernels bound by the memory system, not by arithmetic, so
// no MFMA is used.  Layout of the work:
//   * a wavefront owns one output row and walks that row's CSR slots (4 waves for
//     long rows of wide pieces, 16 waves for rows far above the average, several
//     workgroups for hub rows, a lane group per row on sparse graphs: see the
//     kernels below);
//   * column indices are fetched 256 slots at a time with four independent
//     coalesced 512-byte loads (lane i of load r holds slot 64 r + i) and handed
//     to the lanes that need them with ds_bpermute, so index traffic is read
//     exactly once and one HBM round trip is paid per 256 edges;
//   * a group of `lpe` lanes (power of two) covers one gathered int8 feature
//     row with 16-, 4- or 1-byte loads per lane, so one load instruction of
//     the wavefront pulls 64/lpe neighbour rows (128-byte pieces -> 8 rows,
//     F = 16 -> 64 rows); a matrix far beyond the L2 is walked in 128-byte column
//     tiles, one tile after the other;
//   * a lane always has four gathers (four neighbours, same columns) in flight;
//     their dwords are byte-transposed with v_perm and added into int32 lane
//     accumulators four neighbours at a time with one v_dot4 against a byte
//     vector of multipliers (1 for copy_u, the int8 edge values for u_mul_e,
//     0 for slots past the row's end): 0.75 VALU ops per gathered byte, exact
//     integer arithmetic, order-independent;
//   * the lane groups are folded with ds_bpermute shuffles, the waves of a
//     workgroup through LDS, and the row leaves as fp32 = scale * float(sum).
#include "common.hpp"
#include "spmm_dense.hpp"

namespace tango {

struct SpmmParams {
    float* out;
    const int64_t* indptr;    // CSR kinds: [rows + 1]
    const int64_t* node_ids;  // COO kind: [nnz], sorted
    const int64_t* indices;   // gathered row per slot (COO kind: the edge ids)
    const int64_t* edge_ids;  // weighted kind: slot -> position in evals, or null
    const int8_t* feat;
    const int8_t* evals;
    const float* evals_f32;  // weighted kind, instead of evals: fp32 edge values, rounded to int8 (half to even,
                             // scale scale2[0]) as they are loaded; same strides, counted in elements
    const float* scale;
    const float* scale2;     // optional second factor of the dequantization scale (s = scale[0] * scale2[0])
    const float* row_scale;  // optional: out row r is multiplied by row_scale[r] after dequantization
    const float* bias;       // optional: bias[c] added after the row scale
    int relu;                // activation applied last: 0 none, 1 max(y, 0), 2 ELU (y > 0 ? y : exp(y) - 1)
    uint16_t* sign_bits;     // optional, VEC == 16 and W % 16 == 0: bit c % 16 of word [r, c / 16] = (out[r, c] > 0)
    int64_t rows;
    int64_t num_src;  // rows of the gathered matrix
    int64_t ldf;  // bytes between gathered rows
    int64_t W;    // bytes summed per gathered row (H * F)
    int64_t F;    // bytes per head
    int64_t D;    // edge-value width (1 or F)
    int64_t ev_sh, ev_sd, ev_se;  // strides (bytes) of evals over head, value column, edge
    int64_t nnz;
    int lpe_log2;  // log2(lanes per gathered row piece)
    int64_t tile;  // bytes of a gathered row one workgroup column (blockIdx.y) covers: lanes per piece * VEC
    int ldf_shift; // log2(ldf) when ldf is a power of two and all byte offsets fit 31 bits, else -1
    int out_vec;   // out rows may be stored as 16-byte vectors
    int idx32;     // indices and edge_ids point to int32 arrays (half the index traffic); indptr stays int64
    int64_t long_row;  // rows with more slots than this go to the sixteen-wave kernel
    int64_t hub_row;   // rows with more slots than this are cut over several workgroups
    void* hub_ws;      // caller's workspace for the hub path, or null (then no row counts as a hub)
    int64_t max_row;   // caller's upper bound of the longest row, 0 if unknown
    int64_t group_row; // sparse graphs: rows with at most this many slots are owned by a lane group
    void* span_ws;     // sparse graphs: caller's workspace for the slot-span path, or null
    int64_t span_wp;   // padded row width (int32 entries) of a partial row in span_ws
    size_t span_ws_bytes;
    const int* part;       // optional int32 partial sums added to a row's sum before dequantization (the dense
    const int* part_slot;  // blocks of spmm_dense.hip): row r owns row part_slot[r] of part (stride part_ld ints)
    int part_ld;           // when that is not negative
    float* amax_part;      // optional: [rows][amax_tiles] receives max |out * amax_mul[row]| of every row piece stored
    const float* amax_mul; // (amax_mul optional), from which amax_reduce_kernel forms the scale of the output
    int amax_tiles;
    float* amax_scale;     // where amax_reduce_kernel maxes the scale into (holds 0 or a partial result on entry)
    const int* row_order;  // optional: workgroups take rows in this order (rows of similar length side by side,
                           // whatever the numbering of the nodes) instead of by row number
};

enum { KIND_COPY = 0, KIND_WEIGHTED = 1, KIND_COO = 2, KIND_WEIGHTED_F32 = 3 };
// weighted kinds: int8 edge values, or fp32 edge values rounded as they are loaded (a kind of its own, so that the
// int8 path carries no test for it: on 8-byte rows a uniform branch per slot cost 16 % of the launch)
__host__ __device__ constexpr bool weighted(int kind) { return kind == KIND_WEIGHTED || kind == KIND_WEIGHTED_F32; }

// Byte offset of gathered row j: a shift when the row pitch allows (64-bit multiplies are quarter rate).
__device__ __forceinline__ int64_t row_offset(int j, const SpmmParams& p) {
    return p.ldf_shift >= 0 ? static_cast<int64_t>(static_cast<uint32_t>(j) << p.ldf_shift)
                            : static_cast<int64_t>(j) * p.ldf;
}

template <int VEC>
struct Gather;
template <>
struct Gather<16> {
    using T = u32x4;
    static __device__ __forceinline__ T load(const int8_t* p) { return *reinterpret_cast<const T*>(p); }
    static __device__ __forceinline__ T zero() { return T{0u, 0u, 0u, 0u}; }
};
template <>
struct Gather<4> {
    using T = uint32_t;
    static __device__ __forceinline__ T load(const int8_t* p) { return *reinterpret_cast<const T*>(p); }
    static __device__ __forceinline__ T zero() { return 0u; }
};
template <>
struct Gather<1> {
    using T = int;
    static __device__ __forceinline__ T load(const int8_t* p) { return static_cast<int>(*p); }
    static __device__ __forceinline__ T zero() { return 0; }
};

// Accumulates the four gathered pieces d[0..3] (same columns, four different neighbours) into the
// lane's int32 column sums.  Each group of four dwords is transposed with v_perm so that one dword
// holds ONE column of FOUR neighbours, and a single v_dot4 against `m` adds all four: byte u of `m`
// is neighbour u's multiplier (1, 0 for an invalid slot, or the int8 edge value of u_mul_e).
// 8 v_perm + 4 v_dot4 per 16 gathered bytes, instead of 16 v_dot4 with one-hot masks.
template <int VEC>
__device__ __forceinline__ void accumulate4(int* acc, const typename Gather<VEC>::T* d, uint32_t m);
template <>
__device__ __forceinline__ void accumulate4<16>(int* acc, const u32x4* d, uint32_t m) {
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        uint32_t c[4];
        transpose4x4(d[0][w], d[1][w], d[2][w], d[3][w], c);
#pragma unroll
        for (int j = 0; j < 4; ++j)
            acc[4 * w + j] = __builtin_amdgcn_sdot4(static_cast<int>(c[j]), static_cast<int>(m), acc[4 * w + j], false);
    }
}
template <>
__device__ __forceinline__ void accumulate4<4>(int* acc, const uint32_t* d, uint32_t m) {
    uint32_t c[4];
    transpose4x4(d[0], d[1], d[2], d[3], c);
#pragma unroll
    for (int j = 0; j < 4; ++j)
        acc[j] = __builtin_amdgcn_sdot4(static_cast<int>(c[j]), static_cast<int>(m), acc[j], false);
}
template <>
__device__ __forceinline__ void accumulate4<1>(int* acc, const int* d, uint32_t m) {
#pragma unroll
    for (int u = 0; u < 4; ++u)
        acc[0] += d[u] * static_cast<int>(static_cast<int8_t>(m >> (8 * u)));
}

__device__ __forceinline__ int64_t lower_bound_i64(const int64_t* a, int64_t n, int64_t key) {
    int64_t lo = 0, hi = n;
    while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if (a[mid] < key) lo = mid + 1; else hi = mid;
    }
    return lo;
}

// Entry i of an index array that is int64, or int32 when p.idx32 is set.  `stream`: the array is read
// once front to back (nontemporal: it should not evict gathered rows from the L2).
template <bool STREAM>
__device__ __forceinline__ int load_index(const SpmmParams& p, const int64_t* a, int64_t i) {
    if (p.idx32) {
        const int* a32 = reinterpret_cast<const int*>(a);
        return STREAM ? __builtin_nontemporal_load(a32 + i) : a32[i];
    }
    return static_cast<int>(STREAM ? __builtin_nontemporal_load(a + i) : a[i]);
}

// Per-lane view of the column tile a lane works on.
struct LaneCols {
    int lpe, epi, grp, sub, sh;
    int64_t col;
    bool col_ok;
    const int8_t* fcol;   // feat + col (column 0 for lanes past the row's width)
    const int8_t* wbase;  // weighted kind: evals + this lane's head / value-column offset
    const float* wbase_f;  // the same for fp32 edge values that are quantized on load
    float ev_r;            // 1 / their scale
};

// The int8 edge value at position pos (in units of ev_se) as the multiplier byte of a v_dot4.
template <int KIND>
__device__ __forceinline__ uint32_t edge_value(const SpmmParams& p, const LaneCols& c, int64_t pos) {
    if (KIND == KIND_WEIGHTED_F32)
        return static_cast<uint32_t>(quant_one<TANGO_ROUND_RNE>(c.wbase_f[pos * p.ev_se], c.ev_r, 0.0f)) & 0xffu;
    return static_cast<uint32_t>(static_cast<uint8_t>(c.wbase[pos * p.ev_se]));
}

template <int VEC, int KIND>
__device__ __forceinline__ LaneCols lane_cols(const SpmmParams& p, int lane) {
    LaneCols c;
    c.lpe = 1 << p.lpe_log2;
    c.epi = kWave >> p.lpe_log2;
    c.grp = lane >> p.lpe_log2;
    c.sub = lane & (c.lpe - 1);
    c.sh = 6 - p.lpe_log2;
    c.col = static_cast<int64_t>(blockIdx.y) * p.tile + static_cast<int64_t>(c.sub) * VEC;
    c.col_ok = c.col < p.W;
    // Lanes past the row's width read column 0 (a valid address) and never store, and the
    // group fold only mixes lanes of equal `sub`, so they need no masking.
    c.fcol = p.feat + (c.col_ok ? c.col : 0);
    c.wbase = p.evals;
    c.wbase_f = p.evals_f32;
    c.ev_r = 0.0f;
    if (weighted(KIND) && c.col_ok) {
        const int64_t h = c.col / p.F;
        const int64_t d = (p.D == 1) ? 0 : (c.col - h * p.F);
        c.wbase = p.evals + h * p.ev_sh + d * p.ev_sd;
        if (KIND == KIND_WEIGHTED_F32) {
            c.wbase_f = p.evals_f32 + h * p.ev_sh + d * p.ev_sd;
            c.ev_r = rscale_of(p.scale2[0]);
        }
    }
    return c;
}

// One wavefront sums the gathered rows of CSR slots [start, end) (row_start is the row's first
// slot: edge values in slot order are addressed relative to the whole array).  On return lanes
// [0, lpe) hold the column sums of the lane's VEC columns.
template <int VEC, int KIND>
__device__ __forceinline__ void wave_row_sum(const SpmmParams& p, const LaneCols& c, int lane, int64_t start,
                                             int64_t end, int* acc) {
    constexpr int U = 4;  // gather loads in flight per lane
    const int lpe = c.lpe, epi = c.epi, grp = c.grp, sh = c.sh;
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0;

    // Indices are fetched 256 slots at a time with four independent coalesced loads
    // (lane i of load r holds slot 64 r + i), so one HBM round trip is paid per 256 edges.
    for (int64_t base = start; base < end; base += 4 * kWave) {
        int my[4], my_e[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int64_t q = base + r * kWave + lane;
            const int64_t qc = q < end ? q : end - 1;  // clamped: the load is unconditional
            // streamed once: keep the index array from evicting feature rows out of L2
            const int v = load_index<true>(p, p.indices, qc);
            my[r] = q < end ? v : -1;
            my_e[r] = 0;
            if (weighted(KIND) && p.edge_ids)
                my_e[r] = load_index<true>(p, p.edge_ids, qc);
        }
        // The 256 slots are walked as one flat sequence of steps (64 / lpe slots each), always
        // U steps per batch, so narrow rows (one step per 64 slots) keep U gathers in flight too.
        const int cnt = static_cast<int>((end - base) < 4 * kWave ? (end - base) : 4 * kWave);
        const int total = (cnt + epi - 1) >> sh;
        for (int t = 0; t < total; t += U) {
            int j[U];
            int64_t sl[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int tt = t + u;
                const int r = (tt >> p.lpe_log2) & 3;  // which of the four index registers (wave-uniform)
                const int slot = ((tt & (lpe - 1)) << sh) + grp;
                const int reg = r == 0 ? my[0] : r == 1 ? my[1] : r == 2 ? my[2] : my[3];
                j[u] = __shfl(reg, slot, kWave);
                sl[u] = 0;
                if (weighted(KIND)) {
                    const int rege = r == 0 ? my_e[0] : r == 1 ? my_e[1] : r == 2 ? my_e[2] : my_e[3];
                    // position of this slot's edge value: permuted id, or the CSR slot itself
                    sl[u] = p.edge_ids ? static_cast<int64_t>(__shfl(rege, slot, kWave)) : base + r * kWave + slot;
                }
            }
            typename Gather<VEC>::T d[U];
            uint32_t m = 0u;  // byte u: multiplier of neighbour u (0 = slot not valid)
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const bool ok = (t + u) < total && j[u] >= 0;
                // invalid slots read row 0 with multiplier 0: no branch around the load
                d[u] = Gather<VEC>::load(c.fcol + row_offset(ok ? j[u] : 0, p));
                uint32_t w = 1u;
                if (weighted(KIND))
                    w = edge_value<KIND>(p, c, ok ? sl[u] : 0);
                m |= (ok ? w : 0u) << (8 * u);
            }
            accumulate4<VEC>(acc, d, m);
        }
    }

    // fold the lane groups: afterwards lanes [0, lpe) hold the wave's column sums
    for (int off = lpe; off < kWave; off <<= 1) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] += __shfl_xor(acc[i], off, kWave);
    }
}

__device__ __forceinline__ float activate(float y, int act) {
    if (act == 1) return fmaxf(y, 0.0f);
    // the hardware exponential: exp(y) - 1 carries an absolute error of about 1e-7 for y <= 0 (the library's
    // expm1f is some forty instructions, which these epilogues run under divergence, once per finished row)
    if (act == 2) return y > 0.0f ? y : __expf(y) - 1.0f;
    return y;
}

// The signs of a lane's sixteen consecutive outputs as one 16-bit word (what a backward pass needs of a ReLU's
// output: 1/32 of its bytes).
template <int VEC>
__device__ __forceinline__ void store_sign_bits(const SpmmParams& p, int64_t row, int64_t col, const float* y) {
    unsigned b = 0;
#pragma unroll
    for (int i = 0; i < VEC; ++i) b |= (y[i] > 0.0f ? 1u : 0u) << (i & 15);
    p.sign_bits[row * (p.W >> 4) + (col >> 4)] = static_cast<uint16_t>(b);
}

// Dequantize and store one output row's tile; called by all lanes of one lane group (grp == 0 in the row kernels).
template <int VEC, bool AMAX>
__device__ __forceinline__ float store_row_piece(const SpmmParams& p, const LaneCols& c, int64_t row, const int* acc) {
    const float s = p.scale2 ? p.scale[0] * p.scale2[0] : p.scale[0];
    const float rs = p.row_scale ? p.row_scale[row] : 1.0f;
    float* o = p.out + row * p.W + c.col;
    int extra[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) extra[i] = 0;
    if (p.part) {  // uniform
        const int slot = p.part_slot[row];
        if (slot >= 0) {
            const int* pr = p.part + static_cast<int64_t>(slot) * p.part_ld + c.col;  // rows padded: no column guard
            if (VEC == 16) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const i32x4 v = reinterpret_cast<const i32x4*>(pr)[i];
                    extra[4 * i] = v[0]; extra[4 * i + 1] = v[1]; extra[4 * i + 2] = v[2]; extra[4 * i + 3] = v[3];
                }
            } else {
#pragma unroll
                for (int i = 0; i < VEC; ++i) extra[i] = pr[i];
            }
        }
    }
    float y[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
        // same sequence of roundings as dequantize, then "* norm", "+ bias", relu as separate passes
        y[i] = s * static_cast<float>(acc[i] + extra[i]);
        if (p.row_scale) y[i] = y[i] * rs;
        if (p.bias && c.col + i < p.W) y[i] = y[i] + p.bias[c.col + i];
    }
    if (p.relu) {  // uniform: rows without an activation skip its instructions altogether
#pragma unroll
        for (int i = 0; i < VEC; ++i) y[i] = activate(y[i], p.relu);
    }
    float m = 0.0f;
    if (AMAX) {
        const float mul = p.amax_mul ? p.amax_mul[row] : 1.0f;
#pragma unroll
        for (int i = 0; i < VEC; ++i)
            if (c.col + i < p.W) m = fmaxf(m, fabsf(y[i] * mul));  // * 1.0f is exact
    }
    if (VEC == 16 && p.out_vec && c.col + 16 <= p.W) {
        f32x4* o4 = reinterpret_cast<f32x4*>(o);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            __builtin_nontemporal_store(f32x4{y[4 * i], y[4 * i + 1], y[4 * i + 2], y[4 * i + 3]}, o4 + i);
    } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i)
            if (c.col + i < p.W) o[i] = y[i];
    }
    // after the row's own stores, so that the sixteen values need not all be live at once
    if (VEC == 16 && p.sign_bits) store_sign_bits<VEC>(p, row, c.col, y);
    return m;
}

// AMAX: also leave max |out * amax_mul[row]| of the piece in p.amax_part.  A variant of its own: the few registers
// it takes cost the row kernel one of its eight waves per SIMD, so kernels are built with it only where asked.
template <int VEC, bool AMAX = false>
__device__ __forceinline__ void store_row(const SpmmParams& p, const LaneCols& c, int64_t row, const int* acc) {
    float m = 0.0f;
    if (c.col_ok) m = store_row_piece<VEC, AMAX>(p, c, row, acc);
    if (AMAX) {  // the lanes of the piece are all here, also those past the row's width
        for (int off = c.lpe >> 1; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, kWave));
        if (c.sub == 0) p.amax_part[row * p.amax_tiles + blockIdx.y] = m;
    }
}

// scale[0] = max(scale[0], max(part[0 .. n)) / 127): scale must hold 0 (or an earlier partial result) on entry.
// x -> fl(x / 127) is monotone, so the maximum of the workgroups' quotients is the quotient of the maximum.
__global__ __launch_bounds__(256) void amax_reduce_kernel(const float* __restrict__ part, int64_t n, float* scale) {
    float m = 0.0f;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * 256)
        m = fmaxf(m, part[i]);
    __shared__ float w[4];
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) w[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        m = fmaxf(fmaxf(w[0], w[1]), fmaxf(w[2], w[3]));
        atomicMax(reinterpret_cast<int*>(scale), __float_as_int(m / 127.0f));
    }
}

template <int KIND>
__device__ __forceinline__ void row_range(const SpmmParams& p, int64_t row, int64_t& start, int64_t& end) {
    if (KIND == KIND_COO) {
        start = lower_bound_i64(p.node_ids, p.nnz, row);
        end = lower_bound_i64(p.node_ids, p.nnz, row + 1);
    } else {
        start = p.indptr[row];
        end = p.indptr[row + 1];
    }
}

// lower_bound by all 64 lanes of a converged wavefront: 64 probes per round, so
// at most six dependent loads for 2^31 entries instead of 31.
__device__ __forceinline__ int64_t lower_bound_wave(const int64_t* a, int64_t n, int64_t key, int lane) {
    int64_t lo = 0, hi = n;  // the answer lies in [lo, hi]
    while (lo < hi) {
        const int64_t step = (hi - lo + kWave - 1) >> 6;
        const int64_t idx = lo + (lane + 1) * step - 1;
        const bool below = idx < hi && a[idx] < key;
        const int cnt = __popcll(__ballot(below));  // probes are sorted: the first cnt are below the key
        const int64_t nlo = lo + cnt * step;
        const int64_t nhi = lo + (cnt + 1) * step - 1;
        lo = nlo;
        hi = nhi < hi ? nhi : hi;
    }
    return lo;
}

// blockDim.x = 256.  WPR = waves that share one output row (1 or 4).
// gridDim.y tiles the columns in chunks of p.tile bytes.
// Rows with more than p.long_row slots are left to spmm_long_kernel.
template <int VEC, int WPR, int KIND, bool AMAX = false>
__global__ __launch_bounds__(256) void spmm_kernel(const SpmmParams p) {
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 6);
    int64_t row = (WPR == 4) ? static_cast<int64_t>(blockIdx.x)
                             : static_cast<int64_t>(blockIdx.x) * 4 + wave;
    __shared__ int part[(WPR == 4) ? 3 * 64 * VEC : 1];
    if (WPR == 1 && row >= p.rows) return;  // whole wave leaves; no barrier follows for WPR == 1
    if (p.row_order) row = p.row_order[row];

    int64_t start, end;
    if (KIND == KIND_COO) {
        start = lower_bound_wave(p.node_ids, p.nnz, row, lane);
        end = lower_bound_wave(p.node_ids, p.nnz, row + 1, lane);
    } else {
        row_range<KIND>(p, row, start, end);
    }
    if (end - start > p.long_row) return;  // uniform over the workgroup
    if (WPR == 4) {
        const int64_t per = (end - start + 3) >> 2;
        const int64_t s = start + per * wave;
        const int64_t e = s + per;
        start = s < end ? s : end;
        end = e < end ? e : end;
    }

    const LaneCols c = lane_cols<VEC, KIND>(p, lane);
    int acc[VEC];
    wave_row_sum<VEC, KIND>(p, c, lane, start, end, acc);

    if (WPR == 4) {
        if (wave > 0 && c.grp == 0) {
#pragma unroll
            for (int i = 0; i < VEC; ++i) part[(wave - 1) * 64 * VEC + i * 64 + c.sub] = acc[i];
        }
        __syncthreads();
        if (wave > 0) return;
        if (c.grp == 0) {
#pragma unroll
            for (int i = 0; i < VEC; ++i)
                acc[i] += part[i * 64 + c.sub] + part[64 * VEC + i * 64 + c.sub] + part[2 * 64 * VEC + i * 64 + c.sub];
        }
    }
    if (c.grp == 0) store_row<VEC, AMAX>(p, c, row, acc);
}

// copy_u on column tiles of at most 128 bytes (a slot's piece of a gathered row takes 1 .. 8 lanes) when the rows come
// ordered by length (p.row_order of a dense-block plan): a wavefront that owns one row spends about as many
// instructions on what a row costs whatever its length (index round trip, the fold over its eight or more slot
// groups, the epilogue) as on the slots themselves.  Here 2^RL lanes own a row, 64 >> RL rows to a wavefront: a
// gather instruction serves (1 << RL) / lpe slots of each of those rows, the fold has RL - log2(lpe) stages, and
// prologue and epilogue run once for all of them.  Neighbouring rows in that order are about equally long, so they
// finish together.  Rows above p.long_row are left to spmm_long_kernel, as in spmm_kernel.  U gathers in flight per
// lane.  Measured on the rest of the 114.8 M-edge benchmark graph (232,965 rows of 72 .. 777 slots), per
// aggregation call, against a wavefront per row: RL = 4 (sixteen lanes, four rows) 256 columns 1.467 -> 1.378 ms,
// 128 columns 0.770 -> 0.719, 41 columns 0.563 -> 0.533; RL = 5 1.393 / 0.727; RL = 3 1.48 / 0.75 (41 columns:
// 0.556); RL = 6 (this kernel with a row per wavefront) as spmm_kernel.  With RL = 4: U = 8 +20 us at 256 columns;
// the next batch's indices fetched a batch ahead +25 us; held to eight waves per SIMD by a launch bound (66 VGPRs
// otherwise: seven) +17 us at 41 columns (spills).  blockDim.x = 256; gridDim.x = ceil(rows / (4 * (64 >> RL)));
// gridDim.y tiles the columns.
// LPL = log2 of the lanes per slot, fixed at compile time for tiles of at most 64 bytes (the slot -> index register
// mapping and the fold then are too), or -1: read from p, the form the 128-byte tiles run (their launch moves its
// misses at the fabric's rate, and the leaner instruction stream of a fixed LPL = 3 was measured slower there:
// 1.43 against 1.37 ms per 256-column call; 41 columns with LPL = 2: 0.509 against 0.536).  SHIFT (with LPL >= 0):
// the rows of the gathered matrix are a power of two bytes apart and the whole matrix below 2 GiB
// (p.ldf_shift >= 0), which makes a gather's address a 32-bit offset from one base for the whole wavefront.
template <int RL, int LPL, bool SHIFT>
__global__ __launch_bounds__(256) void spmm_quad_kernel(const SpmmParams p) {
    constexpr int VEC = 16, U = 4, SEGL = 1 << RL;  // SEGL lanes own a row
    const int lpl = LPL >= 0 ? LPL : p.lpe_log2;
    const int sh = RL - lpl;   // log2 of the slots a row advances per step
    const int lpe = 1 << lpl;  // lanes per slot
    const int lane = lane_id();
    const int wave = static_cast<int>(threadIdx.x) >> 6;
    const int seg = lane >> RL, sl = lane & (SEGL - 1);
    LaneCols c;
    c.lpe = lpe;
    c.epi = 1 << sh;
    c.sub = sl & (lpe - 1);
    c.grp = sl >> lpl;  // slot group inside the row's lanes
    c.sh = sh;
    c.col = static_cast<int64_t>(blockIdx.y) * p.tile + static_cast<int64_t>(c.sub) * VEC;
    c.col_ok = c.col < p.W;
    c.fcol = p.feat + (c.col_ok ? c.col : 0);  // lanes past the row's width read a valid piece and never store
    c.wbase = nullptr;
    c.wbase_f = nullptr;
    c.ev_r = 0.0f;
    // SHIFT: address = tile base (the same for all lanes) + a 32-bit lane offset
    const int8_t* tile_base = p.feat + static_cast<int64_t>(blockIdx.y) * p.tile;
    const uint32_t lane_off = c.col_ok ? static_cast<uint32_t>(c.sub) * VEC : 0u;  // (past the width: the tile's first piece)

    const int64_t pos = (static_cast<int64_t>(blockIdx.x) * 4 + wave) * (kWave >> RL) + seg;
    const bool live = pos < p.rows;
    int64_t row = live ? pos : p.rows - 1;
    if (p.row_order) row = p.row_order[row];
    const int64_t start = p.indptr[row];
    int64_t len = p.indptr[row + 1] - start;
    const bool mine = live && len <= p.long_row;
    if (!mine) len = 0;
    const int n = static_cast<int>(len);
    int nmax = n;  // the longest of the wavefront's rows
    for (int off = SEGL; off < kWave; off <<= 1) {
        const int other = __shfl_xor(nmax, off, kWave);
        nmax = other > nmax ? other : nmax;
    }
    const int src_lane = (seg << RL) | c.grp;  // lane that holds the index of this lane group's slot of step 0

    int acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0;
    // indices: 4 SEGL slots of every row at a time, four coalesced loads per lane (lane sl of load r holds slot
    // SEGL r + sl); slots past the row's end hold -1
    for (int base = 0; base < nmax; base += 4 * SEGL) {
        int my[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int q = base + r * SEGL + sl;
            const bool ok = q < n;
            // clamped: the load is unconditional (a row without slots reads the array's first entry)
            const int64_t qc = ok ? start + q : (n > 0 ? start + n - 1 : 0);
            const int v = load_index<true>(p, p.indices, qc);
            my[r] = ok ? v : -1;
        }
        const int cnt = nmax - base < 4 * SEGL ? nmax - base : 4 * SEGL;
        const int total = (cnt + c.epi - 1) >> sh;  // steps of this batch; a step past it finds -1 everywhere
        for (int t = 0; t < total; t += U) {
            int j[U];
            if (LPL >= 2) {
                // the four steps of a round take their slots from one index register
                const int r = (t << sh) >> RL;  // wave-uniform
                const int reg = r == 0 ? my[0] : r == 1 ? my[1] : r == 2 ? my[2] : my[3];
#pragma unroll
                for (int u = 0; u < U; ++u)
                    j[u] = __shfl(reg, src_lane + (((t + u) << sh) & (SEGL - 1)), kWave);
            } else {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int r = ((t + u) << sh) >> RL;  // wave-uniform
                    const int reg = r == 0 ? my[0] : r == 1 ? my[1] : r == 2 ? my[2] : my[3];
                    j[u] = __shfl(reg, src_lane + (((t + u) << sh) & (SEGL - 1)), kWave);
                }
            }
            typename Gather<VEC>::T d[U];
            uint32_t m = 0u;  // byte u: 1 where neighbour u counts
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const bool ok = LPL >= 0 ? j[u] >= 0 : ((t + u) < total && j[u] >= 0);
                const int jj = ok ? j[u] : 0;  // row 0 with multiplier 0: no branch around the load
                if (LPL >= 0 && SHIFT)
                    d[u] = Gather<VEC>::load(tile_base + ((static_cast<uint32_t>(jj) << p.ldf_shift) + lane_off));
                else if (LPL >= 0)
                    d[u] = Gather<VEC>::load(c.fcol + static_cast<int64_t>(jj) * p.ldf);
                else
                    d[u] = Gather<VEC>::load(c.fcol + row_offset(jj, p));
                m |= (ok ? 1u : 0u) << (8 * u);
            }
            accumulate4<VEC>(acc, d, m);
        }
    }
    // fold the row's slot groups: afterwards its lanes [0, lpe) hold the column sums
    for (int off = lpe; off < SEGL; off <<= 1) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] += __shfl_xor(acc[i], off, kWave);
    }
    if (mine && c.grp == 0 && c.col_ok) store_row_piece<VEC, false>(p, c, row, acc);
}

// Sparse graphs (a handful of neighbours per row): a wavefront that owns one row would leave most
// of its gather slots empty and the launch would be bound by per-wave latency chains.  Here every
// group of `lpe` lanes owns a row of its own (64 / lpe rows per wavefront) and walks it four
// neighbours at a time; rows with more than p.group_row slots are left to spmm_medium_kernel.
constexpr int kGroupRow = 32;  // most slots of a row that a lane group owns

template <int VEC, int KIND>
__global__ __launch_bounds__(256) void spmm_group_kernel(const SpmmParams p) {
    constexpr int U = 4;
    // a wave's groups stage their rows' column indices (and edge ids) here, so that the gather loop
    // holds no dependent index load; used when a wave has at most 16 groups
    __shared__ int sidx[4][16 * kGroupRow];
    __shared__ int seid[weighted(KIND) ? 4 : 1][weighted(KIND) ? 16 * kGroupRow : 1];
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 6);
    const LaneCols c = lane_cols<VEC, KIND>(p, lane);
    const int64_t row = ((static_cast<int64_t>(blockIdx.x) * 4 + wave) << c.sh) + c.grp;
    int64_t start = 0, end = 0;
    if (row < p.rows) {
        start = p.indptr[row];
        end = p.indptr[row + 1];
    }
    const bool mine = row < p.rows && end - start <= kGroupRow;
    const int deg = mine ? static_cast<int>(end - start) : 0;
    const bool staged = p.lpe_log2 >= 2;
    const bool permuted = weighted(KIND) && p.edge_ids;
    if (staged) {
        for (int k = c.sub; k < deg; k += c.lpe) {
            sidx[wave][(c.grp << 5) + k] = load_index<false>(p, p.indices, start + k);
            if (permuted) seid[weighted(KIND) ? wave : 0][(c.grp << 5) + k] = load_index<false>(p, p.edge_ids, start + k);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    int acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0;
    // four gathers of slots q .. q + 3 (slots past the row's end read its first neighbour with multiplier 0)
    auto issue = [&](typename Gather<VEC>::T* d, uint32_t& m, int q) {
        m = 0u;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const bool ok = q + u < deg;
            const int slot = ok ? q + u : 0;
            const int j = staged ? sidx[wave][(c.grp << 5) + slot] : load_index<false>(p, p.indices, start + slot);
            d[u] = Gather<VEC>::load(c.fcol + row_offset(j, p));
            uint32_t w = 1u;
            if (weighted(KIND)) {
                int64_t pos = start + slot;
                if (permuted)
                    pos = staged ? seid[weighted(KIND) ? wave : 0][(c.grp << 5) + slot]
                                 : load_index<false>(p, p.edge_ids, start + slot);
                w = edge_value<KIND>(p, c, pos);
            }
            m |= (ok ? w : 0u) << (8 * u);
        }
    };
    // two batches in flight: the next one is issued before the current one is consumed
    typename Gather<VEC>::T da[U], db[U];
    uint32_t ma = 0u, mb = 0u;
    if (deg > 0) issue(da, ma, 0);
    for (int q = 0; q < deg; q += 2 * U) {  // trip counts differ between the groups of a wave
        const bool has_b = q + U < deg;
        if (has_b) issue(db, mb, q + U);
        accumulate4<VEC>(acc, da, ma);
        if (q + 2 * U < deg) issue(da, ma, q + 2 * U);
        if (has_b) accumulate4<VEC>(acc, db, mb);
    }
    if (mine) store_row<VEC>(p, c, row, acc);
}

// Rows with more than p.group_row and at most p.long_row slots of a sparse graph, one wavefront
// per row.  Wavefront w of the launch inspects rows w, w + W, ... (kRowsPerWave of them, W =
// wavefronts launched) and walks the ones of this tier in turn.
constexpr int kRowsPerWave = 8;

template <int VEC, int KIND>
__global__ __launch_bounds__(256) void spmm_medium_kernel(const SpmmParams p) {
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 6);
    const int64_t nwaves = static_cast<int64_t>(gridDim.x) * 4;
    const int64_t w = static_cast<int64_t>(blockIdx.x) * 4 + wave;
    const int64_t mine = w + static_cast<int64_t>(lane) * nwaves;
    int64_t q0 = 0, q1 = 0;
    if (lane < kRowsPerWave && mine < p.rows) {
        q0 = p.indptr[mine];
        q1 = p.indptr[mine + 1];
    }
    uint64_t todo = __ballot(q1 - q0 > p.group_row && q1 - q0 <= p.long_row);
    if (!todo) return;
    const LaneCols c = lane_cols<VEC, KIND>(p, lane);
    while (todo) {
        const int l = __builtin_ctzll(todo);
        todo &= todo - 1;
        const int64_t start = __shfl(q0, l, kWave), end = __shfl(q1, l, kWave);
        int acc[VEC];
        wave_row_sum<VEC, KIND>(p, c, lane, start, end, acc);
        if (c.grp == 0) store_row<VEC>(p, c, w + static_cast<int64_t>(l) * nwaves, acc);
    }
}

// Rows with more than p.long_row slots, sixteen wavefronts per row.  blockDim.x = 1024, a
// fixed number of workgroups (G = gridDim.x): thread t of workgroup b inspects row b + G * t
// (then b + G * (1024 + t), ...; hub rows with neighbouring ids land in different workgroups),
// the long ones are collected in LDS and each is summed by all waves; the waves' partial sums
// meet in LDS through integer atomics, which are exact in any order.
//
// Hub rows (more than p.hub_row slots; needs the caller's workspace) would still keep one
// workgroup busy long after the rest of the launch has drained.  This kernel only records them in
// the workspace's list and zeroes their output rows, viewed as int32; spmm_hub_sum_kernel then
// cuts every hub row into chunks of kHubChunk slots, deals all chunks over its workgroups, and adds
// each chunk's int32 sums into the output row with integer atomics (exact in any order), and
// spmm_hub_store_kernel turns the int32 sums into the fp32 result in place.
constexpr int kLongGrid = 512;
constexpr int kHubChunk = 2048;      // slots per chunk of a hub row: 128 per wave
constexpr int64_t kHubRowMin = 4096; // no row shorter than this is ever treated as a hub
constexpr int kHubSumGrid = 256;
constexpr int kHubBatch = 2048;      // hub rows whose chunk counts a workgroup scans at a time

// workspace: word 0 = number of hub rows (zeroed by the library at the start of a call), byte 64.. = row ids
__device__ __forceinline__ int64_t* hub_list(void* ws) { return reinterpret_cast<int64_t*>(static_cast<char*>(ws) + 64); }

template <int VEC, int KIND>
__global__ __launch_bounds__(1024) void spmm_long_kernel(const SpmmParams p) {
    constexpr int WAVES = 16;
    __shared__ int part[64 * VEC];
    __shared__ int64_t list[1024];
    __shared__ int nlist;
    const int t = threadIdx.x;
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const LaneCols c = lane_cols<VEC, KIND>(p, lane);
    const int64_t G = gridDim.x;
    for (int i = t; i < 64 * VEC; i += 1024) part[i] = 0;
    for (int64_t first = blockIdx.x; first < p.rows; first += 1024 * G) {  // uniform trip count
        if (t == 0) nlist = 0;
        __syncthreads();
        const int64_t mine = first + G * t;
        if (mine < p.rows) {
            int64_t s, e;
            row_range<KIND>(p, mine, s, e);
            if (e - s > p.long_row) list[atomicAdd(&nlist, 1)] = mine;  // any order: rows are independent
        }
        __syncthreads();
        const int n = nlist;
        for (int k = 0; k < n; ++k) {
            const int64_t row = list[k];
            int64_t start, end;
            row_range<KIND>(p, row, start, end);
            if (end - start > p.hub_row) {  // uniform over the workgroup
                if (blockIdx.y == 0 && t == 0) hub_list(p.hub_ws)[atomicAdd(static_cast<int*>(p.hub_ws), 1)] = row;
                int* orow = reinterpret_cast<int*>(p.out) + row * p.W + c.col;  // this lane's VEC output columns
                if (wave == 0 && c.grp == 0 && c.col_ok) {
#pragma unroll
                    for (int i = 0; i < VEC; ++i)
                        if (c.col + i < p.W) orow[i] = 0;
                }
                continue;
            }
            const int64_t per = (end - start + WAVES - 1) / WAVES;
            const int64_t s = start + per * wave;
            const int64_t e = s + per;
            int acc[VEC];
            wave_row_sum<VEC, KIND>(p, c, lane, s < end ? s : end, e < end ? e : end, acc);
            if (c.grp == 0) {
#pragma unroll
                for (int i = 0; i < VEC; ++i) atomicAdd(&part[i * 64 + c.sub], acc[i]);
            }
            __syncthreads();
            if (wave == 0 && c.grp == 0) {
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    acc[i] = part[i * 64 + c.sub];
                    part[i * 64 + c.sub] = 0;
                }
                if (p.amax_part) store_row<VEC, true>(p, c, row, acc);  // uniform
                else store_row<VEC>(p, c, row, acc);
            }
            __syncthreads();
        }
    }
}

// blockDim.x = 1024, grid (kHubSumGrid, column tiles).  All chunks of all hub rows form one
// sequence (hub 0's chunks, hub 1's, ...); workgroup b takes chunks b, b + G, ...
template <int VEC, int KIND>
__global__ __launch_bounds__(1024) void spmm_hub_sum_kernel(const SpmmParams p) {
    constexpr int WAVES = 16;
    __shared__ int part[64 * VEC];
    __shared__ int first_chunk[kHubBatch + 1];  // exclusive prefix sums of the batch's chunk counts
    __shared__ int wsum[WAVES];
    const int t = threadIdx.x;
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const LaneCols c = lane_cols<VEC, KIND>(p, lane);
    const int nhub = *static_cast<const int*>(p.hub_ws);
    const int64_t* hubs = hub_list(p.hub_ws);
    for (int i = t; i < 64 * VEC; i += 1024) part[i] = 0;
    for (int h0 = 0; h0 < nhub; h0 += kHubBatch) {  // uniform trip count
        const int nb = nhub - h0 < kHubBatch ? nhub - h0 : kHubBatch;
        // chunk counts of hubs h0 + 2 t and h0 + 2 t + 1, then a workgroup-wide exclusive scan
        int cnt[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            cnt[u] = 0;
            const int h = 2 * t + u;
            if (h < nb) {
                int64_t s, e;
                row_range<KIND>(p, hubs[h0 + h], s, e);
                cnt[u] = static_cast<int>((e - s + kHubChunk - 1) / kHubChunk);
            }
        }
        int incl = cnt[0] + cnt[1];
        for (int off = 1; off < kWave; off <<= 1) {
            const int v = __shfl_up(incl, off, kWave);
            if (lane >= off) incl += v;
        }
        if (lane == kWave - 1) wsum[wave] = incl;
        __syncthreads();
        int base = 0;
        for (int w = 0; w < wave; ++w) base += wsum[w];
        const int excl = base + incl - cnt[0] - cnt[1];
        if (2 * t < kHubBatch) first_chunk[2 * t] = excl;
        if (2 * t + 1 < kHubBatch) first_chunk[2 * t + 1] = excl + cnt[0];
        if (t == 1023) first_chunk[kHubBatch] = base + incl;
        __syncthreads();
        const int total = first_chunk[kHubBatch];
        for (int gc = blockIdx.x; gc < total; gc += gridDim.x) {
            // the hub this chunk belongs to: last h with first_chunk[h] <= gc
            int lo = 0, hi = nb - 1;
            while (lo < hi) {
                const int mid = (lo + hi + 1) >> 1;
                if (first_chunk[mid] <= gc) lo = mid; else hi = mid - 1;
            }
            const int64_t row = hubs[h0 + lo];
            int64_t start, end;
            row_range<KIND>(p, row, start, end);
            start += static_cast<int64_t>(gc - first_chunk[lo]) * kHubChunk;
            if (start + kHubChunk < end) end = start + kHubChunk;
            const int64_t per = (end - start + WAVES - 1) / WAVES;
            const int64_t s = start + per * wave;
            const int64_t e = s + per;
            int acc[VEC];
            wave_row_sum<VEC, KIND>(p, c, lane, s < end ? s : end, e < end ? e : end, acc);
            if (c.grp == 0) {
#pragma unroll
                for (int i = 0; i < VEC; ++i) atomicAdd(&part[i * 64 + c.sub], acc[i]);
            }
            __syncthreads();
            if (wave == 0 && c.grp == 0 && c.col_ok) {
                int* orow = reinterpret_cast<int*>(p.out) + row * p.W + c.col;
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    const int v = part[i * 64 + c.sub];
                    part[i * 64 + c.sub] = 0;
                    if (c.col + i < p.W) atomicAdd(orow + i, v);
                }
            } else if (wave == 0 && c.grp == 0) {
#pragma unroll
                for (int i = 0; i < VEC; ++i) part[i * 64 + c.sub] = 0;
            }
            __syncthreads();
        }
        __syncthreads();  // first_chunk is rebuilt by the next batch
    }
}

// One wavefront per hub row: out = epilogue(int32 sum), in place.  blockDim.x = 256.
template <int VEC, int KIND>
__global__ __launch_bounds__(256) void spmm_hub_store_kernel(const SpmmParams p) {
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 6);
    const LaneCols c = lane_cols<VEC, KIND>(p, lane);
    const int nhub = *static_cast<const int*>(p.hub_ws);
    const int64_t* hubs = hub_list(p.hub_ws);
    for (int h = blockIdx.x * 4 + wave; h < nhub; h += gridDim.x * 4) {
        const int64_t row = hubs[h];
        if (c.grp == 0) {
            const int* orow = reinterpret_cast<const int*>(p.out) + row * p.W + c.col;
            int acc[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] = (c.col_ok && c.col + i < p.W) ? orow[i] : 0;
            if (p.amax_part) store_row<VEC, true>(p, c, row, acc);  // uniform
            else store_row<VEC>(p, c, row, acc);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Sparse graphs, slot spans.  The tiers above need five launches whose tails run one after the
// other; here the work is cut by CSR slots instead of rows.  Wavefront w owns slots
// [256 w, 256 w + 256) whatever rows they belong to; lane group g (lpe lanes = one gathered row
// piece) walks the K = 256 / groups consecutive slots [g K, g K + K) four at a time and keeps the
// running int32 sums of the row it is in.  Row starts inside the span are bits of a 256-bit mask in
// LDS, built from the row pointers that follow the span's first row (a 64-ary search finds that
// row).  A row that starts and ends inside one group's slots is complete when the group reaches
// its end.  Pieces of rows cut by a group boundary meet in an LDS accumulator (integer atomics,
// exact in any order) owned by the group the row starts in; pieces of rows cut by the span boundary
// go to the caller's workspace as int32 partial rows (at most two per span) and
// spmm_span_fix_kernel adds them up, stores those rows and the rows without any slot.
constexpr int kSpanSlots = 256;
constexpr int kSpanWin = kSpanSlots + kWave;  // row pointers staged per span: 64 empty rows of slack

struct SpanRowMeta {
    int64_t tail_row;   // the row that starts in this span and runs on into the next, or -1
    int64_t head_open;  // the span lies inside one row that began before it and runs on after it
};
__host__ __device__ inline size_t span_parts_offset(int64_t nspans) {
    return (static_cast<size_t>(nspans) * sizeof(SpanRowMeta) + 255) & ~static_cast<size_t>(255);
}
// partial row `piece` (0 = head: began before the span, 1 = tail) of span w
__device__ __forceinline__ int* span_part(const SpmmParams& p, int64_t nspans, int64_t w, int piece) {
    return reinterpret_cast<int*>(static_cast<char*>(p.span_ws) + span_parts_offset(nspans)) +
           (w * 2 + piece) * p.span_wp;
}

// blockDim.x = 256: four spans per workgroup, grid (ceil(spans / 4), column tiles);
// dynamic LDS: span_lds_bytes().
__host__ __device__ inline size_t span_wave_ints(int lpe_log2, int vec) {
    // groups + 1 accumulator rows of one column tile; while the row structure is built the staged
    // row pointers (kSpanWin int64) use the same space
    const size_t acc = ((64 >> lpe_log2) + 1) * (static_cast<size_t>(vec) << lpe_log2);
    const size_t win = static_cast<size_t>(kSpanWin) * 2;
    return ((acc > win ? acc : win) + 1) & ~static_cast<size_t>(1);
}
static size_t span_lds_bytes(int lpe_log2, int vec) { return sizeof(int) * 4 * span_wave_ints(lpe_log2, vec); }

template <int VEC, int KIND>
__global__ __launch_bounds__(256) void spmm_span_kernel(const SpmmParams p) {
    constexpr int U = 4;
    extern __shared__ __align__(16) int dyn_lds[];
    __shared__ int sidx_all[4][kSpanSlots];
    __shared__ int seid_all[weighted(KIND) ? 4 : 1][weighted(KIND) ? kSpanSlots : 1];
    __shared__ int rowof_all[4][kSpanSlots];
    __shared__ unsigned maskw_all[4][12];
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 6);
    const int64_t nspans = (p.nnz + kSpanSlots - 1) / kSpanSlots;
    const int64_t w = static_cast<int64_t>(blockIdx.x) * 4 + wave;
    if (w >= nspans) return;  // the whole wavefront leaves; no workgroup barrier below
    const LaneCols c = lane_cols<VEC, KIND>(p, lane);
    const int tile_ints = c.lpe * VEC;
    int* accbuf = dyn_lds + wave * span_wave_ints(p.lpe_log2, VEC);
    int64_t* win = reinterpret_cast<int64_t*>(accbuf);  // only while the row structure is built
    int* sidx = sidx_all[wave];
    int* seid = seid_all[weighted(KIND) ? wave : 0];
    int* rowof = rowof_all[wave];
    unsigned* maskw = maskw_all[wave];
    const bool permuted = weighted(KIND) && p.edge_ids;
    const int64_t base = w * kSpanSlots;
    const int endl = static_cast<int>(p.nnz - base < kSpanSlots ? p.nnz - base : kSpanSlots);
    const int64_t end = base + endl;

    // the span's column indices (and edge ids), one coalesced pass; issued first so that they are in
    // flight while the row structure is worked out
    int my_idx[kSpanSlots / kWave], my_eid[kSpanSlots / kWave];
#pragma unroll
    for (int u = 0; u < kSpanSlots / kWave; ++u) {
        const int sl = kWave * u + lane;
        my_idx[u] = my_eid[u] = 0;
        if (sl < endl) {
            my_idx[u] = load_index<true>(p, p.indices, base + sl);
            if (permuted) my_eid[u] = load_index<true>(p, p.edge_ids, base + sl);
        }
    }

    // ---- row structure of the span
    const int64_t r0 = row_of_slot_wave(p.indptr, p.rows, base, lane);
    if (lane < 12) maskw[lane] = 0u;
#pragma unroll
    for (int u = 0; u < kSpanSlots / kWave; ++u) rowof[kWave * u + lane] = 0;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int k = 0; k < kSpanWin / kWave; ++k) {
        const int i = lane + kWave * k;
        const int64_t r = r0 + i;
        const int64_t pv = r <= p.rows ? p.indptr[r] : INT64_MAX;
        win[i] = pv;
        if (pv >= base && pv < end) {  // row r0 + i starts at slot pv; of several (empty rows), the last one owns the slot
            const int sl = static_cast<int>(pv - base);
            atomicOr(&maskw[sl >> 5], 1u << (sl & 31));
            atomicMax(&rowof[sl], i);
        }
        if (pv == end) atomicOr(&maskw[8], 1u);  // a row ends exactly at the span's end
    }
#pragma unroll
    for (int u = 0; u < kSpanSlots / kWave; ++u) {
        sidx[kWave * u + lane] = my_idx[u];
        if (permuted) seid[kWave * u + lane] = my_eid[u];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (win[kSpanWin - 1] < end) {  // more than 64 empty rows inside the span: search the array per slot
#pragma unroll
        for (int u = 0; u < kSpanSlots / kWave; ++u) {
            const int sl = kWave * u + lane;
            if (sl < endl) {
                const int64_t s = base + sl;
                int64_t lo = r0, hi = p.rows;
                while (hi - lo > 1) {
                    const int64_t mid = lo + ((hi - lo) >> 1);
                    if (p.indptr[mid] <= s) lo = mid; else hi = mid;
                }
                if (p.indptr[lo] == s) {
                    atomicOr(&maskw[sl >> 5], 1u << (sl & 31));
                    atomicMax(&rowof[sl], static_cast<int>(lo - r0));
                }
                if (sl == endl - 1 && p.indptr[lo + 1] == end) atomicOr(&maskw[8], 1u);
            }
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    for (int i = lane; i < (c.epi + 1) * tile_ints; i += kWave) accbuf[i] = 0;  // the row pointers are done with
    const bool last_open = (maskw[8] & 1u) == 0u;  // the row of the last slot runs on into the next span
    // largest flagged slot < pos, or -1; smallest flagged slot >= pos, or kSpanSlots
    auto prev_flag = [&](int pos) {
        for (int wd = (pos - 1) >> 5; wd >= 0 && pos > 0; --wd) {
            unsigned m = maskw[wd];
            if (wd == ((pos - 1) >> 5)) m &= (2u << ((pos - 1) & 31)) - 1u;  // 2u << 31 wraps to 0: all bits kept
            if (m) return wd * 32 + 31 - __builtin_clz(m);
        }
        return -1;
    };
    auto next_flag = [&](int pos) {
        for (int wd = pos >> 5; wd < kSpanSlots / 32; ++wd) {
            unsigned m = maskw[wd];
            if (wd == (pos >> 5)) m &= ~((1u << (pos & 31)) - 1u);
            if (m) return wd * 32 + __builtin_ctz(m);
        }
        return kSpanSlots;
    };

    // ---- the walk
    const int K = kSpanSlots >> c.sh;  // slots per group: 4 * lpe
    const int gbase = c.grp * K;
    int acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0;
    bool have = false, started = false, tail_partial = false;
    int cur_start = 0, my_last_flag = -1, first_target = -2;
    // Rows end at different slots in different groups, so the end-of-row code runs under divergence
    // many times per wavefront: the scale and the lane's bias values are fetched once, here.
    const float dq = p.scale2 ? p.scale[0] * p.scale2[0] : p.scale[0];
    float breg[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) breg[i] = (p.bias && c.col + i < p.W) ? p.bias[c.col + i] : 0.0f;
    // same sequence of roundings as store_row
    auto finish_row = [&](int64_t row, const int* sum) {
        if (!c.col_ok) return;
        const float rs = p.row_scale ? p.row_scale[row] : 1.0f;
        float* o = p.out + row * p.W + c.col;
        float y[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            y[i] = dq * static_cast<float>(sum[i]);
            if (p.row_scale) y[i] = y[i] * rs;
            if (p.bias) y[i] = y[i] + breg[i];
        }
        if (p.relu) {  // uniform: rows without an activation skip its instructions altogether
#pragma unroll
            for (int i = 0; i < VEC; ++i) y[i] = activate(y[i], p.relu);
        }
        if (VEC == 16 && p.out_vec && c.col + 16 <= p.W) {
            f32x4* o4 = reinterpret_cast<f32x4*>(o);
#pragma unroll
            for (int i = 0; i < 4; ++i) o4[i] = f32x4{y[4 * i], y[4 * i + 1], y[4 * i + 2], y[4 * i + 3]};
        } else {
#pragma unroll
            for (int i = 0; i < VEC; ++i)
                if (c.col + i < p.W) o[i] = y[i];
        }
        if (KIND == KIND_COPY && VEC == 16 && p.sign_bits) store_sign_bits<VEC>(p, row, c.col, y);
    };
    // ends the piece the group is in
    auto flush = [&](bool closed) {
        if (started && closed) {
            finish_row(r0 + rowof[cur_start], acc);
        } else {
            int target = c.grp;
            if (!started) {
                if (first_target == -2) {
                    const int pf = prev_flag(gbase);
                    first_target = pf < 0 ? c.epi : pf / K;
                }
                target = first_target;
            } else {
                tail_partial = true;
            }
            int* ab = accbuf + target * tile_ints + c.sub * VEC;
#pragma unroll
            for (int i = 0; i < VEC; ++i) atomicAdd(&ab[i], acc[i]);
        }
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = 0;
        have = false;
    };
    auto issue = [&](typename Gather<VEC>::T* d, uint32_t& m, int q) {
        m = 0u;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int slot = gbase + q + u;
            const bool ok = slot < endl;
            const int sl = ok ? slot : 0;  // slot 0 exists; its multiplier is 0 here
            d[u] = Gather<VEC>::load(c.fcol + row_offset(sidx[sl], p));
            uint32_t wv = 1u;
            if (weighted(KIND)) {
                const int64_t pos = permuted ? static_cast<int64_t>(seid[sl]) : base + sl;
                wv = edge_value<KIND>(p, c, pos);
            }
            m |= (ok ? wv : 0u) << (8 * u);
        }
    };
    auto consume = [&](const typename Gather<VEC>::T* d, uint32_t m, int q) {
        const int slot0 = gbase + q;
        if (slot0 >= endl) return;
        const unsigned bits = (maskw[slot0 >> 5] >> (slot0 & 31)) & 0xFu;
        int pos = 0;
        while (pos < 4) {  // one pass per row that has slots in this batch
            if ((bits >> pos) & 1u) {
                if (have) flush(true);
                started = true;
                cur_start = slot0 + pos;
                my_last_flag = cur_start;
            }
            const unsigned rest = bits >> (pos + 1);
            const int nxt = rest ? pos + 1 + __builtin_ctz(rest) : 4;
            const uint32_t upto = nxt == 4 ? 0xFFFFFFFFu : ((1u << (8 * nxt)) - 1u);
            accumulate4<VEC>(acc, d, m & upto & ~((1u << (8 * pos)) - 1u));
            if (slot0 + pos < endl) have = true;
            pos = nxt;
        }
    };
    {
        typename Gather<VEC>::T da[U], db[U];
        uint32_t ma = 0u, mb = 0u;
        issue(da, ma, 0);
        for (int q = 0; q < K; q += 2 * U) {  // two batches in flight
            const bool has_b = q + U < K;
            if (has_b) issue(db, mb, q + U);
            consume(da, ma, q);
            if (q + 2 * U < K) issue(da, ma, q + 2 * U);
            if (has_b) consume(db, mb, q + U);
        }
    }
    if (have) {
        const int e = gbase + K;
        flush(e >= endl ? !last_open : ((maskw[e >> 5] >> (e & 31)) & 1u) != 0u);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // ---- rows cut by a group boundary: the group a row starts in finishes it
    if (tail_partial) {
        const int e = gbase + K;
        const bool closed = e >= endl ? !last_open : (next_flag(e) < endl || !last_open);
        const int* ab = accbuf + c.grp * tile_ints + c.sub * VEC;
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = ab[i];
        if (closed) {
            finish_row(r0 + rowof[my_last_flag], acc);
        } else {
            int* part = span_part(p, nspans, w, 1) + c.col;
#pragma unroll
            for (int i = 0; i < VEC; ++i) part[i] = acc[i];
        }
    }
    const bool head = (maskw[0] & 1u) == 0u;  // the first slot's row began before the span
    if (c.grp == 0 && head) {
        const int* ab = accbuf + c.epi * tile_ints + c.sub * VEC;
        int* part = span_part(p, nspans, w, 0) + c.col;
#pragma unroll
        for (int i = 0; i < VEC; ++i) part[i] = ab[i];
    }
    if (lane == 0 && blockIdx.y == 0) {
        const int lf = prev_flag(kSpanSlots);
        SpanRowMeta* meta = static_cast<SpanRowMeta*>(p.span_ws) + w;
        meta->tail_row = (last_open && lf >= 0) ? r0 + rowof[lf] : -1;
        meta->head_open = (last_open && lf < 0) ? 1 : 0;
    }
}

// Adds up the pieces of every row cut by a span boundary (the tail piece of the span it starts in,
// then the head pieces of the following spans) and stores the row; also stores the rows that have
// no slot at all.  Launched like spmm_span_kernel, without dynamic LDS.
template <int VEC>
__global__ __launch_bounds__(256) void spmm_span_fix_kernel(const SpmmParams p) {
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 6);
    const int64_t nspans = (p.nnz + kSpanSlots - 1) / kSpanSlots;
    const int64_t w = static_cast<int64_t>(blockIdx.x) * 4 + wave;
    const LaneCols c = lane_cols<VEC, KIND_COPY>(p, lane);
    const SpanRowMeta* meta = static_cast<const SpanRowMeta*>(p.span_ws);
    if (w < nspans && meta[w].tail_row >= 0) {
        int64_t last = w + 1;  // the first following span whose head piece ends its row
        for (;; last += kWave) {
            const int64_t j = last + lane;
            const uint64_t m = __ballot(j >= nspans || meta[j].head_open == 0);
            if (m) {
                last += __builtin_ctzll(m);
                break;
            }
        }
        if (last >= nspans) last = nspans - 1;
        int acc[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = 0;
        if (c.grp == 0) {
            const int* part = span_part(p, nspans, w, 1) + c.col;
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] = part[i];
        }
        for (int64_t j = w + 1 + c.grp; j <= last; j += c.epi) {
            const int* part = span_part(p, nspans, j, 0) + c.col;
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] += part[i];
        }
        for (int off = c.lpe; off < kWave; off <<= 1) {
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] += __shfl_xor(acc[i], off, kWave);
        }
        if (c.grp == 0) store_row<VEC>(p, c, meta[w].tail_row, acc);
    }
    // rows without slots: out = epilogue(0)
    const int64_t nwaves = static_cast<int64_t>(gridDim.x) * 4;
    for (int64_t rb = (static_cast<int64_t>(blockIdx.x) * 4 + wave) * kWave; rb < p.rows; rb += nwaves * kWave) {
        const int64_t r = rb + lane;
        uint64_t m = __ballot(r < p.rows && p.indptr[r] == p.indptr[r + 1]);
        int zero[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) zero[i] = 0;
        while (m) {
            const int b = __builtin_ctzll(m);
            m &= m - 1;
            if (c.grp == 0) store_row<VEC>(p, c, rb + b, zero);
        }
    }
}

// graphs whose rows average fewer than 64 slots take the slot-span path (given a workspace)
static bool span_graph(int64_t rows, int64_t nnz) { return nnz < 64 * rows; }

static int ilog2_ceil(int64_t v) {
    int l = 0;
    while ((1LL << l) < v) ++l;
    return l;
}

template <int KIND>
static int launch_spmm(SpmmParams p, int vec, hipStream_t s) {
    if (p.rows == 0 || p.W == 0) return TANGO_OK;
    const int64_t lanes = ceil_div(p.W, vec);
    p.lpe_log2 = lanes >= 64 ? 6 : ilog2_ceil(lanes);
    // A gathered matrix far beyond the L2 (4 MB per XCD) is walked one 128-byte column tile at a
    // time: gridDim.y orders the launch tile by tile, so at any moment the resident waves gather
    // the same 128 columns and an L2 holds twice as many distinct rows' pieces as with 256-byte
    // rows.  The index array is streamed once per tile, which the better hit rate outweighs.
    if (vec == 16 && p.W >= 256 && p.num_src * p.ldf >= (16LL << 20) && (KIND == KIND_COO || p.nnz >= 64 * p.rows))
        p.lpe_log2 = 3;  // (sparse graphs are bound by per-row latencies, not by the L2: one pass there)
    p.tile = static_cast<int64_t>(vec) << p.lpe_log2;
    p.out_vec = (reinterpret_cast<uintptr_t>(p.out) & 15) == 0 && (p.W & 3) == 0;
    p.ldf_shift = -1;
    if (p.ldf > 0 && (p.ldf & (p.ldf - 1)) == 0 && p.num_src * p.ldf < (1LL << 31)) {
        p.ldf_shift = 0;
        while ((1LL << p.ldf_shift) < p.ldf) ++p.ldf_shift;
    }
    const int64_t ychunks = ceil_div(p.W, p.tile);
    p.amax_tiles = static_cast<int>(ychunks);
    if (ychunks > 65535) return TANGO_ERR_UNSUPPORTED;
    // four waves split each row when rows are long AND wide (few neighbours per load instruction);
    // otherwise one wave per row, which amortises the per-row latencies over more edges
    const bool wide = p.nnz >= 128 * p.rows && p.lpe_log2 >= 4;
    const int64_t gx = wide ? p.rows : ceil_div(p.rows, 4);
    if (gx > INT32_MAX) return TANGO_ERR_UNSUPPORTED;
    const dim3 grid(static_cast<unsigned>(gx), static_cast<unsigned>(ychunks));
    // A row much longer than one wavefront's share of the whole job would finish long after
    // everything else (hub rows of a small power-law graph): such rows get sixteen waves each.
    // The share is nnz / 8192 (8192 resident waves).  A single wave walks a row 4 * 64 / lpe slots
    // at a time, and below ~16 such batches the sixteen-wave path is not worth its barriers.  On
    // very large jobs the main launch runs for milliseconds and hides rows of a few shares (they
    // sit at the front of the grid), while a separate launch for them would only add its own
    // tail: there the threshold is four shares (measured on the 114.8 M-edge benchmark graph).
    const int64_t by_batches = 16LL * 4 * (64 >> p.lpe_log2);
    const int64_t share = p.nnz >= (64LL << 20) ? (p.nnz >> 11) : (p.nnz >> 13);
    p.long_row = share > by_batches ? share : by_batches;
    const int64_t longest = p.max_row > 0 ? p.max_row : p.nnz;  // no row has more slots than this
    p.hub_row = 4 * p.long_row > kHubRowMin ? 4 * p.long_row : kHubRowMin;
    const bool hubs = p.hub_ws && longest > p.hub_row;
    if (!hubs) p.hub_row = INT64_MAX;
    const dim3 lgrid(static_cast<unsigned>(p.rows < kLongGrid ? p.rows : kLongGrid), static_cast<unsigned>(ychunks));
    const dim3 hgrid(kHubSumGrid, lgrid.y), sgrid(64, lgrid.y);
#define TANGO_SPMM_LONG(V)                                                                          \
    do {                                                                                            \
        if (hubs) fill_u32(p.hub_ws, 0u, 1, s);                                                     \
        hipLaunchKernelGGL((spmm_long_kernel<V, KIND>), lgrid, dim3(1024), 0, s, p);                \
        if (hubs) {                                                                                 \
            hipLaunchKernelGGL((spmm_hub_sum_kernel<V, KIND>), hgrid, dim3(1024), 0, s, p);         \
            hipLaunchKernelGGL((spmm_hub_store_kernel<V, KIND>), sgrid, dim3(256), 0, s, p);        \
        }                                                                                           \
    } while (0)
    const int64_t nspans_all = ceil_div(p.nnz, kSpanSlots);
    const bool span_fits = span_parts_offset(nspans_all) + sizeof(int) * 2 * static_cast<size_t>(nspans_all) *
                               static_cast<size_t>(ychunks * p.tile) <= p.span_ws_bytes;
    if (KIND != KIND_COO && p.span_ws && span_fits && span_graph(p.rows, p.nnz) && !p.part && !p.amax_part) {  // sparse graph: slot spans, two launches
        const int64_t nspans = nspans_all;
        p.span_wp = ychunks * p.tile;
        const dim3 spgrid(static_cast<unsigned>(ceil_div(nspans > 0 ? nspans : 1, 4)), static_cast<unsigned>(ychunks));
        const size_t lds = span_lds_bytes(p.lpe_log2, vec);
#define TANGO_SPMM_SPANS(V)                                                                      \
    do {                                                                                         \
        if (nspans > 0) hipLaunchKernelGGL((spmm_span_kernel<V, KIND>), spgrid, dim3(256), lds, s, p); \
        hipLaunchKernelGGL(spmm_span_fix_kernel<V>, spgrid, dim3(256), 0, s, p);                 \
    } while (0)
        if (vec == 16) TANGO_SPMM_SPANS(16);
        else if (vec == 4) TANGO_SPMM_SPANS(4);
        else TANGO_SPMM_SPANS(1);
#undef TANGO_SPMM_SPANS
        return launch_status();
    }
    if (longest > p.long_row) {
        if (vec == 16) TANGO_SPMM_LONG(16);
        else if (vec == 4) TANGO_SPMM_LONG(4);
        else TANGO_SPMM_LONG(1);
    }
#undef TANGO_SPMM_LONG
    // Sparse graph: lane groups own the short rows, single waves the rest up to long_row.
    if (KIND != KIND_COO && p.nnz < 64 * p.rows && p.lpe_log2 < 6 && !p.part && !p.amax_part) {
        p.group_row = kGroupRow;
        const int64_t rows_per_block = 4LL << (6 - p.lpe_log2);
        const dim3 ggrid(static_cast<unsigned>(ceil_div(p.rows, rows_per_block)), static_cast<unsigned>(ychunks));
        const dim3 mgrid(static_cast<unsigned>(ceil_div(p.rows, 4 * kRowsPerWave)), static_cast<unsigned>(ychunks));
#define TANGO_SPMM_TIERS(V)                                                                     \
    do {                                                                                        \
        hipLaunchKernelGGL((spmm_group_kernel<V, KIND>), ggrid, dim3(256), 0, s, p);            \
        hipLaunchKernelGGL((spmm_medium_kernel<V, KIND>), mgrid, dim3(256), 0, s, p);           \
    } while (0)
        if (vec == 16) TANGO_SPMM_TIERS(16);
        else if (vec == 4) TANGO_SPMM_TIERS(4);
        else TANGO_SPMM_TIERS(1);
#undef TANGO_SPMM_TIERS
        return launch_status();
    }
#define TANGO_SPMM_LAUNCH(V, WPR) \
    hipLaunchKernelGGL((spmm_kernel<V, WPR, KIND>), grid, dim3(256), 0, s, p)
    if (KIND == KIND_COPY && vec == 16 && p.lpe_log2 <= 3 && p.row_order && !p.amax_part && p.nnz > 0) {
        // tiles of at most 128 bytes, rows ordered by length: four rows to a wavefront
        const dim3 qgrid(static_cast<unsigned>(ceil_div(p.rows, 16)), static_cast<unsigned>(ychunks));
#define TANGO_SPMM_QUAD(LPL)                                                                              \
    do {                                                                                                 \
        if (p.ldf_shift >= 0) hipLaunchKernelGGL((spmm_quad_kernel<4, LPL, true>), qgrid, dim3(256), 0, s, p);  \
        else hipLaunchKernelGGL((spmm_quad_kernel<4, LPL, false>), qgrid, dim3(256), 0, s, p);                \
    } while (0)
        if (p.lpe_log2 == 3) hipLaunchKernelGGL((spmm_quad_kernel<4, -1, false>), qgrid, dim3(256), 0, s, p);
        else if (p.lpe_log2 == 2) TANGO_SPMM_QUAD(2);
        else if (p.lpe_log2 == 1) TANGO_SPMM_QUAD(1);
        else TANGO_SPMM_QUAD(0);
#undef TANGO_SPMM_QUAD
        return launch_status();
    }
    if (p.amax_part) {  // copy_u only (the entry points see to that)
        if (vec != 16 || KIND != KIND_COPY) return TANGO_ERR_UNSUPPORTED;
        if (wide) hipLaunchKernelGGL((spmm_kernel<16, 4, KIND_COPY, true>), grid, dim3(256), 0, s, p);
        else hipLaunchKernelGGL((spmm_kernel<16, 1, KIND_COPY, true>), grid, dim3(256), 0, s, p);
    } else if (vec == 16) {
        if (wide) TANGO_SPMM_LAUNCH(16, 4); else TANGO_SPMM_LAUNCH(16, 1);
    } else if (vec == 4) {
        if (wide) TANGO_SPMM_LAUNCH(4, 4); else TANGO_SPMM_LAUNCH(4, 1);
    } else {
        if (wide) TANGO_SPMM_LAUNCH(1, 4); else TANGO_SPMM_LAUNCH(1, 1);
    }
#undef TANGO_SPMM_LAUNCH
    if (p.amax_part) {
        const int64_t n = p.rows * ychunks;
        hipLaunchKernelGGL(amax_reduce_kernel, dim3(static_cast<unsigned>(n < 65536 ? ceil_div(n, 256) : 256)), dim3(256),
                           0, s, p.amax_part, n, p.amax_scale);
    }
    return launch_status();
}

// Widest per-lane load such that every load of a gathered row is aligned and
// stays inside the row's ldf bytes.
static int pick_vec(const int8_t* feat, int64_t ldf, int64_t W) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(feat);
    if ((a & 15) == 0 && (ldf & 15) == 0 && ((W + 15) & ~15LL) <= ldf) return 16;
    if ((a & 3) == 0 && (ldf & 3) == 0 && ((W + 3) & ~3LL) <= ldf) return 4;
    return 1;
}

}  // namespace tango

using namespace tango;

extern "C" {

// floats of per-row-piece maxima an aggregation with a scale output writes: a row has at most W / 64 + 1 pieces
static size_t amax_floats(int64_t rows, int64_t W) { return static_cast<size_t>(rows) * static_cast<size_t>(W / 64 + 2); }

static size_t spmm_base_workspace(int64_t rows, int64_t nnz, int64_t W) {
    if (span_graph(rows, nnz)) {
        // two int32 partial rows per span.  Their padded width is column tiles x tile: below 2 W + 16 while the
        // lanes of a row piece fit a wavefront (tile = vec x the lane count rounded up to a power of two), and
        // below W + 64 vec < 2 W once they do not
        const int64_t nspans = ceil_div(nnz, kSpanSlots);
        return span_parts_offset(nspans) + sizeof(int) * 2 * static_cast<size_t>(nspans) * static_cast<size_t>(2 * W + 16);
    }
    return 64 + sizeof(int64_t) * static_cast<size_t>(nnz / kHubRowMin + 2);
}

size_t tango_spmm_workspace(int64_t rows, int64_t nnz, int64_t W) {
    if (rows < 0 || nnz < 0 || W < 0) return 0;
    return ((spmm_base_workspace(rows, nnz, W) + 255) & ~static_cast<size_t>(255)) + sizeof(float) * amax_floats(rows, W);
}

int tango_spmm_csr_copy_u(float* out, const int64_t* indptr, const int64_t* indices,
                          const int8_t* feat, int64_t ldf, const float* scale, int64_t rows,
                          int64_t num_src, int64_t nnz, int64_t F, tango_stream_t stream) {
    if (rows < 0 || F < 0 || nnz < 0 || num_src < 0 || ldf < F || !scale || !indptr ||
        (rows * F > 0 && !out) || (nnz > 0 && (!indices || !feat)))
        return TANGO_ERR_INVALID_ARG;
    if (num_src >= (1LL << 31) || nnz >= (1LL << 31)) return TANGO_ERR_UNSUPPORTED;
    SpmmParams p{};
    p.out = out; p.indptr = indptr; p.indices = indices; p.feat = feat; p.scale = scale;
    p.rows = rows; p.num_src = num_src; p.ldf = ldf; p.W = F; p.F = F; p.D = 1; p.nnz = nnz;
    return launch_spmm<KIND_COPY>(p, pick_vec(feat, ldf, F), as_stream(stream));
}

int tango_spmm_csr_copy_u_ex(float* out, const int64_t* indptr, const void* indices, int idx_bits,
                             const int8_t* feat, int64_t ldf, const float* scale,
                             const float* row_scale, const float* bias, int relu, uint16_t* sign_bits,
                             int64_t rows, int64_t num_src, int64_t nnz, int64_t F, int64_t max_row_nnz,
                             const float* absmax_row_mul, float* scale_out,
                             void* workspace, size_t workspace_bytes, tango_stream_t stream) {
    if (rows < 0 || F < 0 || nnz < 0 || num_src < 0 || ldf < F || !scale || !indptr || max_row_nnz < 0 ||
        (rows * F > 0 && !out) || (nnz > 0 && (!indices || !feat)) || (idx_bits != 32 && idx_bits != 64) ||
        (scale_out && !workspace))
        return TANGO_ERR_INVALID_ARG;
    if (workspace && (workspace_bytes < tango_spmm_workspace(rows, nnz, F) || (reinterpret_cast<uintptr_t>(workspace) & 15)))
        return TANGO_ERR_WORKSPACE;
    if (num_src >= (1LL << 31) || nnz >= (1LL << 31) || relu < 0 || relu > 2) return TANGO_ERR_UNSUPPORTED;
    SpmmParams p{};
    p.out = out; p.indptr = indptr; p.indices = static_cast<const int64_t*>(indices); p.idx32 = idx_bits == 32;
    p.feat = feat; p.scale = scale;
    const int vec = pick_vec(feat, ldf, F);
    if (sign_bits && (vec != 16 || (F & 15) != 0)) return TANGO_ERR_UNSUPPORTED;
    p.row_scale = row_scale; p.bias = bias; p.relu = relu; p.sign_bits = sign_bits; p.max_row = max_row_nnz; p.hub_ws = workspace;
    p.span_ws = workspace; p.span_ws_bytes = workspace ? (spmm_base_workspace(rows, nnz, F) + 255) & ~static_cast<size_t>(255) : 0;
    if (scale_out && rows * F > 0) {
        p.amax_part = reinterpret_cast<float*>(static_cast<char*>(workspace) + p.span_ws_bytes);
        p.amax_mul = absmax_row_mul; p.amax_scale = scale_out;
    }
    p.rows = rows; p.num_src = num_src; p.ldf = ldf; p.W = F; p.F = F; p.D = 1; p.nnz = nnz;
    return launch_spmm<KIND_COPY>(p, pick_vec(feat, ldf, F), as_stream(stream));
}

static int spmm_u_mul_e_common(float* out, const int64_t* indptr, const void* indices,
                              const void* edge_ids, int idx_bits, const int8_t* feat, const int8_t* evals,
                              const float* evals_f32,
                              int edge_major, const float* scale, const float* scale2, const float* bias,
                              int act, int64_t rows,
                              int64_t num_src, int64_t H, int64_t F, int64_t D, int64_t nnz,
                              int64_t max_row_nnz, void* workspace, size_t workspace_bytes,
                              tango_stream_t stream) {
    if (rows < 0 || H < 0 || F < 0 || nnz < 0 || num_src < 0 || !scale || !indptr || max_row_nnz < 0 ||
        (rows * H * F > 0 && !out) || (nnz > 0 && (!indices || !feat || (!evals && !evals_f32))) ||
        (idx_bits != 32 && idx_bits != 64) || (evals_f32 && !scale2))
        return TANGO_ERR_INVALID_ARG;
    if (workspace && (workspace_bytes < tango_spmm_workspace(rows, nnz, H * F) || (reinterpret_cast<uintptr_t>(workspace) & 15)))
        return TANGO_ERR_WORKSPACE;
    if (D != 1 && D != F) return TANGO_ERR_UNSUPPORTED;
    if (num_src >= (1LL << 31) || nnz >= (1LL << 31) || act < 0 || act > 2) return TANGO_ERR_UNSUPPORTED;
    SpmmParams p{};
    p.out = out; p.indptr = indptr; p.indices = static_cast<const int64_t*>(indices);
    p.edge_ids = static_cast<const int64_t*>(edge_ids); p.idx32 = idx_bits == 32; p.feat = feat;
    p.relu = act; p.max_row = max_row_nnz; p.hub_ws = workspace; p.span_ws = workspace; p.span_ws_bytes = workspace_bytes;
    p.evals = evals; p.evals_f32 = evals_f32; p.scale = scale; p.scale2 = scale2; p.bias = bias; p.rows = rows; p.num_src = num_src; p.ldf = H * F; p.W = H * F; p.F = F; p.D = D;
    p.nnz = nnz;
    if (edge_major) {  // evals[nnz, H, D]: the H * D bytes of one edge share a cache sector
        p.ev_se = H * D; p.ev_sh = D; p.ev_sd = 1;
    } else {           // evals[H, D, nnz], the reference's transposed layout
        p.ev_se = 1; p.ev_sh = D * nnz; p.ev_sd = nnz;
    }
    // a lane's bytes must share one edge value: vector loads only when they stay inside a head
    int vec = 1;
    if (D == 1 && F > 0) {
        const uintptr_t a = reinterpret_cast<uintptr_t>(feat);
        if ((F & 15) == 0 && (a & 15) == 0) vec = 16;
        else if ((F & 3) == 0 && (a & 3) == 0) vec = 4;
    }
    if (evals_f32) return launch_spmm<KIND_WEIGHTED_F32>(p, vec, as_stream(stream));
    return launch_spmm<KIND_WEIGHTED>(p, vec, as_stream(stream));
}

int tango_spmm_csr_u_mul_e_ex(float* out, const int64_t* indptr, const void* indices,
                              const void* edge_ids, int idx_bits, const int8_t* feat, const int8_t* evals,
                              int edge_major, const float* scale, const float* scale2, const float* bias,
                              int act, int64_t rows, int64_t num_src, int64_t H, int64_t F, int64_t D, int64_t nnz,
                              int64_t max_row_nnz, void* workspace, size_t workspace_bytes,
                              tango_stream_t stream) {
    return spmm_u_mul_e_common(out, indptr, indices, edge_ids, idx_bits, feat, evals, nullptr, edge_major, scale, scale2,
                               bias, act, rows, num_src, H, F, D, nnz, max_row_nnz, workspace, workspace_bytes, stream);
}

int tango_spmm_csr_u_mul_e_f32e(float* out, const int64_t* indptr, const void* indices,
                                const void* edge_ids, int idx_bits, const int8_t* feat, const float* evals_f32,
                                int edge_major, const float* scale, const float* scale_e, const float* bias,
                                int act, int64_t rows, int64_t num_src, int64_t H, int64_t F, int64_t D, int64_t nnz,
                                int64_t max_row_nnz, void* workspace, size_t workspace_bytes,
                                tango_stream_t stream) {
    if (nnz > 0 && !evals_f32) return TANGO_ERR_INVALID_ARG;
    if ((reinterpret_cast<uintptr_t>(evals_f32) & 3) != 0) return TANGO_ERR_INVALID_ARG;
    return spmm_u_mul_e_common(out, indptr, indices, edge_ids, idx_bits, feat, nullptr, evals_f32, edge_major, scale,
                               scale_e, bias, act, rows, num_src, H, F, D, nnz, max_row_nnz, workspace, workspace_bytes,
                               stream);
}

int tango_spmm_csr_u_mul_e(float* out, const int64_t* indptr, const int64_t* indices,
                           const int64_t* edge_ids, const int8_t* feat, const int8_t* evals,
                           const float* scale, int64_t rows, int64_t num_src, int64_t H,
                           int64_t F, int64_t D, int64_t nnz, tango_stream_t stream) {
    return tango_spmm_csr_u_mul_e_ex(out, indptr, indices, edge_ids, 64, feat, evals, 0, scale, nullptr, nullptr, 0, rows, num_src,
                                     H, F, D, nnz, 0, nullptr, 0, stream);
}

size_t tango_spmm_dense_workspace(const tango_spmm_dense_plan* plan, int64_t F) {
    if (!plan || F < 0) return 0;
    const size_t dense = dense_workspace_bytes(*plan, F);
    if (!dense) return 0;
    // the gather kernels' own workspace for hub rows of the rest follows the dense part
    return dense + ((64 + sizeof(int64_t) * static_cast<size_t>(plan->res_nnz / kHubRowMin + 2) + 255) & ~static_cast<size_t>(255)) +
           sizeof(float) * amax_floats(plan->rows, F);
}

int tango_spmm_dense_partial(const tango_spmm_dense_plan* plan, const int8_t* feat, int64_t ldf, int64_t F,
                             void* workspace, size_t workspace_bytes, tango_stream_t stream) {
    if (!plan || F <= 0 || ldf < F || !feat) return TANGO_ERR_INVALID_ARG;
    if (plan->row_blocks <= 0) return TANGO_OK;
    const size_t need = tango_spmm_dense_workspace(plan, F);
    if (!need) return TANGO_ERR_UNSUPPORTED;
    if (!workspace || workspace_bytes < need) return TANGO_ERR_WORKSPACE;
    const int* part;
    int ld;
    return launch_dense_block(*plan, feat, ldf, F, workspace, workspace_bytes, &part, &ld, as_stream(stream));
}

// ``run_dense``: stage and multiply the bit blocks first; without it the gather kernel adds whatever partial sums a
// preceding tango_spmm_dense_partial call (same plan, F and workspace) left in the workspace.
static int copy_u_dense_impl(float* out, const tango_spmm_dense_plan* plan, const int8_t* feat, int64_t ldf,
                             const float* scale, const float* row_scale, const float* bias, int relu,
                             uint16_t* sign_bits, int64_t F, const float* absmax_row_mul, float* scale_out,
                             void* workspace, size_t workspace_bytes, tango_stream_t stream, bool run_dense) {
    if (!plan || F < 0 || !scale || ldf < F || !feat || plan->rows < 0 || plan->res_nnz < 0 || !plan->res_indptr ||
        !plan->row_slot || (plan->rows * F > 0 && !out) || (plan->res_nnz > 0 && !plan->res_indices))
        return TANGO_ERR_INVALID_ARG;
    if (plan->num_src >= (1LL << 31) || plan->res_nnz >= (1LL << 31) || relu < 0 || relu > 2) return TANGO_ERR_UNSUPPORTED;
    if (sign_bits && (F & 15) != 0) return TANGO_ERR_UNSUPPORTED;
    if (plan->rows == 0 || F == 0) return TANGO_OK;
    const size_t need = tango_spmm_dense_workspace(plan, F);
    if (!need) return TANGO_ERR_UNSUPPORTED;
    if (!workspace || workspace_bytes < need) return TANGO_ERR_WORKSPACE;
    SpmmParams p{};
    if (plan->row_blocks > 0) {
        if (run_dense) {
            const int st = launch_dense_block(*plan, feat, ldf, F, workspace, workspace_bytes, &p.part, &p.part_ld,
                                              as_stream(stream));
            if (st != TANGO_OK) return st;
        } else {
            const int st = dense_partial_sums(*plan, feat, ldf, F, workspace, workspace_bytes, &p.part, &p.part_ld);
            if (st != TANGO_OK) return st;
        }
        p.part_slot = plan->row_slot;
    } else if (pick_vec(feat, ldf, F) != 16) {
        return TANGO_ERR_UNSUPPORTED;
    }
    p.out = out; p.indptr = plan->res_indptr; p.indices = reinterpret_cast<const int64_t*>(plan->res_indices); p.idx32 = 1;
    p.feat = feat; p.scale = scale;
    p.row_scale = row_scale; p.bias = bias; p.relu = relu; p.sign_bits = sign_bits; p.max_row = plan->res_max_row;
    p.row_order = plan->row_order;
    p.hub_ws = static_cast<char*>(workspace) + dense_workspace_bytes(*plan, F);
    if (scale_out) {
        p.amax_part = reinterpret_cast<float*>(static_cast<char*>(p.hub_ws) +
                                               ((64 + sizeof(int64_t) * static_cast<size_t>(plan->res_nnz / kHubRowMin + 2) + 255) & ~static_cast<size_t>(255)));
        p.amax_mul = absmax_row_mul; p.amax_scale = scale_out;
    }
    p.rows = plan->rows; p.num_src = plan->num_src; p.ldf = ldf; p.W = F; p.F = F; p.D = 1; p.nnz = plan->res_nnz;
    return launch_spmm<KIND_COPY>(p, 16, as_stream(stream));
}

int tango_spmm_csr_copy_u_dense(float* out, const tango_spmm_dense_plan* plan, const int8_t* feat,
                                int64_t ldf, const float* scale, const float* row_scale,
                                const float* bias, int relu, uint16_t* sign_bits, int64_t F,
                                const float* absmax_row_mul, float* scale_out,
                                void* workspace, size_t workspace_bytes, tango_stream_t stream) {
    return copy_u_dense_impl(out, plan, feat, ldf, scale, row_scale, bias, relu, sign_bits, F, absmax_row_mul, scale_out,
                             workspace, workspace_bytes, stream, true);
}

int tango_spmm_dense_rest(float* out, const tango_spmm_dense_plan* plan, const int8_t* feat,
                          int64_t ldf, const float* scale, const float* row_scale,
                          const float* bias, int relu, uint16_t* sign_bits, int64_t F,
                          void* workspace, size_t workspace_bytes, tango_stream_t stream) {
    return copy_u_dense_impl(out, plan, feat, ldf, scale, row_scale, bias, relu, sign_bits, F, nullptr, nullptr,
                             workspace, workspace_bytes, stream, false);
}

int tango_spmm_incidence(float* out, const int64_t* node_ids, const int64_t* edge_ids,
                         const int8_t* E, const float* scale, int64_t num_nodes, int64_t nnz,
                         int64_t num_edges, int64_t F, tango_stream_t stream) {
    if (num_nodes < 0 || nnz < 0 || num_edges < 0 || F < 0 || !scale ||
        (num_nodes * F > 0 && !out) || (nnz > 0 && (!node_ids || !edge_ids || !E)))
        return TANGO_ERR_INVALID_ARG;
    if (num_edges >= (1LL << 31) || nnz >= (1LL << 31)) return TANGO_ERR_UNSUPPORTED;
    SpmmParams p{};
    p.out = out; p.node_ids = node_ids; p.indices = edge_ids; p.feat = E; p.scale = scale;
    p.rows = num_nodes; p.num_src = num_edges; p.ldf = F; p.W = F; p.F = F; p.D = 1; p.nnz = nnz;
    return launch_spmm<KIND_COO>(p, pick_vec(E, F, F), as_stream(stream));
}

}  // extern "C"
