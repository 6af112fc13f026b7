// Batch normalisation over the rows of a dense fp32 matrix [rows, C] (training mode: statistics of the batch),
// with the ReLU that follows it and the scale of the result for the next quantized layer folded in.
//
// Not part of the reference's primitive layer: its arxiv drivers use torch.nn.BatchNorm1d followed by the
// activation between the graph layers (evaluation/arxiv_gat.py:376-448, evaluation/arxiv_gcn.py:156-209).  On
// [169343, 128] torch's training-mode kernels take 0.42 ms per layer and step (statistics 0.15, transform 0.03,
// backward reduction 0.20, backward element-wise 0.04); the passes here are bound by HBM: forward = one read
// for the statistics, one read + one write for the result; backward = two reads for the column sums, three
// reads + one write for the input gradient.  Every reduction runs in a fixed order (register sums over a
// thread's rows -> LDS over the workgroup's row lanes -> one partial per workgroup -> a finishing kernel), so
// results do not depend on scheduling.
//
// Variance: every workgroup forms sums of (x - k) and (x - k)^2 over its rows with k = the median of the column's
// elements in the workgroup's first three rows (the shifted-data form; the plain sum of squares cancels when |mean| >> std), turns them
// into (mean, sum of squared deviations) of its rows, and the finishing kernel merges the workgroups' pairs with
// the pairwise update of Chan et al. (mean += d n_b / n, M2 += M2_b + d^2 n_a n_b / n): a shift that happens to be an
// unlucky value then costs precision in one workgroup's few hundred rows only.
#include "common.hpp"

namespace tango {

constexpr int kBnMaxGroups = 512;  // workgroups (partials) of the column reductions

// Rows that workgroup b of `groups` reduces: row r belongs to workgroup (r / row_lanes) % groups.
__host__ __device__ inline int64_t bn_group_rows(int64_t rows, int row_lanes, int groups, int b) {
    const int64_t period = static_cast<int64_t>(groups) * row_lanes;
    const int64_t rem = rows % period - static_cast<int64_t>(b) * row_lanes;
    return rows / period * row_lanes + (rem < 0 ? 0 : (rem > row_lanes ? row_lanes : rem));
}

// The shift of a workgroup's sums in column c: the median of the column's elements in the workgroup's first three
// rows (one outlier among them is not taken).
__device__ __forceinline__ float bn_shift(const float* __restrict__ x, int64_t first_row, int64_t rows, int C, int c) {
    const int64_t r1 = first_row + 1 < rows ? first_row + 1 : first_row, r2 = first_row + 2 < rows ? first_row + 2 : first_row;
    const float a = x[first_row * C + c], b = x[r1 * C + c], d = x[r2 * C + c];
    return fmaxf(fminf(a, b), fminf(fmaxf(a, b), d));
}

// Column layout of the reductions: a thread owns VEC consecutive columns (VEC = 4, 2 or 1: the widest that divides C
// and keeps the loads aligned) of one row lane.  gridDim.y cuts the C / VEC column groups into chunks of at most
// 256; a workgroup has 256 / (groups of its chunk) row lanes (threads beyond are idle).
struct BnChunk {
    int g0, cg, cw, row_lanes;  // first column group, groups and columns of the chunk, row lanes of its workgroups
};
__host__ __device__ inline BnChunk bn_chunk(int C, int vec, int chunk) {
    const int cg_all = C / vec;
    BnChunk k;
    k.g0 = chunk * 256;
    k.cg = cg_all - k.g0 < 256 ? cg_all - k.g0 : 256;
    k.cw = k.cg * vec;
    k.row_lanes = 256 / k.cg;
    return k;
}

template <int VEC>
struct BnVec {
    typedef float T __attribute__((ext_vector_type(VEC)));
    static __device__ __forceinline__ void load(const float* p, float* v) {
        const T t = __builtin_nontemporal_load(reinterpret_cast<const T*>(p));
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[i] = t[i];
    }
    static __device__ __forceinline__ void store(float* p, const float* v) {
        T t;
#pragma unroll
        for (int i = 0; i < VEC; ++i) t[i] = v[i];
        __builtin_nontemporal_store(t, reinterpret_cast<T*>(p));
    }
};
template <>
struct BnVec<1> {
    static __device__ __forceinline__ void load(const float* p, float* v) { v[0] = __builtin_nontemporal_load(p); }
    static __device__ __forceinline__ void store(float* p, const float* v) { __builtin_nontemporal_store(v[0], p); }
};

// DYNAMIC LDS: 2 * 256 * VEC floats (2 * row_lanes * columns of the chunk at most).
// MODE 0: partial = (mean, sum of squared deviations) of the workgroup's rows, from s1 = sum(x - k), s2 = sum((x - k)^2).
// MODE 1: s1 = sum(dy'), s2 = sum(dy' * xhat), dy' = dy where the forward output was positive (relu) else 0.
template <int MODE, int VEC>
__global__ __launch_bounds__(256) void bn_reduce_kernel(const float* __restrict__ x, const float* __restrict__ dy,
                                                        const float* __restrict__ mean, const float* __restrict__ rstd,
                                                        const float* __restrict__ gamma, const float* __restrict__ beta,
                                                        int64_t rows, int C, int relu, float* __restrict__ partial) {
    extern __shared__ float red[];  // [2][row_lanes][cw]
    const BnChunk ck = bn_chunk(C, VEC, blockIdx.y);
    const int row_lanes = ck.row_lanes, cw = ck.cw;
    const int grp = threadIdx.x % ck.cg, rl = threadIdx.x / ck.cg;
    const bool active = rl < row_lanes;
    const int c0 = (ck.g0 + grp) * VEC;
    float k[VEC], a[VEC], b[VEC], mu[VEC], rs[VEC], s1[VEC], s2[VEC];
    // The number of workgroups comes from the chunk with the fewest row lanes; in a narrower chunk (more row lanes)
    // the last workgroups may have no row at all: they read nothing and hand in an empty partial.
    const int64_t first_row = static_cast<int64_t>(blockIdx.x) * row_lanes;
    const bool has_rows = first_row < rows;
    float sh[3][VEC];
    if (MODE == 0 && has_rows) {  // the three rows of bn_shift, one load each
        const int64_t r1 = first_row + 1 < rows ? first_row + 1 : first_row, r2 = first_row + 2 < rows ? first_row + 2 : first_row;
        BnVec<VEC>::load(x + first_row * C + c0, sh[0]);
        BnVec<VEC>::load(x + r1 * C + c0, sh[1]);
        BnVec<VEC>::load(x + r2 * C + c0, sh[2]);
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
        k[i] = a[i] = b[i] = mu[i] = rs[i] = s1[i] = s2[i] = 0.0f;
        if (MODE == 0) {
            if (has_rows) k[i] = fmaxf(fminf(sh[0][i], sh[1][i]), fminf(fmaxf(sh[0][i], sh[1][i]), sh[2][i]));
        } else {
            mu[i] = mean[c0 + i];
            rs[i] = rstd[c0 + i];
            a[i] = rs[i] * gamma[c0 + i];
            b[i] = beta[c0 + i];
        }
    }
    const int64_t step = static_cast<int64_t>(gridDim.x) * row_lanes;
    auto take = [&](const float* xs, const float* ds) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            if (MODE == 0) {
                const float d = xs[i] - k[i];
                s1[i] += d;
                s2[i] += d * d;
            } else {
                const float c = xs[i] - mu[i];
                float g = ds[i];
                if (relu && !(c * a[i] + b[i] > 0.0f)) g = 0.0f;  // the forward's own arithmetic: same sign
                s1[i] += g;
                s2[i] += g * (c * rs[i]);
            }
        }
    };
    if (active) {
        int64_t r = static_cast<int64_t>(blockIdx.x) * row_lanes + rl;
        for (; r + 3 * step < rows; r += 4 * step) {  // four rows in flight per thread
            float xv[4][VEC], dv[4][VEC];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                BnVec<VEC>::load(x + (r + u * step) * C + c0, xv[u]);
                if (MODE == 1) BnVec<VEC>::load(dy + (r + u * step) * C + c0, dv[u]);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) take(xv[u], dv[u]);
        }
        for (; r < rows; r += step) {
            float xv[VEC], dv[VEC];
            BnVec<VEC>::load(x + r * C + c0, xv);
            if (MODE == 1) BnVec<VEC>::load(dy + r * C + c0, dv);
            take(xv, dv);
        }
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            red[rl * cw + grp * VEC + i] = s1[i];
            red[(row_lanes + rl) * cw + grp * VEC + i] = s2[i];
        }
    }
    __syncthreads();
    float* mine = partial + static_cast<int64_t>(blockIdx.x) * 2 * C + ck.g0 * VEC;  // this chunk's columns of slab b
    if (MODE == 0) {
        const int64_t nb = bn_group_rows(rows, row_lanes, gridDim.x, blockIdx.x);
        for (int c = threadIdx.x; c < cw; c += 256) {  // the row lanes in order
            float t1 = 0.0f, t2 = 0.0f;
            for (int l = 0; l < row_lanes; ++l) {
                t1 += red[l * cw + c];
                t2 += red[(row_lanes + l) * cw + c];
            }
            if (!has_rows) {  // nb == 0: skipped by the merge
                mine[c] = 0.0f;
                mine[C + c] = 0.0f;
                continue;
            }
            const float n = static_cast<float>(nb);
            const float m2 = t2 - t1 * (t1 / n);
            mine[c] = bn_shift(x, first_row, rows, C, ck.g0 * VEC + c) + t1 / n;
            mine[C + c] = m2 > 0.0f ? m2 : 0.0f;
        }
        return;
    }
    for (int j = threadIdx.x; j < 2 * cw; j += 256) {  // (which, column of the chunk): the row lanes in order
        const int which = j / cw, c = j - which * cw;
        float t = 0.0f;
        for (int l = 0; l < row_lanes; ++l) t += red[(which * row_lanes + l) * cw + c];
        mine[which * C + c] = t;
    }
}

// Merges the partials of 16 columns (64 partial lanes each, fixed order) and finishes the statistics.
// MODE 0: the workgroups' (mean, M2) pairs -> mean, biased variance, 1 / sqrt(var + eps).
// MODE 1: out1 = sum of the first partials (dbeta), out2 = sum of the second (dgamma).
template <int MODE>
__global__ __launch_bounds__(1024) void bn_finish_kernel(const float* __restrict__ partial, int groups, int C, int64_t rows,
                                                         int vec, float eps, float* __restrict__ out1,
                                                         float* __restrict__ out2, float* __restrict__ out3) {
    __shared__ float red[3][64][16];
    const int e = threadIdx.x & 15, sl = threadIdx.x >> 4;
    const int c = blockIdx.x * 16 + e;
    // MODE 0: (n, mean, M2) of the rows merged so far; MODE 1: t1, t2 = plain sums
    float n = 0.0f, t1 = 0.0f, t2 = 0.0f;
    auto merge = [&](float nb, float mb, float m2b) {
        if (nb <= 0.0f) return;
        const float tot = n + nb, d = mb - t1;
        t1 = t1 + d * (nb / tot);
        t2 = t2 + m2b + d * d * (n * (nb / tot));
        n = tot;
    };
    // rows of workgroup g (bn_group_rows, with the row lanes of this column's chunk): whole periods, plus its window
    // of the last, partial one
    const int row_lanes = bn_chunk(C, vec, (c < C ? c : 0) / vec / 256).row_lanes;
    const int64_t period = static_cast<int64_t>(groups) * row_lanes;
    const int64_t whole = rows / period * row_lanes, tail = rows % period;
    if (c < C)
        for (int g = sl; g < groups; g += 64) {
            const float p1 = partial[static_cast<int64_t>(g) * 2 * C + c];
            const float p2 = partial[static_cast<int64_t>(g) * 2 * C + C + c];
            if (MODE == 0) {
                const int64_t rem = tail - static_cast<int64_t>(g) * row_lanes;
                merge(static_cast<float>(whole + (rem < 0 ? 0 : (rem > row_lanes ? row_lanes : rem))), p1, p2);
            } else {
                t1 += p1;
                t2 += p2;
            }
        }
    red[0][sl][e] = n;
    red[1][sl][e] = t1;
    red[2][sl][e] = t2;
    __syncthreads();
    // the 64 partial lanes of a column fold pairwise: lane sl takes in lane sl + half (a fixed tree)
    for (int half = 32; half >= 1; half >>= 1) {
        if (sl < half) {
            if (MODE == 0) {
                merge(red[0][sl + half][e], red[1][sl + half][e], red[2][sl + half][e]);
            } else {
                t1 += red[1][sl + half][e];
                t2 += red[2][sl + half][e];
            }
            red[0][sl][e] = n;
            red[1][sl][e] = t1;
            red[2][sl][e] = t2;
        }
        __syncthreads();
    }
    if (sl == 0 && c < C) {
        if (MODE == 0) {
            const float var = t2 / n;  // biased variance
            out1[c] = t1;
            out2[c] = var;
            out3[c] = 1.0f / sqrtf(var + eps);
        } else {
            out1[c] = t1;
            out2[c] = t2;
        }
    }
}

// y = (x - mean) * (rstd * gamma) + beta, ReLU if asked; optionally max|y| / 127 into scale_out (pre-zeroed).
// Backward (BWD): dx = (rstd * gamma) * (dy' - dbeta / n - xhat * dgamma / n).
template <bool BWD, int VEC>
__global__ __launch_bounds__(256) void bn_apply_kernel(float* __restrict__ out, const float* __restrict__ x,
                                                       const float* __restrict__ dy, const float* __restrict__ mean,
                                                       const float* __restrict__ rstd, const float* __restrict__ gamma,
                                                       const float* __restrict__ beta, const float* __restrict__ dbeta,
                                                       const float* __restrict__ dgamma, int64_t rows, int C, int relu,
                                                       float* __restrict__ scale_out) {
    extern __shared__ float par[];  // [6][C]: mean, rstd, a = rstd * gamma, beta, dbeta / n, dgamma / n
    const float inv_n = 1.0f / static_cast<float>(rows);
    for (int c = threadIdx.x; c < C; c += 256) {
        par[c] = mean[c];
        par[C + c] = rstd[c];
        par[2 * C + c] = rstd[c] * gamma[c];
        par[3 * C + c] = beta[c];
        par[4 * C + c] = BWD ? dbeta[c] * inv_n : 0.0f;
        par[5 * C + c] = BWD ? dgamma[c] * inv_n : 0.0f;
    }
    __syncthreads();
    const int cg = C / VEC;
    const int64_t nv = rows * cg;
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int64_t nthr = static_cast<int64_t>(gridDim.x) * blockDim.x;
    int grp = static_cast<int>(tid % cg);
    const int gstep = static_cast<int>(nthr % cg);
    float m = 0.0f;
    for (int64_t i = tid; i < nv; i += nthr) {
        const int c0 = grp * VEC;
        float xs[VEC], ds[VEC], o[VEC];
        BnVec<VEC>::load(x + i * VEC, xs);
        if (!BWD) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                float y = (xs[k] - par[c0 + k]) * par[2 * C + c0 + k] + par[3 * C + c0 + k];
                if (relu && !(y > 0.0f)) y = 0.0f;
                o[k] = y;
                m = fmaxf(m, fabsf(y));
            }
        } else {
            BnVec<VEC>::load(dy + i * VEC, ds);
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                const float c = xs[k] - par[c0 + k];
                float g = ds[k];
                if (relu && !(c * par[2 * C + c0 + k] + par[3 * C + c0 + k] > 0.0f)) g = 0.0f;
                o[k] = par[2 * C + c0 + k] * (g - par[4 * C + c0 + k] - (c * par[C + c0 + k]) * par[5 * C + c0 + k]);
            }
        }
        BnVec<VEC>::store(out + i * VEC, o);
        grp += gstep;
        if (grp >= cg) grp -= cg;
    }
    if (!BWD && scale_out) block_absmax_to_global(m / 127.0f, scale_out);
}

constexpr int kBnMaxCols = 2048;

// the widest vector that divides the row length and keeps every row's loads aligned
static int bn_vec(int64_t C, uintptr_t addr_bits) {
    return (C % 4 == 0 && (addr_bits & 15) == 0) ? 4 : (C % 2 == 0 && (addr_bits & 7) == 0) ? 2 : 1;
}

// Workgroups of the reductions; sized for the narrowest vector so that the workspace does not depend on alignment
static int bn_groups(int64_t rows, int64_t C, int vec) {
    const int64_t cg = C / vec;
    const int64_t row_lanes = 256 / (cg < 256 ? cg : 256);
    const int64_t g = ceil_div(rows, row_lanes * 8);  // at least eight rows per thread
    return static_cast<int>(g < 1 ? 1 : (g < kBnMaxGroups ? g : kBnMaxGroups));
}

static bool bn_shape_ok(int64_t rows, int64_t C) { return rows > 0 && C >= 1 && C <= kBnMaxCols; }

template <int MODE>
static void bn_launch_reduce(int vec, dim3 grid, hipStream_t s, const float* x, const float* dy, const float* mean,
                             const float* rstd, const float* gamma, const float* beta, int64_t rows, int C, int relu,
                             float* partial) {
    const size_t lds = sizeof(float) * 2 * 256 * vec;
    if (vec == 4)
        hipLaunchKernelGGL((bn_reduce_kernel<MODE, 4>), grid, dim3(256), lds, s, x, dy, mean, rstd, gamma, beta, rows, C, relu, partial);
    else if (vec == 2)
        hipLaunchKernelGGL((bn_reduce_kernel<MODE, 2>), grid, dim3(256), lds, s, x, dy, mean, rstd, gamma, beta, rows, C, relu, partial);
    else
        hipLaunchKernelGGL((bn_reduce_kernel<MODE, 1>), grid, dim3(256), lds, s, x, dy, mean, rstd, gamma, beta, rows, C, relu, partial);
}

template <bool BWD>
static void bn_launch_apply(int vec, hipStream_t s, float* out, const float* x, const float* dy, const float* mean,
                            const float* rstd, const float* gamma, const float* beta, const float* dbeta,
                            const float* dgamma, int64_t rows, int C, int relu, float* scale_out) {
    const dim3 grid(grid_for(rows * (C / vec), 256));
    const size_t lds = sizeof(float) * 6 * C;
    if (vec == 4)
        hipLaunchKernelGGL((bn_apply_kernel<BWD, 4>), grid, dim3(256), lds, s, out, x, dy, mean, rstd, gamma, beta, dbeta, dgamma, rows, C, relu, scale_out);
    else if (vec == 2)
        hipLaunchKernelGGL((bn_apply_kernel<BWD, 2>), grid, dim3(256), lds, s, out, x, dy, mean, rstd, gamma, beta, dbeta, dgamma, rows, C, relu, scale_out);
    else
        hipLaunchKernelGGL((bn_apply_kernel<BWD, 1>), grid, dim3(256), lds, s, out, x, dy, mean, rstd, gamma, beta, dbeta, dgamma, rows, C, relu, scale_out);
}

}  // namespace tango

using namespace tango;

extern "C" {

size_t tango_batchnorm_workspace(int64_t rows, int64_t cols) {
    if (!bn_shape_ok(rows, cols)) return 0;
    return static_cast<size_t>(kBnMaxGroups) * 2 * cols * sizeof(float);
}

int tango_batchnorm_fwd_f32(float* y, float* mean, float* var, float* rstd, float* scale_y, const float* x,
                            const float* gamma, const float* beta, int64_t rows, int64_t cols, float eps, int relu,
                            void* workspace, size_t workspace_bytes, tango_stream_t stream) {
    if (rows < 0 || cols < 0) return TANGO_ERR_INVALID_ARG;
    if (rows == 0 || cols == 0) return TANGO_OK;
    if (!bn_shape_ok(rows, cols)) return TANGO_ERR_UNSUPPORTED;
    if (!y || !mean || !var || !rstd || !x || !gamma || !beta) return TANGO_ERR_INVALID_ARG;
    if (((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 3) != 0) return TANGO_ERR_INVALID_ARG;
    const size_t need = tango_batchnorm_workspace(rows, cols);
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15) != 0)
        return TANGO_ERR_WORKSPACE;
    hipStream_t s = as_stream(stream);
    const int C = static_cast<int>(cols);
    const int vec = bn_vec(cols, reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y));
    const int groups = bn_groups(rows, cols, vec);
    const dim3 rgrid(groups, static_cast<unsigned>(ceil_div(cols / vec, 256)));
    float* partial = static_cast<float*>(workspace);
    if (scale_y) fill_u32(scale_y, 0u, 1, s);
    bn_launch_reduce<0>(vec, rgrid, s, x, nullptr, nullptr, nullptr, nullptr, nullptr, rows, C, 0, partial);
    hipLaunchKernelGGL(bn_finish_kernel<0>, dim3((C + 15) / 16), dim3(1024), 0, s, partial, groups, C, rows, vec, eps, mean, var,
                       rstd);
    bn_launch_apply<false>(vec, s, y, x, nullptr, mean, rstd, gamma, beta, nullptr, nullptr, rows, C, relu, scale_y);
    return launch_status();
}

int tango_batchnorm_bwd_f32(float* dx, float* dgamma, float* dbeta, const float* dy, const float* x,
                            const float* mean, const float* rstd, const float* gamma, const float* beta, int64_t rows,
                            int64_t cols, int relu, void* workspace, size_t workspace_bytes, tango_stream_t stream) {
    if (rows < 0 || cols < 0) return TANGO_ERR_INVALID_ARG;
    if (rows == 0 || cols == 0) return TANGO_OK;
    if (!bn_shape_ok(rows, cols)) return TANGO_ERR_UNSUPPORTED;
    if (!dx || !dgamma || !dbeta || !dy || !x || !mean || !rstd || !gamma || !beta) return TANGO_ERR_INVALID_ARG;
    const uintptr_t bits = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(dy) | reinterpret_cast<uintptr_t>(dx);
    if ((bits & 3) != 0) return TANGO_ERR_INVALID_ARG;
    const size_t need = tango_batchnorm_workspace(rows, cols);
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15) != 0)
        return TANGO_ERR_WORKSPACE;
    hipStream_t s = as_stream(stream);
    const int C = static_cast<int>(cols);
    const int vec = bn_vec(cols, bits);
    const int groups = bn_groups(rows, cols, vec);
    const dim3 rgrid(groups, static_cast<unsigned>(ceil_div(cols / vec, 256)));
    float* partial = static_cast<float*>(workspace);
    bn_launch_reduce<1>(vec, rgrid, s, x, dy, mean, rstd, gamma, beta, rows, C, relu, partial);
    hipLaunchKernelGGL(bn_finish_kernel<1>, dim3((C + 15) / 16), dim3(1024), 0, s, partial, groups, C, rows, vec, 0.0f, dbeta,
                       dgamma, nullptr);
    bn_launch_apply<true>(vec, s, dx, x, dy, mean, rstd, gamma, beta, dbeta, dgamma, rows, C, relu, nullptr);
    return launch_status();
}

}  // extern "C"
