// GAT attention logits per node and head, with their backward.
//
//   el[n, h] = sum_d feat[n, h, d] * attn_l[h, d]      er likewise with attn_r
//
// Not part of the reference's primitive layer: its GAT driver writes this as
// broadcast-multiply + sum in torch (evaluation/test_gat.py:135-137), which costs
// four elementwise/reduction passes forward and, backward, two column reductions
// over all nodes that torch runs far below memory speed.  fp32, HBM-bound: the
// forward reads feat once (4 bytes per element), the backward reads feat once and
// writes d_feat once (8 bytes per element) and reduces the two [H, D] parameter
// gradients in a fixed order (registers over a thread's rows, LDS over a
// workgroup's threads, one slab per workgroup, then a finishing kernel), so the
// result is deterministic.
#include "common.hpp"

namespace tango {

constexpr int kBwdGroups = 1024;  // workgroups (slabs) of the backward reduction

// One (node, head) item per thread and loop step.  SCALES: the launch is a fixed number of large workgroups
// walking the items with a grid stride, and each ends with one atomic max per output of max|el| / 127 and
// max|er| / 127 into pre-zeroed slots, so the quantize passes that follow need no absmax pass of their own.
template <bool SCALES>
__global__ __launch_bounds__(SCALES ? 1024 : 256) void attn_scores_fwd_kernel(
    float* __restrict__ el, float* __restrict__ er, float* __restrict__ scale_el, float* __restrict__ scale_er,
    const float* __restrict__ feat, const float* __restrict__ al, const float* __restrict__ ar, int64_t total,
    int H, int D, int vec4) {
    const int64_t nthr = static_cast<int64_t>(gridDim.x) * blockDim.x;
    float ml = 0.0f, mr = 0.0f;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += nthr) {
        const int h = static_cast<int>(i % H);
        const float* f = feat + i * D;
        const float* a = al + static_cast<int64_t>(h) * D;
        const float* b = ar + static_cast<int64_t>(h) * D;
        float sl = 0.0f, sr = 0.0f;
        if (vec4) {
            for (int d = 0; d < D; d += 4) {
                const f32x4 x = *reinterpret_cast<const f32x4*>(f + d);
                const f32x4 u = *reinterpret_cast<const f32x4*>(a + d);
                const f32x4 v = *reinterpret_cast<const f32x4*>(b + d);
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    sl += x[k] * u[k];
                    sr += x[k] * v[k];
                }
            }
        } else {
            for (int d = 0; d < D; ++d) {
                sl += f[d] * a[d];
                sr += f[d] * b[d];
            }
        }
        el[i] = sl;
        er[i] = sr;
        if (SCALES) {
            ml = fmaxf(ml, fabsf(sl));
            mr = fmaxf(mr, fabsf(sr));
        }
    }
    if (SCALES) {
        block_absmax_to_global(ml / 127.0f, scale_el);
        __syncthreads();  // the helper's staging array is reused by the second call
        block_absmax_to_global(mr / 127.0f, scale_er);
    }
}

// Wide heads (D >= 128): one wavefront per (node, head) item, its lanes striding over the head's columns VEC floats
// at a time (consecutive bytes per load instruction, where a thread per item reads D floats at a stride of D floats),
// then a butterfly over the lanes: a fixed order.  Launched like attn_scores_fwd_kernel.
template <bool SCALES, int VEC>
__global__ __launch_bounds__(SCALES ? 1024 : 256) void attn_scores_fwd_wide_kernel(
    float* __restrict__ el, float* __restrict__ er, float* __restrict__ scale_el, float* __restrict__ scale_er,
    const float* __restrict__ feat, const float* __restrict__ al, const float* __restrict__ ar, int64_t total,
    int H, int D) {
    typedef float fvec __attribute__((ext_vector_type(VEC == 1 ? 2 : VEC)));  // (unused for VEC == 1)
    const int lane = threadIdx.x & 63;
    const int64_t nwaves = static_cast<int64_t>(gridDim.x) * (blockDim.x >> 6);
    float ml = 0.0f, mr = 0.0f;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6); i < total; i += nwaves) {
        const int h = static_cast<int>(i % H);
        const float* f = feat + i * D;
        const float* a = al + static_cast<int64_t>(h) * D;
        const float* b = ar + static_cast<int64_t>(h) * D;
        float sl = 0.0f, sr = 0.0f;
        for (int d = lane * VEC; d < D; d += 64 * VEC) {
            if (VEC > 1) {
                const fvec x = __builtin_nontemporal_load(reinterpret_cast<const fvec*>(f + d));
                const fvec u = *reinterpret_cast<const fvec*>(a + d);
                const fvec v = *reinterpret_cast<const fvec*>(b + d);
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    sl += x[k] * u[k];
                    sr += x[k] * v[k];
                }
            } else {
                sl += f[d] * a[d];
                sr += f[d] * b[d];
            }
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            sl += __shfl_xor(sl, off, 64);
            sr += __shfl_xor(sr, off, 64);
        }
        if (lane == 0) {
            el[i] = sl;
            er[i] = sr;
        }
        if (SCALES) {
            ml = fmaxf(ml, fabsf(sl));
            mr = fmaxf(mr, fabsf(sr));
        }
    }
    if (SCALES) {
        block_absmax_to_global(ml / 127.0f, scale_el);
        __syncthreads();  // the helper's staging array is reused by the second call
        block_absmax_to_global(mr / 127.0f, scale_er);
    }
}

// d_feat = del * attn_l + der * attn_r and the two [H, D] parameter gradients (sums over the rows of del * feat and
// der * feat), with the rows read the way they lie in memory: a thread owns VEC consecutive columns
// (of the H * D of a row; VEC = 4 or 2 needs D % VEC == 0 so that they share a head) of one of the row lanes of its
// workgroup: a wavefront's loads and stores cover consecutive bytes (a thread per (row, head) would read D floats
// at a stride of D floats).  part[b][2][H][D]: workgroup b's sums.  gridDim.y cuts the H * D / VEC column groups into chunks of at most 256; a workgroup
// has 256 / (groups of its chunk) row lanes.
// ACC: d_feat = addend + (del * attn_l + der * attn_r), the sum autograd would form in a pass of its own when feat
// has a second consumer whose gradient is ``addend``, and max|d_feat| / 127 goes to *scale_out (which holds 0).
// DYNAMIC LDS: 2 * 256 * VEC floats at most (2 * row_lanes * columns of the chunk).
template <int VEC, bool ACC>
__global__ __launch_bounds__(256) void attn_scores_bwd_rows_kernel(
    float* __restrict__ dfeat, float* __restrict__ part, const float* __restrict__ del,
    const float* __restrict__ der, const float* __restrict__ feat, const float* __restrict__ al,
    const float* __restrict__ ar, const float* __restrict__ addend, float* __restrict__ scale_out, int64_t n, int H,
    int D) {
    extern __shared__ float red_rows[];  // [2][row_lanes][cw]
    typedef float fvec __attribute__((ext_vector_type(VEC == 1 ? 2 : VEC)));  // (unused for VEC == 1)
    const int C = H * D;
    const int cg_all = C / VEC;
    const int g0 = blockIdx.y * 256;                               // first column group of this chunk
    const int cg = cg_all - g0 < 256 ? cg_all - g0 : 256;          // column groups of this chunk
    const int cw = cg * VEC;                                       // its columns
    const int row_lanes = 256 / cg;
    const int grp = threadIdx.x % cg, rl = threadIdx.x / cg;
    const int c0 = (g0 + grp) * VEC;
    const int h = c0 / D;
    float wl[VEC], wr[VEC], accl[VEC], accr[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        wl[k] = al[c0 + k];
        wr[k] = ar[c0 + k];
        accl[k] = accr[k] = 0.0f;
    }
    float m = 0.0f;
    if (rl < row_lanes) {
        const int64_t step = static_cast<int64_t>(gridDim.x) * row_lanes;
        for (int64_t r = static_cast<int64_t>(blockIdx.x) * row_lanes + rl; r < n; r += step) {
            const float gl = del[r * H + h], gr = der[r * H + h];
            float x[VEC], y[VEC], a[VEC];
            if (VEC > 1) {
                const fvec v = __builtin_nontemporal_load(reinterpret_cast<const fvec*>(feat + r * C + c0));
                fvec u = v;
                if (ACC) u = __builtin_nontemporal_load(reinterpret_cast<const fvec*>(addend + r * C + c0));
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    x[k] = v[k];
                    a[k] = u[k];
                }
            } else {
                x[0] = feat[r * C + c0];
                a[0] = ACC ? addend[r * C + c0] : 0.0f;
            }
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                y[k] = gl * wl[k] + gr * wr[k];
                if (ACC) {
                    y[k] = a[k] + y[k];
                    m = fmaxf(m, fabsf(y[k]));
                }
                accl[k] += gl * x[k];
                accr[k] += gr * x[k];
            }
            if (VEC > 1) {
                fvec o;
#pragma unroll
                for (int k = 0; k < VEC; ++k) o[k] = y[k];
                *reinterpret_cast<fvec*>(dfeat + r * C + c0) = o;
            } else {
                dfeat[r * C + c0] = y[0];
            }
        }
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            red_rows[rl * cw + grp * VEC + k] = accl[k];
            red_rows[(row_lanes + rl) * cw + grp * VEC + k] = accr[k];
        }
    }
    __syncthreads();
    for (int j = threadIdx.x; j < 2 * cw; j += 256) {  // (which, column of the chunk): the row lanes in order
        const int which = j / cw, c = j - which * cw;
        float t = 0.0f;
        for (int l = 0; l < row_lanes; ++l) t += red_rows[(which * row_lanes + l) * cw + c];
        part[(static_cast<int64_t>(blockIdx.x) * 2 + which) * C + g0 * VEC + c] = t;
    }
    if (ACC) block_absmax_to_global(m / 127.0f, scale_out);
}

// out[0 .. 2 H D) = sum over slabs, 64 slab lanes per element, fixed order.
__global__ __launch_bounds__(1024) void attn_scores_finish_kernel(float* __restrict__ dal, float* __restrict__ dar,
                                                                  const float* __restrict__ part, int slabs,
                                                                  int64_t hd) {
    __shared__ float red[64][16];
    const int e = threadIdx.x & 15, sl = threadIdx.x >> 4;
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 16 + e;
    float s = 0.0f;
    if (idx < 2 * hd)
        for (int b = sl; b < slabs; b += 64) s += part[static_cast<int64_t>(b) * 2 * hd + idx];
    red[sl][e] = s;
    __syncthreads();
    if (sl == 0 && idx < 2 * hd) {
        float tot = 0.0f;
#pragma unroll
        for (int w = 0; w < 64; ++w) tot += red[w][e];
        if (idx < hd) dal[idx] = tot; else dar[idx - hd] = tot;
    }
}

static int bwd_groups(int64_t n, int64_t H) {
    const int64_t slots = (256 / H);
    const int64_t g = ceil_div(n, slots);
    return static_cast<int>(g < kBwdGroups ? (g < 1 ? 1 : g) : kBwdGroups);
}

}  // namespace tango

using namespace tango;

extern "C" {

int tango_attn_scores_fwd(float* el, float* er, float* scale_el, float* scale_er, const float* feat,
                          const float* attn_l, const float* attn_r, int64_t n, int64_t H, int64_t D,
                          tango_stream_t stream) {
    if (n < 0 || H < 0 || D < 0 || H >= (1LL << 31) || D >= (1LL << 31)) return TANGO_ERR_INVALID_ARG;
    if ((scale_el == nullptr) != (scale_er == nullptr)) return TANGO_ERR_INVALID_ARG;
    if (n * H == 0) return TANGO_OK;
    if (!el || !er || (D > 0 && (!feat || !attn_l || !attn_r))) return TANGO_ERR_INVALID_ARG;
    const int64_t total = n * H;
    if (ceil_div(total, 256) > INT32_MAX) return TANGO_ERR_UNSUPPORTED;
    const uintptr_t bits = reinterpret_cast<uintptr_t>(feat) | reinterpret_cast<uintptr_t>(attn_l) |
                           reinterpret_cast<uintptr_t>(attn_r);
    const int vec4 = (D % 4 == 0) && (bits & 15) == 0;
    if (D >= 128) {  // a wavefront per item
        const int vec = vec4 ? 4 : (D % 2 == 0 && (bits & 7) == 0) ? 2 : 1;
        const int64_t want = ceil_div(total, scale_el ? 16 : 4);  // items per workgroup = its wavefronts
        const hipStream_t s = as_stream(stream);
        const int Hi = static_cast<int>(H), Di = static_cast<int>(D);
        if (scale_el) {
            const dim3 grid(static_cast<unsigned>(want < 512 ? want : 512));
            if (vec == 4) hipLaunchKernelGGL((attn_scores_fwd_wide_kernel<true, 4>), grid, dim3(1024), 0, s, el, er, scale_el, scale_er, feat, attn_l, attn_r, total, Hi, Di);
            else if (vec == 2) hipLaunchKernelGGL((attn_scores_fwd_wide_kernel<true, 2>), grid, dim3(1024), 0, s, el, er, scale_el, scale_er, feat, attn_l, attn_r, total, Hi, Di);
            else hipLaunchKernelGGL((attn_scores_fwd_wide_kernel<true, 1>), grid, dim3(1024), 0, s, el, er, scale_el, scale_er, feat, attn_l, attn_r, total, Hi, Di);
        } else {
            const dim3 grid(static_cast<unsigned>(want < 8192 ? want : 8192));
            if (vec == 4) hipLaunchKernelGGL((attn_scores_fwd_wide_kernel<false, 4>), grid, dim3(256), 0, s, el, er, scale_el, scale_er, feat, attn_l, attn_r, total, Hi, Di);
            else if (vec == 2) hipLaunchKernelGGL((attn_scores_fwd_wide_kernel<false, 2>), grid, dim3(256), 0, s, el, er, scale_el, scale_er, feat, attn_l, attn_r, total, Hi, Di);
            else hipLaunchKernelGGL((attn_scores_fwd_wide_kernel<false, 1>), grid, dim3(256), 0, s, el, er, scale_el, scale_er, feat, attn_l, attn_r, total, Hi, Di);
        }
        return launch_status();
    }
    if (scale_el) {
        // one 16-wave workgroup per compute unit at most: a few hundred atomics per slot in all
        const int64_t want = ceil_div(total, 1024);
        const unsigned groups = static_cast<unsigned>(want < 256 ? want : 256);
        hipLaunchKernelGGL(attn_scores_fwd_kernel<true>, dim3(groups), dim3(1024), 0, as_stream(stream), el, er,
                           scale_el, scale_er, feat, attn_l, attn_r, total, static_cast<int>(H),
                           static_cast<int>(D), vec4);
    } else {
        hipLaunchKernelGGL(attn_scores_fwd_kernel<false>, dim3(static_cast<unsigned>(ceil_div(total, 256))),
                           dim3(256), 0, as_stream(stream), el, er, scale_el, scale_er, feat, attn_l, attn_r, total,
                           static_cast<int>(H), static_cast<int>(D), vec4);
    }
    return launch_status();
}

size_t tango_attn_scores_bwd_workspace(int64_t n, int64_t H, int64_t D) {
    if (n <= 0 || H <= 0 || D <= 0 || H > 256) return 0;
    return static_cast<size_t>(bwd_groups(n, H)) * 2 * H * D * sizeof(float);
}

static int attn_scores_bwd_impl(float* dfeat, float* dattn_l, float* dattn_r, const float* del, const float* der,
                               const float* feat, const float* attn_l, const float* attn_r, const float* addend,
                               float* scale_out, int64_t n, int64_t H, int64_t D, void* workspace,
                               size_t workspace_bytes, tango_stream_t stream) {
    if (n < 0 || H < 0 || D < 0) return TANGO_ERR_INVALID_ARG;
    if (H * D == 0) return TANGO_OK;
    if (H > 256 || D >= (1LL << 31) || H * D > (1LL << 23)) return TANGO_ERR_UNSUPPORTED;
    if (!dattn_l || !dattn_r || !attn_l || !attn_r || (n > 0 && (!dfeat || !del || !der || !feat)))
        return TANGO_ERR_INVALID_ARG;
    hipStream_t s = as_stream(stream);
    int groups = 0;
    float* part = static_cast<float*>(workspace);
    if (n > 0) {
        const size_t need = tango_attn_scores_bwd_workspace(n, H, D);
        if (!workspace || workspace_bytes < need) return TANGO_ERR_WORKSPACE;
        if ((reinterpret_cast<uintptr_t>(workspace) & 3) != 0) return TANGO_ERR_INVALID_ARG;
        groups = bwd_groups(n, H);
        const uintptr_t bits = reinterpret_cast<uintptr_t>(feat) | reinterpret_cast<uintptr_t>(dfeat) |
                               reinterpret_cast<uintptr_t>(addend);
        const int64_t C = H * D;
        const int vec = (D % 4 == 0 && (bits & 15) == 0) ? 4 : (D % 2 == 0 && (bits & 7) == 0) ? 2 : 1;
        const int64_t cg_all = C / vec, chunks = ceil_div(cg_all, 256);
        {
            const int row_lanes = static_cast<int>(256 / (cg_all < 256 ? cg_all : 256));
            int64_t want = ceil_div(n, static_cast<int64_t>(row_lanes) * 8);  // eight rows per thread or more,
            if (want > 512) want = 512;                                          // two workgroups per compute unit at most
            groups = static_cast<int>(want < groups ? (want < 1 ? 1 : want) : groups);
            const size_t lds = sizeof(float) * 2 * 256 * vec;
            const dim3 grid(static_cast<unsigned>(groups), static_cast<unsigned>(chunks));
#define TANGO_ATTN_BWD(V, A)                                                                                    \
    hipLaunchKernelGGL((attn_scores_bwd_rows_kernel<V, A>), grid, dim3(256), lds, s, dfeat, part, del, der, feat,   \
                       attn_l, attn_r, addend, scale_out, n, static_cast<int>(H), static_cast<int>(D))
            if (addend) {
                if (vec == 4) TANGO_ATTN_BWD(4, true);
                else if (vec == 2) TANGO_ATTN_BWD(2, true);
                else TANGO_ATTN_BWD(1, true);
            } else {
                if (vec == 4) TANGO_ATTN_BWD(4, false);
                else if (vec == 2) TANGO_ATTN_BWD(2, false);
                else TANGO_ATTN_BWD(1, false);
            }
#undef TANGO_ATTN_BWD
        }
    }
    hipLaunchKernelGGL(attn_scores_finish_kernel, dim3(static_cast<unsigned>(ceil_div(2 * H * D, 16))), dim3(1024), 0,
                       s, dattn_l, dattn_r, part, groups, H * D);
    return launch_status();
}

int tango_attn_scores_bwd(float* dfeat, float* dattn_l, float* dattn_r, const float* del,
                          const float* der, const float* feat, const float* attn_l,
                          const float* attn_r, int64_t n, int64_t H, int64_t D, void* workspace,
                          size_t workspace_bytes, tango_stream_t stream) {
    return attn_scores_bwd_impl(dfeat, dattn_l, dattn_r, del, der, feat, attn_l, attn_r, nullptr, nullptr, n, H, D,
                                workspace, workspace_bytes, stream);
}

int tango_attn_scores_bwd_acc(float* dfeat, float* dattn_l, float* dattn_r, float* scale_out, const float* addend,
                              const float* del, const float* der, const float* feat, const float* attn_l,
                              const float* attn_r, int64_t n, int64_t H, int64_t D, void* workspace,
                              size_t workspace_bytes, tango_stream_t stream) {
    if (!scale_out || (n > 0 && H * D > 0 && !addend)) return TANGO_ERR_INVALID_ARG;
    if (addend == dfeat && n > 0 && H * D > 0) return TANGO_ERR_INVALID_ARG;  // the kernel's pointers do not alias
    return attn_scores_bwd_impl(dfeat, dattn_l, dattn_r, del, der, feat, attn_l, attn_r, addend, scale_out, n, H, D,
                                workspace, workspace_bytes, stream);
}

}  // extern "C"
