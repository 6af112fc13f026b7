/*
 * CPU oracle for the quantized-GNN primitive layer.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C with IEEE fp32 arithmetic and no fused
 * multiply-add, what each primitive of the reference computes.  It is the
 * checker for the HIP kernels and the CPU leg of the benchmark; nothing in the
 * shipped package may link, import or call it.
 *
 * Canonical semantics (the reference is compiled with --use_fast_math, whose
 * exact V100 bits cannot be reproduced anywhere else):
 *   scale  s = fl(max|x| / 127)
 *   rscale r = s > 0 ? fl(1 / s) : 0          (all-zero tensors quantize to 0)
 *   q      = clamp(round(fl(x * r)), -127, 127)
 * where round is half-to-even (stand-alone quantize), toward-zero (the GEMM's
 * fused quantize-on-load) or floor(. + u) (stochastic, an extension).
 *
 * Every integer accumulation is done in int64 and checked to fit int32, the
 * accumulator width of the reference; orc_overflow_count() reports violations.
 *
 * Parity status.  The reference holds no golden vectors for this path, so each
 * function is pinned by closed forms, brute force and invariants in
 * tests/test_oracle_*.py.  What stays "parity unpinned" because only NVIDIA
 * hardware or closed libraries could settle it: the fast-math bits of 1/scale
 * and max/127; cuSPARSE's fp32 summation order once |sum| >= 2^24 (u_mul_e);
 * whether the CUTLASS epilogue contracts bias + scale*acc; DGL's edge_softmax
 * numerics.  These are covered by tolerance, not by bit equality.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_ROUND_RNE 0
#define ORC_ROUND_TRUNC 1
#define ORC_ROUND_STOCHASTIC 2

static int64_t g_overflow = 0;

int64_t orc_overflow_count(void) { return g_overflow; }
void orc_overflow_reset(void) { g_overflow = 0; }

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void orc_set_num_threads(int n) {
#ifdef _OPENMP
    omp_set_num_threads(n);
#else
    (void)n;
#endif
}

static inline int32_t narrow_i32(int64_t v) {
    if (v > INT32_MAX || v < INT32_MIN) {
#pragma omp atomic
        g_overflow++;
    }
    /* two's-complement wrap, as the reference's int32 accumulators do
       (cuda/src/QGEMM_backward.cu:54 sums 232,965 products in int32) */
    return (int32_t)(uint32_t)(uint64_t)v;
}

/* ---------------------------------------------------------------- Philox -- */
/* Philox4x32-10 (Salmon et al., SC'11; Random123).  No counterpart in the
   reference: stochastic rounding is an extension.  Pinned by the published
   known-answer vectors. */
static inline void philox_round(uint32_t c[4], const uint32_t k[2]) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c[0];
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c[2];
    const uint32_t hi0 = (uint32_t)(p0 >> 32), lo0 = (uint32_t)p0;
    const uint32_t hi1 = (uint32_t)(p1 >> 32), lo1 = (uint32_t)p1;
    const uint32_t n0 = hi1 ^ c[1] ^ k[0];
    const uint32_t n2 = hi0 ^ c[3] ^ k[1];
    c[0] = n0;
    c[1] = lo1;
    c[2] = n2;
    c[3] = lo0;
}

void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
    uint32_t c[4] = {ctr[0], ctr[1], ctr[2], ctr[3]};
    uint32_t k[2] = {key[0], key[1]};
    for (int r = 0; r < 10; ++r) {
        philox_round(c, k);
        k[0] += 0x9E3779B9u;
        k[1] += 0xBB67AE85u;
    }
    memcpy(out, c, sizeof(c));
}

/* Uniform in [0,1) for global element index g: counter = (g >> 2) split into
   two 32-bit words, key = seed split likewise, lane = g & 3, u = top 24 bits
   scaled by 2^-24. */
float orc_philox_uniform(uint64_t seed, uint64_t g) {
    uint32_t ctr[4] = {(uint32_t)(g >> 2), (uint32_t)((g >> 2) >> 32), 0u, 0u};
    uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    uint32_t out[4];
    orc_philox4x32_10(ctr, key, out);
    return (float)(out[g & 3] >> 8) * 0x1.0p-24f;
}

/* ----------------------------------------------------------- quantization -- */

/* cuda/src/quantization.cu:45-93 (kernel_get_scale, get_scale_impl) with the
   tail fixed to cover every element (the reference skips element size4*4 and
   reads one past the end when numel % 4 != 0, quantization.cu:59-62). */
float orc_absmax_scale(const float *x, int64_t n) {
    float m = 0.0f;
    for (int64_t i = 0; i < n; ++i) {
        float a = fabsf(x[i]);
        if (a > m) m = a; /* NaN never wins, as with CUDA's max() */
    }
    volatile float s = m / 127.0f;
    return s;
}

/* Per-row variant (extension): s[r] = max_c |x[r, c]| / 127. */
void orc_absmax_rows(const float *x, int64_t rows, int64_t cols, int64_t ld, float *s) {
    for (int64_t r = 0; r < rows; ++r) s[r] = orc_absmax_scale(x + r * ld, cols);
}

static inline float rscale_of(float s) {
    volatile float r = s > 0.0f ? 1.0f / s : 0.0f;
    return r;
}

static inline int8_t quant_one(float x, float r, int mode, float u) {
    volatile float p = x * r; /* one rounding, never contracted */
    float v;
    if (mode == ORC_ROUND_RNE) {
        v = rintf(p); /* cuda/src/quantization.cu:10 (rintf) */
    } else if (mode == ORC_ROUND_TRUNC) {
        v = truncf(p); /* cuda/src/iterator.h:161 ((int8_t)(x * div_scale)) */
    } else {
        volatile float t = p + u;
        v = floorf(t);
    }
    if (!(v == v)) return 0; /* NaN input */
    if (v > 127.0f) v = 127.0f; /* cuda/src/quantization.cu:6 (clamp) */
    if (v < -127.0f) v = -127.0f;
    return (int8_t)(int)v;
}

/* cuda/src/quantization.cu:6-43 (kernel_quantize) for mode RNE;
   cuda/src/iterator.h:156-164 for mode TRUNC; extension for STOCHASTIC with
   either an injected noise tensor or Philox keyed by (seed, offset + i). */
void orc_quantize(const float *x, int64_t n, float scale, int8_t *q, int mode,
                  const float *noise, uint64_t seed, uint64_t offset) {
    const float r = rscale_of(scale);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        float u = 0.0f;
        if (mode == ORC_ROUND_STOCHASTIC)
            u = noise ? noise[i] : orc_philox_uniform(seed, offset + (uint64_t)i);
        q[i] = quant_one(x[i], r, mode, u);
    }
}

/* Row-strided form with one scale per row or one for the whole matrix. */
void orc_quantize_rows(const float *x, int64_t rows, int64_t cols, int64_t ldx,
                       const float *scales, int per_row, int8_t *q, int64_t ldq,
                       int mode, const float *noise, uint64_t seed, uint64_t offset) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float rs = rscale_of(per_row ? scales[r] : scales[0]);
        for (int64_t c = 0; c < cols; ++c) {
            float u = 0.0f;
            const int64_t lin = r * cols + c;
            if (mode == ORC_ROUND_STOCHASTIC)
                u = noise ? noise[lin] : orc_philox_uniform(seed, offset + (uint64_t)lin);
            q[r * ldq + c] = quant_one(x[r * ldx + c], rs, mode, u);
        }
        for (int64_t c = cols; c < ldq; ++c) q[r * ldq + c] = 0;
    }
}

/* cuda/src/quantization.cu:95-167 (kernel_transpose_quant):
   x[nrow, ncol] fp32 -> out[ncol, nrow] int8, half-even.  The reference does
   not clamp; with the tensor's own absmax scale nothing leaves [-127, 127],
   and outside that contract its float->int8 store is undefined, so the
   canonical form clamps. */
void orc_transpose_quant(const float *x, int64_t nrow, int64_t ncol, float scale,
                         int8_t *out) {
    const float r = rscale_of(scale);
    for (int64_t i = 0; i < nrow; ++i)
        for (int64_t j = 0; j < ncol; ++j)
            out[j * nrow + i] = quant_one(x[i * ncol + j], r, ORC_ROUND_RNE, 0.0f);
}

/* ------------------------------------------------------------------ GEMM -- */

/* cuda/src/epilogue.h:62-100 (Dequant): scale = sA*sB rounded once, then
   y = scale * float(acc); with a source operand y = source + that. */
static inline float dequant(int32_t acc, float s) {
    volatile float y = s * (float)acc;
    return y;
}

/* Integer kernel shared by the three GEMMs: C[m,n] = sum_k A[m,k] * B[n,k],
   both operands with the reduction index contiguous. */
static void igemm_nt(const int8_t *A, int64_t lda, const int8_t *B, int64_t ldb,
                     int32_t *C, int64_t ldc, int64_t M, int64_t N, int64_t K) {
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        const int8_t *a = A + m * lda;
        for (int64_t n = 0; n < N; ++n) {
            const int8_t *b = B + n * ldb;
            int64_t acc = 0;
            /* int32 partial sums over blocks short enough not to overflow
               (4096 * 127^2 < 2^31), widened to int64 between blocks */
            for (int64_t k0 = 0; k0 < K; k0 += 4096) {
                const int64_t k1 = k0 + 4096 < K ? k0 + 4096 : K;
                int32_t part = 0;
                for (int64_t k = k0; k < k1; ++k) part += (int32_t)a[k] * (int32_t)b[k];
                acc += part;
            }
            C[m * ldc + n] = narrow_i32(acc);
        }
    }
}

/* cuda/src/QGEMM_forward.cu:125-157 + QuantizedGemmKernel.h:373-578 +
   iterator.h:156-164 + epilogue.h:84-100,392,521.
   X[M,K] (row stride ldx) and W[N,K] (row stride ldw) are quantized with
   `mode` (the reference truncates), the int8 copies are stored to Xq[M,K] and
   Wq[N,K] (dense), acc = Xq . Wq^T in int32, Y = dequant(acc) (+ bias[n]).
   If scaleY is non-null it receives max|Y| / 127 over the stored outputs.
   acc_out (optional, [M,N] dense) receives the raw accumulators. */
void orc_qgemm_fwd(float *Y, int64_t ldy, const float *X, int64_t ldx, int8_t *Xq,
                   const float *W, int64_t ldw, int8_t *Wq, const float *bias,
                   float *scaleY, float scaleX, float scaleW, int64_t M, int64_t N,
                   int64_t K, int mode, int32_t *acc_out) {
    orc_quantize_rows(X, M, K, ldx, &scaleX, 0, Xq, K, mode, NULL, 0, 0);
    orc_quantize_rows(W, N, K, ldw, &scaleW, 0, Wq, K, mode, NULL, 0, 0);
    int32_t *acc = acc_out ? acc_out : (int32_t *)malloc(sizeof(int32_t) * (size_t)(M * N));
    igemm_nt(Xq, K, Wq, K, acc, N, M, N, K);
    volatile float s = scaleX * scaleW; /* epilogue.h:71 */
    float m = 0.0f;
    for (int64_t i = 0; i < M; ++i)
        for (int64_t j = 0; j < N; ++j) {
            float y = dequant(acc[i * N + j], s);
            if (bias) {
                volatile float yb = bias[j] + y; /* epilogue.h:98-99 */
                y = yb;
            }
            Y[i * ldy + j] = y;
            float a = fabsf(y);
            if (a > m) m = a;
        }
    if (scaleY) {
        volatile float sy = m / 127.0f; /* epilogue.h:392,521 */
        *scaleY = sy;
    }
    if (!acc_out) free(acc);
}

/* cuda/src/QGEMM_backward.cu:21-48: dX[M,K] = (s_dY*s_W) * (dYq[M,N] . Wq[N,K]). */
void orc_qgemm_bwd_dx(float *dX, int64_t lddx, const int8_t *dYq, int64_t lddy,
                      const int8_t *Wq, int64_t ldw, float s_dY, float s_W, int64_t M,
                      int64_t N, int64_t K) {
    volatile float s = s_dY * s_W;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m)
        for (int64_t k = 0; k < K; ++k) {
            int64_t acc = 0;
            for (int64_t n = 0; n < N; ++n)
                acc += (int32_t)dYq[m * lddy + n] * (int32_t)Wq[n * ldw + k];
            dX[m * lddx + k] = dequant(narrow_i32(acc), s);
        }
}

/* cuda/src/QGEMM_backward.cu:50-113: dW[N,K] = (s_dY*s_X) * (dYq^T[N,M] . Xq[M,K]).
   Split-K in the reference sums int32 partials, which is exact, so the slice
   count does not appear here. */
void orc_qgemm_bwd_dw(float *dW, int64_t lddw, const int8_t *dYq, int64_t lddy,
                      const int8_t *Xq, int64_t ldx, float s_dY, float s_X, int64_t M,
                      int64_t N, int64_t K) {
    volatile float s = s_dY * s_X;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        int64_t *acc = (int64_t *)calloc((size_t)K, sizeof(int64_t));
        for (int64_t m = 0; m < M; ++m) {
            const int32_t d = dYq[m * lddy + n];
            if (d == 0) continue;
            const int8_t *x = Xq + m * ldx;
            for (int64_t k = 0; k < K; ++k) acc[k] += d * (int32_t)x[k];
        }
        for (int64_t k = 0; k < K; ++k) dW[n * lddw + k] = dequant(narrow_i32(acc[k]), s);
        free(acc);
    }
}

/* cuda/src/Qgemm_impl.cu:6-125 (legacy QgemmNT/NN/TN): scale from min/max
   (= absmax), half-even quantize, int8 GEMM, out = float(acc) * (s0*s1).
   A is [m,k] (or [k,m] if trans_a), B is [k,n] (or [n,k] if trans_b). */
void orc_qgemm_legacy(float *C, const float *A, const float *B, int64_t m, int64_t n,
                      int64_t k, int trans_a, int trans_b) {
    const float sA = orc_absmax_scale(A, m * k), sB = orc_absmax_scale(B, n * k);
    int8_t *Aq = (int8_t *)malloc((size_t)(m * k)), *Bq = (int8_t *)malloc((size_t)(n * k));
    orc_quantize(A, m * k, sA, Aq, ORC_ROUND_RNE, NULL, 0, 0);
    orc_quantize(B, n * k, sB, Bq, ORC_ROUND_RNE, NULL, 0, 0);
    volatile float s = sA * sB;
    for (int64_t i = 0; i < m; ++i)
        for (int64_t j = 0; j < n; ++j) {
            int64_t acc = 0;
            for (int64_t p = 0; p < k; ++p) {
                const int32_t a = trans_a ? Aq[p * m + i] : Aq[i * k + p];
                const int32_t b = trans_b ? Bq[j * k + p] : Bq[p * n + j];
                acc += a * b;
            }
            volatile float y = (float)narrow_i32(acc) * s; /* Qgemm_impl.cu:102-104 */
            C[i * n + j] = y;
        }
    free(Aq);
    free(Bq);
}

/* ------------------------------------------------------------------ SpMM -- */

/* cuda/src/SPMM.cu:23-68 (cusp_SPMM_csr_impl): all-ones CSR times int8 dense,
   out[r,:] = s * sum_{p in row r} feat[indices[p], :].  Integer accumulate,
   one fp32 multiply (the reference accumulates the same integers in fp32,
   which is identical while |sum| < 2^24). */
void orc_spmm_csr_copy_u(float *out, const int64_t *indptr, const int64_t *indices,
                         const int8_t *feat, int64_t ldf, float scale, int64_t rows,
                         int64_t F) {
#pragma omp parallel
    {
        int64_t *acc = (int64_t *)malloc(sizeof(int64_t) * (size_t)(F > 0 ? F : 1));
#pragma omp for schedule(dynamic, 64)
        for (int64_t r = 0; r < rows; ++r) {
            for (int64_t f = 0; f < F; ++f) acc[f] = 0;
            for (int64_t p = indptr[r]; p < indptr[r + 1]; ++p) {
                const int8_t *u = feat + indices[p] * ldf;
                for (int64_t f = 0; f < F; ++f) acc[f] += u[f];
            }
            for (int64_t f = 0; f < F; ++f) {
                volatile float y = scale * (float)narrow_i32(acc[f]);
                out[r * F + f] = y;
            }
        }
        free(acc);
    }
}

/* cuda/src/SPMM.cu:70-130 (broadcast E, D == 1) and :132-194 (element-wise E,
   D == F) behind the dispatcher at cuda/src/cuda.cpp:147-157.
   feat[k, H, F] int8, evals[H, D, nnz] int8 in CSR slot order, or in edge-id
   order when edge_ids is given (then slot p reads evals[.., edge_ids[p]],
   the index_select of cuda/kernels.py:133-135 folded in).
   out[r,h,f] = s * sum_p evals[h, d(f), p] * feat[indices[p], h, f]. */
void orc_spmm_csr_u_mul_e(float *out, const int64_t *indptr, const int64_t *indices,
                          const int64_t *edge_ids, const int8_t *feat,
                          const int8_t *evals, float scale, int64_t rows, int64_t H,
                          int64_t F, int64_t D, int64_t nnz) {
    const int64_t HF = H * F;
#pragma omp parallel
    {
        int64_t *acc = (int64_t *)malloc(sizeof(int64_t) * (size_t)(HF > 0 ? HF : 1));
#pragma omp for schedule(dynamic, 64)
        for (int64_t r = 0; r < rows; ++r) {
            for (int64_t t = 0; t < HF; ++t) acc[t] = 0;
            for (int64_t p = indptr[r]; p < indptr[r + 1]; ++p) {
                const int8_t *u = feat + indices[p] * HF;
                const int64_t e = edge_ids ? edge_ids[p] : p;
                for (int64_t h = 0; h < H; ++h)
                    for (int64_t f = 0; f < F; ++f) {
                        const int64_t d = (D == 1) ? 0 : f;
                        acc[h * F + f] +=
                            (int32_t)evals[(h * D + d) * nnz + e] * (int32_t)u[h * F + f];
                    }
            }
            for (int64_t t = 0; t < HF; ++t) {
                volatile float y = scale * (float)narrow_i32(acc[t]);
                out[r * HF + t] = y;
            }
        }
        free(acc);
    }
}

/* cuda/src/SPMM.cu:259-303 (incidence_SPMM_impl): COO (node, edge) pairs with
   all-ones values, out[v,:] = s * sum_{i: node[i]==v} E[edge[i], :].  Pairs
   may come in any order here (the shipped kernel requires them sorted by
   node, as cuda/util.py:6-7 produces them). */
void orc_spmm_incidence(float *out, const int64_t *node, const int64_t *edge,
                        const int8_t *E, float scale, int64_t num_nodes, int64_t nnz,
                        int64_t F) {
    int64_t *acc = (int64_t *)calloc((size_t)(num_nodes * F + 1), sizeof(int64_t));
    for (int64_t i = 0; i < nnz; ++i) {
        const int8_t *e = E + edge[i] * F;
        int64_t *a = acc + node[i] * F;
        for (int64_t f = 0; f < F; ++f) a[f] += e[f];
    }
    for (int64_t t = 0; t < num_nodes * F; ++t) {
        volatile float y = scale * (float)narrow_i32(acc[t]);
        out[t] = y;
    }
    free(acc);
}

/* ----------------------------------------------------------------- SDDMM -- */

/* cuda/src/SDDMM.cu:8-47 (kernel_SDDMM_dot_int8): scale = sU*sV first (:16),
   out[e,h] = float(sum_d U[src,h,d]*V[dst,h,d]) * scale (:36); optional
   scaleOut = max|out| / 127 (:39,45). */
void orc_sddmm_dot(float *out, float *scaleOut, const int64_t *src, const int64_t *dst,
                   const int8_t *U, const int8_t *V, float sU, float sV, int64_t E,
                   int64_t H, int64_t D) {
    volatile float s = sU * sV;
    float m = 0.0f;
    for (int64_t e = 0; e < E; ++e) {
        const int8_t *u = U + src[e] * H * D, *v = V + dst[e] * H * D;
        for (int64_t h = 0; h < H; ++h) {
            int64_t acc = 0;
            for (int64_t d = 0; d < D; ++d) acc += (int32_t)u[h * D + d] * (int32_t)v[h * D + d];
            volatile float y = (float)narrow_i32(acc) * s;
            out[e * H + h] = y;
            float a = fabsf(y);
            if (a > m) m = a;
        }
    }
    if (scaleOut) {
        volatile float so = m / 127.0f;
        *scaleOut = so;
    }
}

/* cuda/src/SDDMM.cu:49-100 (kernel_SDDMM_int8<OP>):
   out[e,t] = OP(float(U[src,t])*sU, float(V[dst,t])*sV), three roundings,
   op: 0 add, 1 sub, 2 mul, 3 div. */
void orc_sddmm_ewise(int op, float *out, float *scaleOut, const int64_t *src,
                     const int64_t *dst, const int8_t *U, const int8_t *V, float sU,
                     float sV, int64_t E, int64_t T) {
    float m = 0.0f;
    for (int64_t e = 0; e < E; ++e) {
        const int8_t *u = U + src[e] * T, *v = V + dst[e] * T;
        for (int64_t t = 0; t < T; ++t) {
            volatile float a = (float)u[t] * sU;
            volatile float b = (float)v[t] * sV;
            volatile float y;
            switch (op) {
            case 0: y = a + b; break;
            case 1: y = a - b; break;
            case 2: y = a * b; break;
            default: y = a / b; break;
            }
            out[e * T + t] = y;
            float ab = fabsf(y);
            if (ab > m) m = ab;
        }
    }
    if (scaleOut) {
        volatile float so = m / 127.0f;
        *scaleOut = so;
    }
}

/* ---------------------------------------------------------- edge softmax -- */

/* DGL's edge_softmax(norm_by='dst') as called at evaluation/test_gat.py:146,
   preceded by LeakyReLU (test_gat.py:57,144) when slope != 1.  indptr/eids
   are the destination-major CSR (adj_csc) with its edge-id permutation; e and
   a are [E, H] in edge-id order.  Computed in double and rounded once, so the
   fp32 kernels are judged against it by tolerance. */
void orc_edge_softmax_fwd(float *a, const float *e, const int64_t *indptr,
                          const int64_t *eids, int64_t rows, int64_t H, float slope) {
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t h = 0; h < H; ++h) {
            double mx = -INFINITY, sum = 0.0;
            for (int64_t p = indptr[r]; p < indptr[r + 1]; ++p) {
                const int64_t id = eids ? eids[p] : p;
                double v = e[id * H + h];
                if (v < 0) v *= (double)slope;
                if (v > mx) mx = v;
            }
            for (int64_t p = indptr[r]; p < indptr[r + 1]; ++p) {
                const int64_t id = eids ? eids[p] : p;
                double v = e[id * H + h];
                if (v < 0) v *= (double)slope;
                sum += exp(v - mx);
            }
            for (int64_t p = indptr[r]; p < indptr[r + 1]; ++p) {
                const int64_t id = eids ? eids[p] : p;
                double v = e[id * H + h];
                if (v < 0) v *= (double)slope;
                a[id * H + h] = (float)(exp(v - mx) / sum);
            }
        }
}

/* Backward of the above: with z = leaky(e), a = softmax(z):
   dz = a * (da - sum_dst a*da), de = dz * (e > 0 ? 1 : slope). */
void orc_edge_softmax_bwd(float *de, const float *a, const float *da, const float *e,
                          const int64_t *indptr, const int64_t *eids, int64_t rows,
                          int64_t H, float slope) {
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t h = 0; h < H; ++h) {
            double dot = 0.0;
            for (int64_t p = indptr[r]; p < indptr[r + 1]; ++p) {
                const int64_t id = eids ? eids[p] : p;
                dot += (double)a[id * H + h] * (double)da[id * H + h];
            }
            for (int64_t p = indptr[r]; p < indptr[r + 1]; ++p) {
                const int64_t id = eids ? eids[p] : p;
                double g = (double)a[id * H + h] * ((double)da[id * H + h] - dot);
                if (!(e[id * H + h] > 0)) g *= (double)slope;
                de[id * H + h] = (float)g;
            }
        }
}

/* ------------------------------------------------------------ fused forms -- */
/* The layer glue of evaluation/test_gcn.py:86-94,123-137 and evaluation/test_gat.py:160-165
   (separate torch passes in the reference) folded into the primitives.  Every fused step
   performs the same fp32 operations, each rounded once, in the order the separate passes
   would: these restate that order. */

/* element of a gradient taken back through an activation whose output (or sign mask) is known:
   mode 0 (ReLU, mask fp32): x where mask > 0, else 0
   mode 1 (ELU,  mask fp32 = the activation's output): x where mask > 0, else x * (mask + 1)
   mode 2 (ReLU, mask = 16-bit words, bit c % 16 of word [r, c / 16]): x where the bit is set, else 0 */
static inline float masked_elem(float x, const void *mask, int64_t ldm, int mode, int64_t r, int64_t c) {
    if (!mask) return x;
    if (mode == 2) {
        const uint16_t w = ((const uint16_t *)mask)[r * ldm + (c >> 4)];
        return ((w >> (c & 15)) & 1u) ? x : 0.0f;
    }
    const float m = ((const float *)mask)[r * ldm + c];
    if (m > 0.0f) return x;
    if (mode == 0) return 0.0f;
    volatile float t = m + 1.0f;
    volatile float y = x * t;
    return y;
}

/* scale_out = max|x' * row_mul| / 127 over the masked elements x'; colsum_out[c] = sum_r x'[r, c]
   (not multiplied), accumulated in double here (the shipped kernel adds fp32 partials in a fixed
   order: compared with a tolerance). */
void orc_absmax_ex(const float *x, int64_t rows, int64_t cols, int64_t ldx, const float *row_mul,
                   const void *mask, int64_t ldm, int mask_mode, float *scale_out, double *colsum_out) {
    float m = 0.0f;
    if (colsum_out)
        for (int64_t c = 0; c < cols; ++c) colsum_out[c] = 0.0;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) {
            const float v = masked_elem(x[r * ldx + c], mask, ldm, mask_mode, r, c);
            if (colsum_out) colsum_out[c] += (double)v;
            volatile float t = row_mul ? v * row_mul[r] : v;
            const float a = fabsf(t);
            if (a > m) m = a;
        }
    volatile float s = m / 127.0f;
    *scale_out = s;
}

/* q[r, c] = quantize(x'[r, c] * row_mul[r]) with one scale (or one per row); q[r, cols..ldq) = 0.
   Noise / Philox index r * cols + c, as orc_quantize_rows. */
void orc_quantize_rows_ex(const float *x, int64_t rows, int64_t cols, int64_t ldx, const float *row_mul,
                          const void *mask, int64_t ldm, int mask_mode, const float *scales, int per_row,
                          int8_t *q, int64_t ldq, int mode, const float *noise, uint64_t seed,
                          uint64_t offset) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float rs = rscale_of(per_row ? scales[r] : scales[0]);
        for (int64_t c = 0; c < cols; ++c) {
            const float v = masked_elem(x[r * ldx + c], mask, ldm, mask_mode, r, c);
            volatile float t = row_mul ? v * row_mul[r] : v;
            float u = 0.0f;
            const int64_t lin = r * cols + c;
            if (mode == ORC_ROUND_STOCHASTIC)
                u = noise ? noise[lin] : orc_philox_uniform(seed, offset + (uint64_t)lin);
            q[r * ldq + c] = quant_one(t, rs, mode, u);
        }
        for (int64_t c = cols; c < ldq; ++c) q[r * ldq + c] = 0;
    }
}

/* Forward GEMM on operands that are already int8 (the cached-input form of cuda/QLinear.py's
   forward and the second of two chained layers): Y = (sA*sB) * float(A . B^T) (+ bias), optional
   scaleY = max|Y| / 127.  Epilogue as orc_qgemm_fwd (cuda/src/epilogue.h:62-100). */
void orc_qgemm_i8_nt(float *Y, int64_t ldy, const int8_t *A, int64_t lda, const int8_t *B, int64_t ldb,
                     const float *bias, float *scaleY, float sA, float sB, int64_t M, int64_t N,
                     int64_t K) {
    int32_t *acc = (int32_t *)malloc(sizeof(int32_t) * (size_t)(M * N > 0 ? M * N : 1));
    igemm_nt(A, lda, B, ldb, acc, N, M, N, K);
    volatile float s = sA * sB;
    float m = 0.0f;
    for (int64_t i = 0; i < M; ++i)
        for (int64_t j = 0; j < N; ++j) {
            float y = dequant(acc[i * N + j], s);
            if (bias) {
                volatile float yb = bias[j] + y;
                y = yb;
            }
            Y[i * ldy + j] = y;
            const float a = fabsf(y);
            if (a > m) m = a;
        }
    if (scaleY) {
        volatile float sy = m / 127.0f;
        *scaleY = sy;
    }
    free(acc);
}

/* gradX with the backward of a folded row multiplier and an optional accumulation into dX:
   y = (s_dY*s_W) * float(acc); y = y * row_scale[m]; dX = accumulate ? dX + y : y. */
void orc_qgemm_bwd_dx_ex(float *dX, int64_t lddx, const int8_t *dYq, int64_t lddy, const int8_t *Wq,
                         int64_t ldw, float s_dY, float s_W, const float *row_scale, int accumulate,
                         int64_t M, int64_t N, int64_t K) {
    volatile float s = s_dY * s_W;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m)
        for (int64_t k = 0; k < K; ++k) {
            int64_t acc = 0;
            for (int64_t n = 0; n < N; ++n)
                acc += (int32_t)dYq[m * lddy + n] * (int32_t)Wq[n * ldw + k];
            volatile float y = dequant(narrow_i32(acc), s);
            if (row_scale) y = y * row_scale[m];
            if (accumulate) y = dX[m * lddx + k] + y;
            dX[m * lddx + k] = y;
        }
}

/* copy_u aggregation with the epilogue of a GCN layer: y = s * float(sum); y = y * row_scale[r];
   y = y + bias[f]; act 1: max(y, 0); act 2: ELU (y > 0 ? y : exp(y) - 1, libm here, the hardware
   exponential in the shipped kernel: compared with a tolerance); sign_bits (optional, F % 16 == 0):
   bit f % 16 of word [r, f / 16] = (y > 0). */
void orc_spmm_csr_copy_u_ex(float *out, uint16_t *sign_bits, const int64_t *indptr,
                            const int64_t *indices, const int8_t *feat, int64_t ldf, float scale,
                            const float *row_scale, const float *bias, int act, int64_t rows, int64_t F) {
#pragma omp parallel
    {
        int64_t *acc = (int64_t *)malloc(sizeof(int64_t) * (size_t)(F > 0 ? F : 1));
#pragma omp for schedule(dynamic, 64)
        for (int64_t r = 0; r < rows; ++r) {
            for (int64_t f = 0; f < F; ++f) acc[f] = 0;
            for (int64_t p = indptr[r]; p < indptr[r + 1]; ++p) {
                const int8_t *u = feat + indices[p] * ldf;
                for (int64_t f = 0; f < F; ++f) acc[f] += u[f];
            }
            if (sign_bits)
                for (int64_t w = 0; w < F / 16; ++w) sign_bits[r * (F / 16) + w] = 0;
            for (int64_t f = 0; f < F; ++f) {
                volatile float y = scale * (float)narrow_i32(acc[f]);
                if (row_scale) y = y * row_scale[r];
                if (bias) y = y + bias[f];
                if (act == 1) y = y > 0.0f ? y : 0.0f;
                if (act == 2 && !(y > 0.0f)) y = expf(y) - 1.0f;
                out[r * F + f] = y;
                if (sign_bits && y > 0.0f) sign_bits[r * (F / 16) + (f >> 4)] |= (uint16_t)(1u << (f & 15));
            }
        }
        free(acc);
    }
}

/* u_mul_e aggregation with the epilogue of a GAT layer (evaluation/test_gat.py:160-165):
   y = (scale * scale2) * float(sum) with the product of the two scales rounded first; + bias[h, f]; act. */
void orc_spmm_csr_u_mul_e_ex(float *out, const int64_t *indptr, const int64_t *indices,
                             const int64_t *edge_ids, const int8_t *feat, const int8_t *evals,
                             int edge_major, float scale, const float *scale2, const float *bias, int act,
                             int64_t rows, int64_t H, int64_t F, int64_t D, int64_t nnz) {
    const int64_t HF = H * F;
    volatile float s = scale2 ? scale * scale2[0] : scale;
#pragma omp parallel
    {
        int64_t *acc = (int64_t *)malloc(sizeof(int64_t) * (size_t)(HF > 0 ? HF : 1));
#pragma omp for schedule(dynamic, 64)
        for (int64_t r = 0; r < rows; ++r) {
            for (int64_t t = 0; t < HF; ++t) acc[t] = 0;
            for (int64_t p = indptr[r]; p < indptr[r + 1]; ++p) {
                const int8_t *u = feat + indices[p] * HF;
                const int64_t e = edge_ids ? edge_ids[p] : p;
                for (int64_t h = 0; h < H; ++h)
                    for (int64_t f = 0; f < F; ++f) {
                        const int64_t d = (D == 1) ? 0 : f;
                        const int8_t ev = edge_major ? evals[(e * H + h) * D + d] : evals[(h * D + d) * nnz + e];
                        acc[h * F + f] += (int32_t)ev * (int32_t)u[h * F + f];
                    }
            }
            for (int64_t t = 0; t < HF; ++t) {
                volatile float y = s * (float)narrow_i32(acc[t]);
                if (bias) y = y + bias[t];
                if (act == 1) y = y > 0.0f ? y : 0.0f;
                if (act == 2 && !(y > 0.0f)) y = expf(y) - 1.0f;
                out[r * HF + t] = y;
            }
        }
        free(acc);
    }
}
