// int8 x int8 -> int32 GEMMs on the CDNA4 matrix cores (v_mfma_i32_16x16x64_i8)
// with the dequant (+bias) (+absmax) epilogue fused, for gfx950.
//
// Shapes here are tall and skinny (M ~ 2e5 rows, N and K <= a few hundred), so
// every GEMM streams one big operand from HBM exactly once and keeps the small
// one on chip:
//   * NT kernel (forward, gradX): a wavefront owns 32 rows of the tall operand
//     and loads them from global memory straight into MFMA fragment layout
//     (16 bytes per lane, a 4-deep register ring keeps several k-steps in
//     flight); the small operand is staged through LDS, shared by the
//     workgroup's four wavefronts, double-buffered, bank-swizzled.
//   * TN kernel (gradW): both operands are tall and reduction-strided.  Tiles
//     are staged through LDS in their natural layout and transposed in
//     registers (v_perm 4x4 byte blocks) on the way into the fragments; the
//     reduction over rows is split across workgroups, each writing an int32
//     slab of its own; a second kernel adds the slabs (exact, independent of
//     the split) and dequantizes.
#include "common.hpp"

namespace tango {

// ----------------------------------------------------------------- helpers
__device__ __forceinline__ i32x4 mfma_16x16x64(i32x4 a, i32x4 b, i32x4 c) {
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
}

// 16 bytes of one int8 row starting at p; `avail` = bytes that may be read
// (<= 0: none).  VEC is the widest aligned access the row layout allows.
template <int VEC>
__device__ __forceinline__ i32x4 load16(const int8_t* p, int64_t avail) {
    i32x4 v = {0, 0, 0, 0};
    if (avail <= 0) return v;
    if (VEC == 16) {
        v = *reinterpret_cast<const i32x4*>(p);  // caller guarantees 16 readable bytes
    } else if (VEC == 4) {
        const int* q = reinterpret_cast<const int*>(p);
        if (avail > 0) v.x = q[0];
        if (avail > 4) v.y = q[1];
        if (avail > 8) v.z = q[2];
        if (avail > 12) v.w = q[3];
    } else {
        uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int b = 0; b < 16; ++b)
            if (b < avail) w[b >> 2] |= static_cast<uint32_t>(static_cast<uint8_t>(p[b])) << (8 * (b & 3));
        v = i32x4{static_cast<int>(w[0]), static_cast<int>(w[1]), static_cast<int>(w[2]), static_cast<int>(w[3])};
    }
    return v;
}

struct NtParams {
    float* C;            // [M, N] fp32, row stride ldc
    const int8_t* A;     // [M, Kr] int8, row stride lda: the tall operand
    const int8_t* B;     // [N, Kp] int8 packed: 16-byte aligned rows of stride ldb, zero-filled to Kp
    const float* bias;   // [N] or null
    const float* row_scale;  // [M] or null: row m of the dequantized product is multiplied by it
    float* absmax_out;   // null, or receives max|C| / 127 (pre-zeroed)
    const float* sA;
    const float* sB;
    int64_t M, N, Kr;    // Kr = reduction length
    int64_t lda, ldb, ldc;
    int64_t a_row_bytes; // bytes that may be read from each row of A (>= Kr)
    int accumulate;      // nonzero: the product is added to what C holds (gradients of one tensor from several layers)
    int8_t* Cq;          // stationary form with an int8 epilogue: [M, N] int8, row stride ldcq
    int64_t ldcq;
    const float* q_scale;  // the scale Cq is rounded with
    int q_mode;          // TANGO_ROUND_RNE or TANGO_ROUND_TRUNC
    // stationary form, fp32 output: also max |C[m, n] * mask_mul[m]| / 127 over the elements whose sign bit is set
    // (bit n % 16 of word mask_bits[m * ldmask + n / 16]): the scale the consumer of a gradient needs when it takes
    // the gradient back through a ReLU and multiplies its rows (pre-zeroed; mask_mul may be null)
    const uint16_t* mask_bits;
    int64_t ldmask;
    const float* mask_mul;
    float* masked_absmax_out;
};

// Workgroup = 4 waves = 128 rows x (16 * NT) columns.  gridDim = (ceil(M/128), ceil(N/(16 NT))).
template <int NT, int VEC>
__global__ __launch_bounds__(256, 2) void gemm_nt_kernel(const NtParams p) {
    constexpr int PF = 4;                 // A fragments in flight (k-steps)
    constexpr int BROWS = NT * 16;        // rows of B per tile
    __shared__ i32x4 ldsB[2][BROWS * 4];  // [buffer][row][16-byte chunk], chunk index swizzled
    __shared__ __attribute__((aligned(16))) float bias_s[BROWS];  // this tile's bias, zero where there is none

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 4;    // k-chunk of the fragment this lane holds
    const int r16 = lane & 15;  // row (A) / column (B, C) within a 16x16 tile
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * 128 + wave * 32;
    const int64_t n0 = static_cast<int64_t>(blockIdx.y) * BROWS;
    const int ksteps = static_cast<int>((p.Kr + 63) >> 6);

    const int64_t ra0 = row0 + r16, ra1 = row0 + 16 + r16;
    const int8_t* pa0 = p.A + ra0 * p.lda + g * 16;
    const int8_t* pa1 = p.A + ra1 * p.lda + g * 16;
    const bool ok0 = ra0 < p.M, ok1 = ra1 < p.M;

    auto load_a = [&](i32x4* dst, int step) {
        const int64_t kc = static_cast<int64_t>(step) * 64 + g * 16;
        const int64_t avail = (step < ksteps && kc < p.Kr) ? (p.a_row_bytes - kc) : 0;
        dst[0] = load16<VEC>(pa0 + static_cast<int64_t>(step) * 64, ok0 ? avail : 0);
        dst[1] = load16<VEC>(pa1 + static_cast<int64_t>(step) * 64, ok1 ? avail : 0);
    };

    // B tile: BROWS rows x 4 chunks; thread handles chunks tid, tid + 256, ...
    constexpr int BCH = (BROWS * 4 + 255) / 256;
    auto load_b = [&](i32x4* dst, int step) {
#pragma unroll
        for (int c = 0; c < BCH; ++c) {
            const int idx = tid + c * 256;
            const int n = idx >> 2, kc = idx & 3;
            dst[c] = i32x4{0, 0, 0, 0};
            if (idx < BROWS * 4 && n0 + n < p.N && step < ksteps)
                dst[c] = *reinterpret_cast<const i32x4*>(p.B + (n0 + n) * p.ldb + static_cast<int64_t>(step) * 64 + kc * 16);
        }
    };
    auto store_b = [&](const i32x4* src, int buf) {
#pragma unroll
        for (int c = 0; c < BCH; ++c) {
            const int idx = tid + c * 256;
            const int n = idx >> 2, kc = idx & 3;
            if (idx < BROWS * 4) ldsB[buf][n * 4 + (kc ^ ((n >> 1) & 3))] = src[c];
        }
    };

    i32x4 acc[2][NT];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[i][j] = i32x4{0, 0, 0, 0};

    i32x4 a[PF][2];
#pragma unroll
    for (int s = 0; s < PF; ++s) load_a(a[s], s);
    i32x4 breg[BCH];
    load_b(breg, 0);
    for (int n = tid; n < BROWS; n += 256) bias_s[n] = (p.bias && n0 + n < p.N) ? p.bias[n0 + n] : 0.0f;
    store_b(breg, 0);
    __syncthreads();

    for (int t = 0; t < ksteps; t += PF) {
#pragma unroll
        for (int s = 0; s < PF; ++s) {
            const int step = t + s;
            if (step < ksteps) {  // uniform across the workgroup
                const int buf = step & 1;
                load_b(breg, step + 1);
#pragma unroll
                for (int j = 0; j < NT; ++j) {
                    const int n = j * 16 + r16;
                    const i32x4 b = ldsB[buf][n * 4 + (g ^ ((n >> 1) & 3))];
                    // operands swapped (C^T = B A^T): the lane then holds four CONSECUTIVE columns
                    // of one output row, which makes the epilogue's stores 16 bytes wide
                    acc[0][j] = mfma_16x16x64(b, a[s][0], acc[0][j]);
                    acc[1][j] = mfma_16x16x64(b, a[s][1], acc[1][j]);
                }
                load_a(a[s], step + PF);
                store_b(breg, buf ^ 1);
                __syncthreads();
            }
        }
    }

    // epilogue: lane holds C[row0 + 16 i + r16][n0 + 16 j + 4 g + v], v = 0..3
    const float s = p.sA[0] * p.sB[0];
    float m = 0.0f;
    const uintptr_t ca = reinterpret_cast<uintptr_t>(p.C);
    const int wide = ((ca & 15) == 0 && (p.ldc & 3) == 0) ? 4 : ((ca & 7) == 0 && (p.ldc & 1) == 0) ? 2 : 1;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int64_t row = row0 + i * 16 + r16;
        if (row < p.M) {
            float* crow = p.C + row * p.ldc;
            const float rsc = p.row_scale ? p.row_scale[row] : 1.0f;
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                const int64_t col = n0 + j * 16 + g * 4;
                float y[4];
                const f32x4 bv = *reinterpret_cast<const f32x4*>(bias_s + j * 16 + g * 4);
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    y[v] = s * static_cast<float>(acc[i][j][v]);
                    if (p.row_scale) y[v] = y[v] * rsc;
                    if (p.bias) y[v] = bv[v] + y[v];
                    if (col + v < p.N) m = fmaxf(m, fabsf(y[v]));
                }
                if (p.accumulate) {  // uniform; the absmax above is of the product alone and is not asked for with it
                    if (col + 4 <= p.N && wide == 4) {
                        const f32x4 o = *reinterpret_cast<const f32x4*>(crow + col);
                        *reinterpret_cast<f32x4*>(crow + col) = f32x4{o[0] + y[0], o[1] + y[1], o[2] + y[2], o[3] + y[3]};
                    } else {
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            if (col + v < p.N) crow[col + v] += y[v];
                    }
                    continue;
                }
                if (col + 4 <= p.N && wide == 4) {
                    *reinterpret_cast<f32x4*>(crow + col) = f32x4{y[0], y[1], y[2], y[3]};
                } else if (col + 4 <= p.N && wide == 2) {
                    typedef float f32x2 __attribute__((ext_vector_type(2)));
                    // plain stores: these half-aligned pieces rely on L2 to merge them into full lines
                    *reinterpret_cast<f32x2*>(crow + col) = f32x2{y[0], y[1]};
                    *reinterpret_cast<f32x2*>(crow + col + 2) = f32x2{y[2], y[3]};
                } else {
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        if (col + v < p.N) crow[col + v] = y[v];
                }
            }
        }
    }
    if (p.absmax_out) block_absmax_to_global(m / 127.0f, p.absmax_out);
}

// NT kernel with the small operand stationary in LDS, for reductions of at most 256 (four k-steps).
// A persistent workgroup of WAVES waves first copies its 16 * NT rows of the packed B into LDS (in fragment
// order: the 1 KB a wave reads for one MFMA is contiguous, lane after lane) and
// then never synchronises again: the 16-row tiles of A are dealt round-robin over all waves of the
// launch, a wave loads the whole 16 x K tile as its A fragments (and the next tile's while it works on
// this one), reads the B fragments from LDS, and stores 16 rows x 16 NT columns.  The kernels above pay
// one L2 round trip per k-step (several microseconds under load) in every workgroup; here the only
// global loads are the A tiles, requested one tile ahead, so loads, MFMAs and the output stores of the
// sixteen waves of a CU overlap.
// EPI 0: the tile goes to C as fp32.  EPI 1: nothing is stored, only max|C| / 127 is found.  EPI 2: the tile
// is rounded to int8 with the scale q_scale and goes to Cq (the fp32 values are the same in all three, so
// 1 then 2 store exactly what a quantize pass over the fp32 output of 0 would).
template <int NT, int VEC, int WAVES, int EPI = 0, int PASSES = 1>
__global__ __launch_bounds__(64 * WAVES) void gemm_nts_kernel(const NtParams p, int ntiles) {
    constexpr bool F32OUT = EPI == 0 || EPI == 3;  // EPI 3: EPI 0 that also finds the masked maximum
    // B in fragment order: block (j, st) of 1 KB holds, at 16 lane bytes, the 16 bytes lane `lane` feeds the MFMA
    // of column tile j at k-step st, so a fragment read is one linear 1 KB sweep (no bank conflicts by construction)
    extern __shared__ __attribute__((aligned(16))) int8_t b_lds[];  // [PASSES NT][ksteps][64 lanes][16]
    constexpr int KS = 4;
    constexpr int TT = NT * PASSES;  // column tiles of the block: a wave walks them NT at a time (PASSES rounds over
                                     // one A tile held in registers), so that the accumulators stay at 4 NT registers
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 4, r16 = lane & 15;
    const int64_t n0 = static_cast<int64_t>(blockIdx.y) * (16 * TT);
    const int ksteps = static_cast<int>((p.Kr + 63) >> 6);  // <= KS (host)
    // Which column of the block the LDS row n = 16 j + 4 g + v (column 4 g + v of MFMA tile j) stands for.  A lane
    // holds columns 4 g .. 4 g + 3 of every tile: four output bytes in the int8 epilogue.  There the tiles of a
    // group of four are interleaved, so that a lane's four tiles cover sixteen adjacent columns (one 16-byte
    // store, 64 contiguous bytes per row from the four lanes) instead of four 4-byte pieces.
    constexpr bool PERM = EPI == 2 && NT % 4 == 0;
    auto lds_row_column = [](int n) {
        if (!PERM) return n;
        const int j = n >> 4, gq = (n >> 2) & 3, v = n & 3;
        return 64 * (j >> 2) + 16 * gq + 4 * (j & 3) + v;
    };
    {
        const int kchunks = ksteps * 4;  // 16-byte chunks of a packed row that hold data or its zero fill
        for (int idx = tid; idx < 16 * TT * kchunks; idx += 64 * WAVES) {
            const int n = idx / kchunks, c = idx - n * kchunks;
            i32x4 v{0, 0, 0, 0};
            const int64_t nb = n0 + lds_row_column(n);
            if (nb < p.N) v = *reinterpret_cast<const i32x4*>(p.B + nb * p.ldb + c * 16);
            // row n = 16 j + r16, chunk c = 4 st + g  ->  block (j, st), lane 16 g + r16
            *reinterpret_cast<i32x4*>(b_lds + ((((n >> 4) * ksteps + (c >> 2)) << 6) + ((c & 3) << 4) + (n & 15)) * 16) = v;
        }
    }
    float* bias_lds = reinterpret_cast<float*>(b_lds + TT * ksteps * 1024);  // [16 TT], zero where there is none
    for (int n = tid; n < 16 * TT; n += 64 * WAVES) {
        const int64_t nb = n0 + lds_row_column(n);
        bias_lds[n] = (p.bias && nb < p.N) ? p.bias[nb] : 0.0f;
    }
    __syncthreads();

    const float s = p.sA[0] * p.sB[0];
    const uintptr_t ca = reinterpret_cast<uintptr_t>(p.C);
    const int wide = ((ca & 15) == 0 && (p.ldc & 3) == 0) ? 4 : ((ca & 7) == 0 && (p.ldc & 1) == 0) ? 2 : 1;
    const float qr = EPI == 2 ? rscale_of(p.q_scale[0]) : 0.0f;
    const bool qwide = EPI == 2 && (reinterpret_cast<uintptr_t>(p.Cq) & 3) == 0 && (p.ldcq & 3) == 0;
    const bool q16 = EPI == 2 && (reinterpret_cast<uintptr_t>(p.Cq) & 15) == 0 && (p.ldcq & 15) == 0;
    float m = 0.0f, m2 = 0.0f;
    // the masked maximum: only with the plain fp32 epilogue over whole blocks of NT tiles (checked by the host)
    constexpr bool want_masked = EPI == 3 && PASSES == 1 && NT % 2 == 0;
    constexpr int BW = want_masked ? NT / 2 : 1;
    auto load_tile = [&](i32x4* a, float& rsc, float& mmul, uint32_t* bw, int t) {
        const int64_t row = static_cast<int64_t>(t) * 16 + r16;
        const bool ok = t < ntiles && row < p.M;
        rsc = (p.row_scale && ok) ? p.row_scale[row] : 1.0f;  // requested with the tile, not in the epilogue
        if (want_masked) {  // uniform: the row's sign words of this block's columns, two per register
            const uint32_t* w = reinterpret_cast<const uint32_t*>(p.mask_bits + (ok ? row : 0) * p.ldmask + (n0 >> 4));
#pragma unroll
            for (int j = 0; j < BW; ++j) bw[j] = w[j];
            mmul = (p.mask_mul && ok) ? p.mask_mul[row] : 1.0f;
        }
        const int8_t* pa = p.A + (ok ? row : 0) * p.lda + g * 16;
#pragma unroll
        for (int st = 0; st < KS; ++st) {
            const int64_t kc = static_cast<int64_t>(st) * 64 + g * 16;
            const int64_t avail = (ok && st < ksteps && kc < p.Kr) ? p.a_row_bytes - kc : 0;
            a[st] = load16<VEC>(pa + st * 64, avail);
        }
    };
    const int stride = static_cast<int>(gridDim.x) * WAVES;
    i32x4 cur[KS], nxt[KS];
    float rsc, rsc_nxt, mmul = 1.0f, mmul_nxt = 1.0f;
    uint32_t bw[BW], bw_nxt[BW];
    int t = static_cast<int>(blockIdx.x) * WAVES + wave;
    load_tile(cur, rsc, mmul, bw, t);
    // fp32 output with nothing but the dequantization (and the optional row scale) in the epilogue: the common case
    // gets a loop without a branch per tile (the general loop below tests six uniform conditions per column tile)
    const bool plain = F32OUT && !p.bias && !p.accumulate && wide == 4;
    const bool want_max = EPI == 1 || (F32OUT && p.absmax_out != nullptr);
    // columns of this block, as a 32-bit count: the bounds tests of the epilogue are 32-bit compares
    const int ncols = static_cast<int>(p.N - n0 < 16 * TT ? p.N - n0 : 16 * TT);
    // columns that may be written: a row's padding up to its pitch takes the zeros of the zero-filled rows of B
    // (never past the next multiple of 16 columns: what lies beyond may belong to the caller)
    const int64_t wlim = ((p.N + 15) & ~static_cast<int64_t>(15)) < p.ldc ? ((p.N + 15) & ~static_cast<int64_t>(15)) : p.ldc;
    const int wcols = F32OUT ? static_cast<int>(wlim - n0 < 16 * TT ? wlim - n0 : 16 * TT) : ncols;
    for (; t < ntiles; t += stride) {
        load_tile(nxt, rsc_nxt, mmul_nxt, bw_nxt, t + stride);
        const int64_t row = static_cast<int64_t>(t) * 16 + r16;
        float* crow = p.C + row * p.ldc + n0;
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
        i32x4 acc[NT];
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[j] = i32x4{0, 0, 0, 0};
#pragma unroll
        for (int st = 0; st < KS; ++st) {
            if (st < ksteps) {
#pragma unroll
                for (int j = 0; j < NT; ++j) {
                    const i32x4 b = *reinterpret_cast<const i32x4*>(b_lds + ((((ps * NT + j) * ksteps + st) << 6) + lane) * 16);
                    acc[j] = mfma_16x16x64(b, cur[st], acc[j]);  // operands swapped, see gemm_nt_kernel
                }
            }
        }
        // lane holds C[16 t + r16][n0 + 16 (ps NT + j) + 4 g + v] (PERM: the column lds_row_column gives)
        if (row < p.M) {
            const int c0 = ps * 16 * NT;  // first column of this pass inside the block
            if (plain && c0 + 16 * NT <= wcols) {
                f32x4* cp = reinterpret_cast<f32x4*>(crow + c0 + 4 * g);
                if (want_masked) {
#pragma unroll
                    for (int j = 0; j < NT; ++j) {
                        const f32x4 y{(s * static_cast<float>(acc[j][0])) * rsc, (s * static_cast<float>(acc[j][1])) * rsc,
                                      (s * static_cast<float>(acc[j][2])) * rsc, (s * static_cast<float>(acc[j][3])) * rsc};
                        const uint32_t keep = bw[(j >> 1) % BW] >> (16 * (j & 1) + 4 * g);  // bits of columns 16 j + 4 g ..
#pragma unroll
                        for (int v = 0; v < 4; ++v) {
                            const float e = ((keep >> v) & 1u) ? y[v] : 0.0f;
                            m2 = fmaxf(m2, fabsf(p.mask_mul ? e * mmul : e));
                        }
                        if (want_max) m = fmaxf(fmaxf(m, fmaxf(fabsf(y[0]), fabsf(y[1]))), fmaxf(fabsf(y[2]), fabsf(y[3])));
                        cp[4 * j] = y;
                    }
                } else if (want_max) {
#pragma unroll
                    for (int j = 0; j < NT; ++j) {
                        const f32x4 y{(s * static_cast<float>(acc[j][0])) * rsc, (s * static_cast<float>(acc[j][1])) * rsc,
                                      (s * static_cast<float>(acc[j][2])) * rsc, (s * static_cast<float>(acc[j][3])) * rsc};
                        m = fmaxf(fmaxf(m, fmaxf(fabsf(y[0]), fabsf(y[1]))), fmaxf(fabsf(y[2]), fabsf(y[3])));
                        cp[4 * j] = y;
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < NT; ++j)
                        cp[4 * j] = f32x4{(s * static_cast<float>(acc[j][0])) * rsc, (s * static_cast<float>(acc[j][1])) * rsc,
                                          (s * static_cast<float>(acc[j][2])) * rsc, (s * static_cast<float>(acc[j][3])) * rsc};
                }
                continue;
            }
            uint32_t qw[4];
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                const int cl = c0 + (PERM ? 64 * (j >> 2) + 16 * g + 4 * (j & 3) : j * 16 + g * 4);  // column inside the block
                const int col = cl;  // relative to crow / qrow, which start at the block's first column
                const bool full = cl + 4 <= ncols;
                float y[4];
                const f32x4 bv = *reinterpret_cast<const f32x4*>(bias_lds + c0 + j * 16 + g * 4);
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    y[v] = s * static_cast<float>(acc[j][v]);
                    if (p.row_scale) y[v] = y[v] * rsc;
                    if (p.bias) y[v] = bv[v] + y[v];
                }
                if (want_max) {  // uniform
                    if (full) {
                        m = fmaxf(fmaxf(m, fmaxf(fabsf(y[0]), fabsf(y[1]))), fmaxf(fabsf(y[2]), fabsf(y[3])));
                    } else {
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            if (cl + v < ncols) m = fmaxf(m, fabsf(y[v]));
                    }
                }
                if (EPI == 1) continue;
                if (EPI == 2) {
                    int q[4];
                    if (p.q_mode == TANGO_ROUND_TRUNC) {  // uniform
#pragma unroll
                        for (int v = 0; v < 4; ++v) q[v] = quant_one<TANGO_ROUND_TRUNC>(y[v], qr, 0.0f);
                    } else {
#pragma unroll
                        for (int v = 0; v < 4; ++v) q[v] = quant_one<TANGO_ROUND_RNE>(y[v], qr, 0.0f);
                    }
                    int8_t* qrow = p.Cq + row * p.ldcq + n0;
                    if (PERM) {
                        qw[j & 3] = pack4(q[0], q[1], q[2], q[3]);
                        if ((j & 3) != 3) continue;
                        const int col0 = col - 12;  // 64 (j / 4) + 16 g
                        if (col0 + 16 <= ncols && q16) {
                            typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
                            *reinterpret_cast<u32x4*>(qrow + col0) = u32x4{qw[0], qw[1], qw[2], qw[3]};
                        } else {
#pragma unroll
                            for (int b = 0; b < 16; ++b)
                                if (col0 + b < ncols) qrow[col0 + b] = static_cast<int8_t>(qw[b >> 2] >> (8 * (b & 3)));
                        }
                        continue;
                    }
                    if (full && qwide) {
                        *reinterpret_cast<uint32_t*>(qrow + col) = pack4(q[0], q[1], q[2], q[3]);
                    } else {
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            if (cl + v < ncols) qrow[col + v] = static_cast<int8_t>(q[v]);
                    }
                    continue;
                }
                if (p.accumulate) {  // uniform
                    if (full && wide == 4) {
                        const f32x4 o = *reinterpret_cast<const f32x4*>(crow + col);
                        *reinterpret_cast<f32x4*>(crow + col) = f32x4{o[0] + y[0], o[1] + y[1], o[2] + y[2], o[3] + y[3]};
                    } else {
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            if (cl + v < ncols) crow[col + v] += y[v];
                    }
                    continue;
                }
                if (full && wide == 4) {
                    *reinterpret_cast<f32x4*>(crow + col) = f32x4{y[0], y[1], y[2], y[3]};
                } else if (full && wide == 2) {
                    typedef float f32x2 __attribute__((ext_vector_type(2)));
                    *reinterpret_cast<f32x2*>(crow + col) = f32x2{y[0], y[1]};
                    *reinterpret_cast<f32x2*>(crow + col + 2) = f32x2{y[2], y[3]};
                } else {
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        if (cl + v < ncols) crow[col + v] = y[v];
                }
            }
        }
        }  // passes
#pragma unroll
        for (int st = 0; st < KS; ++st) cur[st] = nxt[st];
        rsc = rsc_nxt;
        if (want_masked) {
            mmul = mmul_nxt;
#pragma unroll
            for (int j = 0; j < BW; ++j) bw[j] = bw_nxt[j];
        }
    }
    if (p.absmax_out) block_absmax_to_global(m / 127.0f, p.absmax_out);
    if (want_masked) {
        __syncthreads();  // the reduction above and this one share their LDS words
        block_absmax_to_global(m2 / 127.0f, p.masked_absmax_out);
    }
}

// NT kernel with the small operand stationary in registers, for wide fp32 outputs (257 to 960 columns) and
// reductions of at most 64 KS.  The workgroup's waves share one 16-row tile of A at a time and split its output
// row into pieces of 64 columns: wave w holds the B fragments of column tiles 4 w .. 4 w + 3 for the whole launch
// (16 KS registers), reads the A tile from LDS, runs its 4 KS MFMAs and stores a 16 x 64 piece.  A tile's rows
// leave the compute unit together, so the launch writes one compact window that moves through C front to back;
// with a wave per tile (gemm_nts_kernel) some three thousand separate rows of C are open at once, and a
// store-only kernel of that shape sustains 5.0 TB/s on outputs beyond the Infinity Cache against 6.0 TB/s for
// this one.
// The last wave of the workgroup only fetches: it reads the next tiles of A in whole rows (a quarter-wave per
// 256-byte row; loading fragments directly costs a cache line look-up per lane, which a dozen waves asking for
// the same tile cannot afford) and writes them to a two-slot LDS ring, rotated per row so that the fragment
// reads of a quarter-wave (one 16-byte chunk of sixteen rows) fall on sixteen different bank groups.  Memory
// operations of a wave complete in order; because the fetching wave stores nothing and the storing waves load
// nothing, no wave ever waits for a store.  One barrier per tile hands a slot over.
// Epilogue: dequantization, the optional row scale and absmax only; C must be 16-byte aligned with a pitch that
// is a multiple of 4 floats; rows of A must be readable in aligned 16-byte pieces.
template <int KS>
__global__ __launch_bounds__(1024) void gemm_ntr_kernel(const NtParams p, int ntiles) {
    constexpr int CT = 4;
    constexpr int CH = 4 * KS;            // 16-byte chunks of a tile row
    constexpr int SLOT = 16 * CH * 16 + 64;  // bytes of a ring slot: the tile, then sixteen row scales
    __shared__ __attribute__((aligned(16))) int8_t ring[2 * SLOT];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
    const int consumers = static_cast<int>(blockDim.x >> 6) - 1;
    const int g = lane >> 4, r16 = lane & 15;
    const int stride = static_cast<int>(gridDim.x);
    const int t0 = static_cast<int>(blockIdx.x);
    const int rounds = t0 < ntiles ? (ntiles - t0 + stride - 1) / stride : 0;  // the same for every wave
    // chunk c of row r lives at 16-byte position CH r + (c + r / (16 / CH)) mod CH of its slot
    auto position = [](int r, int c) { return CH * r + ((c + r / (16 / CH)) & (CH - 1)); };
    auto hand_over = [] { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    if (wave == consumers) {  // the fetching wave
        constexpr int NI = CH / 4;  // 16-byte loads per lane and tile: 64 lanes x NI chunks = 16 rows x CH chunks
        int8_t* dst[NI];
        int64_t off[NI];  // byte offset of the lane's chunk inside a row of A; negative: not readable
        int rr[NI];
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int pos = 64 * i + lane;  // lanes cover positions in order: a run of CH lanes is one whole row
            const int r = pos / CH;
            const int c = ((pos & (CH - 1)) - r / (16 / CH)) & (CH - 1);
            rr[i] = r;
            off[i] = 16 * c < p.a_row_bytes ? 16 * c : -1;
            dst[i] = ring + pos * 16;
        }
        auto fetch = [&](i32x4* v, float& rs, int t) {
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                int64_t row = static_cast<int64_t>(t) * 16 + rr[i];
                if (row >= p.M) row = p.M - 1;  // rows past the end (last tile) are computed and not stored
                v[i] = i32x4{0, 0, 0, 0};
                if (off[i] >= 0) v[i] = *reinterpret_cast<const i32x4*>(p.A + row * p.lda + off[i]);
            }
            int64_t row = static_cast<int64_t>(t) * 16 + r16;
            if (row >= p.M) row = p.M - 1;
            rs = p.row_scale ? p.row_scale[row] : 1.0f;
        };
        auto put = [&](const i32x4* v, float rs, int slot) {
#pragma unroll
            for (int i = 0; i < NI; ++i) *reinterpret_cast<i32x4*>(dst[i] + slot * SLOT) = v[i];
            if (lane < 16) *reinterpret_cast<float*>(ring + slot * SLOT + 16 * CH * 16 + 4 * lane) = rs;
        };
        // tiles are requested four rounds ahead (one round lasts less than a trip to memory); the four register
        // sets take turns by unrolling, so that no set is copied while its load is in flight
        i32x4 v[4][NI];
        float rs[4] = {1.0f, 1.0f, 1.0f, 1.0f};
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (u < rounds) fetch(v[u], rs[u], t0 + u * stride);
        if (rounds > 0) put(v[0], rs[0], 0);
        if (4 < rounds) fetch(v[0], rs[0], t0 + 4 * stride);
        hand_over();  // slot 0 holds the first tile
        // round k: the tile of round k + 1 goes to slot (k + 1) % 2 while the other waves read slot k % 2
        for (int kb = 0; kb < rounds; kb += 4) {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int k = kb + u;
                if (k >= rounds) break;
                const int set = (u + 1) & 3;
                if (k + 1 < rounds) put(v[set], rs[set], (k + 1) & 1);
                if (k + 5 < rounds) fetch(v[set], rs[set], t0 + (k + 5) * stride);
                hand_over();
            }
        }
        if (p.absmax_out) block_absmax_to_global(0.0f, p.absmax_out);
        return;
    }

    i32x4 b[CT][KS];
#pragma unroll
    for (int j = 0; j < CT; ++j) {
        const int64_t n = 16 * static_cast<int64_t>(CT * wave + j) + r16;
#pragma unroll
        for (int st = 0; st < KS; ++st) {
            // zero rows past the last column, zero fill of the packed rows past the reduction length: whatever
            // the ring holds at those places does not count
            b[j][st] = i32x4{0, 0, 0, 0};
            if (n < p.N && st * 64 < p.Kr) b[j][st] = *reinterpret_cast<const i32x4*>(p.B + n * p.ldb + st * 64 + g * 16);
        }
    }
    const float s = p.sA[0] * p.sB[0];
    const bool want_max = p.absmax_out != nullptr;
    const int col0 = 64 * wave + 4 * g;  // first of the lane's four columns in tile j = 0
    // columns that may be written: a row's padding, up to the next multiple of 16 columns, takes the zeros of the
    // zero-filled rows of B
    const int n16c = static_cast<int>((p.N + 15) >> 4) * 16;
    const int wcols = p.ldc < n16c ? static_cast<int>(p.ldc) : n16c;
    int frag[KS];  // byte offset of the lane's fragment of k-step st inside a slot
#pragma unroll
    for (int st = 0; st < KS; ++st) frag[st] = position(r16, 4 * st + g) * 16;
    float m = 0.0f;
    hand_over();
    for (int k = 0; k < rounds; ++k) {
        const int8_t* slot = ring + (k & 1) * SLOT;
        i32x4 a[KS];
#pragma unroll
        for (int st = 0; st < KS; ++st) a[st] = *reinterpret_cast<const i32x4*>(slot + frag[st]);
        const float rsc = *reinterpret_cast<const float*>(slot + 16 * CH * 16 + 4 * r16);
        i32x4 acc[CT];
#pragma unroll
        for (int j = 0; j < CT; ++j) acc[j] = i32x4{0, 0, 0, 0};
#pragma unroll
        for (int st = 0; st < KS; ++st)
#pragma unroll
            for (int j = 0; j < CT; ++j)
                acc[j] = mfma_16x16x64(b[j][st], a[st], acc[j]);  // operands swapped, see gemm_nt_kernel
        const int64_t row = static_cast<int64_t>(t0 + k * stride) * 16 + r16;
        if (row < p.M) {
            float* crow = p.C + row * p.ldc + col0;
#pragma unroll
            for (int j = 0; j < CT; ++j) {
                if (col0 + 16 * j + 4 <= wcols) {
                    const f32x4 y{(s * static_cast<float>(acc[j][0])) * rsc, (s * static_cast<float>(acc[j][1])) * rsc,
                                  (s * static_cast<float>(acc[j][2])) * rsc, (s * static_cast<float>(acc[j][3])) * rsc};
                    if (want_max) m = fmaxf(fmaxf(m, fmaxf(fabsf(y[0]), fabsf(y[1]))), fmaxf(fabsf(y[2]), fabsf(y[3])));
                    *reinterpret_cast<f32x4*>(crow + 16 * j) = y;
                }
            }
        }
        hand_over();  // the slot just read may be refilled, the other one is complete
    }
    if (p.absmax_out) block_absmax_to_global(m / 127.0f, p.absmax_out);
}

// ------------------------------------ forward GEMM with the quantize fused in
// Workgroup = 4 waves = 64 rows of X.  Phase A: the waves stream their rows of the
// fp32 X from HBM (each lane 4 consecutive floats per step, a wavefront 1 KiB of one
// row), quantize in registers and write the int8 bytes twice: to Xq (the cache the
// backward pass reads) and to an LDS copy of the whole 64 x K block.  Phase B: every
// wave takes a quarter of the output columns, reads A fragments from that LDS block
// and B fragments straight from the packed small operand (L2-resident), and runs the
// MFMA k-loop without any further barrier.  X is read once, Xq written once, Y once.
struct FqParams {
    float* C;
    const float* X;
    int8_t* Xq;
    const int8_t* B;      // packed [N, Kp]
    const float* bias;
    const float* x_row_mul;  // optional per-row multiplier applied before quantization
    float* absmax_out;
    const float* sA;
    const float* sB;
    int64_t M, N, K;
    int64_t ldx, ldxq, ldb, ldc;
    int kp;               // K rounded up to 64
    int pitch;            // bytes between rows of the LDS block (fq_pitch)
    int b_frag;           // B is in fragment order (see quantize_pack_w_kernel), rows zero-filled to a multiple of 16
};

// TPW = 16-column tiles per wave (the workgroup covers 64 * TPW columns), XV = floats per load,
// RT = 16-row tiles per workgroup (BM = 16 * RT rows), IT = 256-column chunks of a row a lane
// loads from (kp <= 256 IT): sizes the prefetch registers.
template <int TPW, int XV, int MODE, int RT, int IT>
__global__ __launch_bounds__(256, 2) void gemm_fq_kernel(const FqParams p) {
    extern __shared__ __attribute__((aligned(16))) int8_t a_lds[];  // [BM][pitch] + 64, then 64 TPW floats of bias
    constexpr int BM = 16 * RT;
    const int pitch = p.pitch;
    float* bias_lds = reinterpret_cast<float*>(a_lds + BM * pitch + 64);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t row_base = static_cast<int64_t>(blockIdx.x) * BM;
    const float rs = rscale_of(p.sA[0]);
    const bool store_q = blockIdx.y == 0;
    if (threadIdx.x < 64 * TPW) {  // this workgroup's slice of the bias, zero where there is none
        const int64_t n = static_cast<int64_t>(blockIdx.y) * (64 * TPW) + threadIdx.x;
        bias_lds[threadIdx.x] = (p.bias && n < p.N) ? p.bias[n] : 0.0f;
    }

    // ---- phase A: rows wave, wave + 4, ... ; lane owns columns 4 * (lane + 64 it) .. + 3
    const float* __restrict__ Xp = p.X;
    int8_t* __restrict__ Xqp = p.Xq;
    const int iters = (p.kp + 255) >> 8;  // <= IT (1, 2 or 3 by the host: kp <= 768)
    auto fetch = [&](float (*f)[IT][4], int rr) {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int64_t row = row_base + wave + 4 * (rr + b);
            const float* xr = Xp + row * p.ldx;
#pragma unroll
            for (int it = 0; it < IT; ++it) {
                const int64_t c0 = (static_cast<int64_t>(lane) + 64 * it) << 2;
                f[b][it][0] = f[b][it][1] = f[b][it][2] = f[b][it][3] = 0.0f;
                if (it < iters && row < p.M && c0 < p.K) {
                    if (XV == 4 && c0 + 4 <= p.K) {
                        const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(xr + c0));
                        f[b][it][0] = v.x; f[b][it][1] = v.y; f[b][it][2] = v.z; f[b][it][3] = v.w;
                    } else if (XV == 2 && c0 + 4 <= p.K) {
                        typedef float f32x2 __attribute__((ext_vector_type(2)));
                        const f32x2 v0 = __builtin_nontemporal_load(reinterpret_cast<const f32x2*>(xr + c0));
                        const f32x2 v1 = __builtin_nontemporal_load(reinterpret_cast<const f32x2*>(xr + c0 + 2));
                        f[b][it][0] = v0.x; f[b][it][1] = v0.y; f[b][it][2] = v1.x; f[b][it][3] = v1.y;
                    } else {
#pragma unroll
                        for (int k = 0; k < 4; ++k)
                            if (c0 + k < p.K) f[b][it][k] = xr[c0 + k];
                    }
                }
            }
        }
    };
    auto emit = [&](float (*f)[IT][4], int rr) {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int lr = wave + 4 * (rr + b);
            const int64_t row = row_base + lr;
            const float rm = (p.x_row_mul && row < p.M) ? p.x_row_mul[row] : 1.0f;
#pragma unroll
            for (int it = 0; it < IT; ++it) {
                const int64_t c0 = (static_cast<int64_t>(lane) + 64 * it) << 2;
                if (it < iters && c0 < p.kp) {
                    float x0 = f[b][it][0], x1 = f[b][it][1], x2 = f[b][it][2], x3 = f[b][it][3];
                    if (p.x_row_mul) { x0 = x0 * rm; x1 = x1 * rm; x2 = x2 * rm; x3 = x3 * rm; }
                    const uint32_t q = pack4(quant_one<MODE>(x0, rs, 0.f), quant_one<MODE>(x1, rs, 0.f),
                                             quant_one<MODE>(x2, rs, 0.f), quant_one<MODE>(x3, rs, 0.f));
                    if (c0 < pitch) *reinterpret_cast<uint32_t*>(a_lds + lr * pitch + c0) = q;
                    if (store_q && row < p.M && c0 < p.ldxq)
                        *reinterpret_cast<uint32_t*>(Xqp + row * p.ldxq + c0) = q;
                }
            }
        }
    };
    if (IT == 1 && RT == 4 && TPW <= 2) {
        // rows of at most 256 columns, at most 128 output columns: all sixteen rows of the wave are requested
        // at once (64 registers), so the phase pays the memory latency once instead of four times
        // (232,965 x 256 x 41: 0.092 -> 0.085 ms; at 256 output columns it measured 3 % slower)
        float f0[4][IT][4], f1[4][IT][4], f2[4][IT][4], f3[4][IT][4];
        fetch(f0, 0);
        fetch(f1, 4);
        fetch(f2, 8);
        fetch(f3, 12);
        emit(f0, 0);
        emit(f1, 4);
        emit(f2, 8);
        emit(f3, 12);
    } else {
        // two register buffers: the loads of the next four rows are in flight while these are quantized
        float fa[4][IT][4], fb[4][IT][4];
        fetch(fa, 0);
        fetch(fb, 4);
        emit(fa, 0);
        if (RT == 4) fetch(fa, 8);
        emit(fb, 4);
        if (RT == 4) {
            fetch(fb, 12);
            emit(fa, 8);
            emit(fb, 12);
        }
    }
    __syncthreads();

    // ---- phase B
    const int g = lane >> 4, r16 = lane & 15;
    const int64_t n0 = static_cast<int64_t>(blockIdx.y) * (64 * TPW) + static_cast<int64_t>(wave) * (16 * TPW);
    const int ksteps = p.kp >> 6;
    i32x4 acc[RT][TPW];
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int j = 0; j < TPW; ++j) acc[i][j] = i32x4{0, 0, 0, 0};

    if (n0 < p.N) {  // wave-uniform: waves whose columns lie beyond N only take part in phase A
        const int8_t* pb[TPW];
        bool bok[TPW];
        // row-major B: a lane reads its 16 bytes from its own row (a cache line look-up per lane); fragment
        // order: the wave reads one contiguous KB per fragment
        const int64_t bstep = p.b_frag ? 1024 : 64;
#pragma unroll
        for (int j = 0; j < TPW; ++j) {
            const int64_t n = n0 + j * 16 + r16;
            bok[j] = n < p.N;
            if (p.b_frag) {
                const int64_t tile = n0 + j * 16 < p.N ? (n0 >> 4) + j : 0;
                pb[j] = p.B + ((tile * ksteps) << 10) + lane * 16;
            } else {
                pb[j] = p.B + (bok[j] ? n : 0) * p.ldb + g * 16;
            }
        }
        // B fragments run two k-steps ahead of the MFMAs that consume them
        i32x4 b0[TPW], b1[TPW], b2[TPW];
        auto load_bfrag = [&](i32x4* dst, int step) {
            const int sc = step < ksteps ? step : ksteps - 1;
#pragma unroll
            for (int j = 0; j < TPW; ++j) dst[j] = *reinterpret_cast<const i32x4*>(pb[j] + static_cast<int64_t>(sc) * bstep);
        };
        auto mma_step = [&](const i32x4* bf, int step) {
#pragma unroll
            for (int i = 0; i < RT; ++i) {
                const i32x4 a = *reinterpret_cast<const i32x4*>(a_lds + (i * 16 + r16) * pitch + step * 64 + g * 16);
#pragma unroll
                for (int j = 0; j < TPW; ++j) {
                    const i32x4 b = bok[j] ? bf[j] : i32x4{0, 0, 0, 0};
                    acc[i][j] = mfma_16x16x64(b, a, acc[i][j]);
                }
            }
        };
        if (TPW >= 4) {
            // sixteen accumulator tiles per wave: one k-step of B fragments ahead keeps the kernel
            // under 128 registers (four waves per SIMD instead of three)
            load_bfrag(b0, 0);
            for (int step = 0; step < ksteps; step += 2) {
                load_bfrag(b1, step + 1);
                mma_step(b0, step);
                if (step + 1 < ksteps) {
                    load_bfrag(b0, step + 2);
                    mma_step(b1, step + 1);
                }
            }
        } else {
            load_bfrag(b0, 0);
            load_bfrag(b1, 1);
            for (int step = 0; step < ksteps; step += 3) {
                load_bfrag(b2, step + 2);
                mma_step(b0, step);
                if (step + 1 < ksteps) {
                    load_bfrag(b0, step + 3);
                    mma_step(b1, step + 1);
                }
                if (step + 2 < ksteps) {
                    load_bfrag(b1, step + 4);
                    mma_step(b2, step + 2);
                }
            }
        }
    }

    // ---- epilogue: lane holds C[row_base + 16 i + r16][n0 + 16 j + 4 g + v]
    const float s = p.sA[0] * p.sB[0];
    float m = 0.0f;
    const uintptr_t ca = reinterpret_cast<uintptr_t>(p.C);
    const int wide = ((ca & 15) == 0 && (p.ldc & 3) == 0) ? 4 : ((ca & 7) == 0 && (p.ldc & 1) == 0) ? 2 : 1;
    if (n0 < p.N) {
#pragma unroll
        for (int i = 0; i < RT; ++i) {
            const int64_t row = row_base + i * 16 + r16;
            if (row < p.M) {
                float* crow = p.C + row * p.ldc;
#pragma unroll
                for (int j = 0; j < TPW; ++j) {
                    const int64_t col = n0 + j * 16 + g * 4;
                    float y[4];
                    const f32x4 bv = *reinterpret_cast<const f32x4*>(bias_lds + wave * (16 * TPW) + j * 16 + g * 4);
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        y[v] = s * static_cast<float>(acc[i][j][v]);
                        if (p.bias) y[v] = bv[v] + y[v];
                        if (col + v < p.N) m = fmaxf(m, fabsf(y[v]));
                    }
                    if (col + 4 <= p.N && wide == 4) {
                        *reinterpret_cast<f32x4*>(crow + col) = f32x4{y[0], y[1], y[2], y[3]};
                    } else if (col + 4 <= p.N && wide == 2) {
                        typedef float f32x2 __attribute__((ext_vector_type(2)));
                        *reinterpret_cast<f32x2*>(crow + col) = f32x2{y[0], y[1]};
                        *reinterpret_cast<f32x2*>(crow + col + 2) = f32x2{y[2], y[3]};
                    } else {
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            if (col + v < p.N) crow[col + v] = y[v];
                    }
                }
            }
        }
    }
    if (p.absmax_out) block_absmax_to_global(m / 127.0f, p.absmax_out);
}

// Forward GEMM with the quantize fused in, for tall X, 129 to 256 output columns and K <= 64 KSTEPS: one
// persistent workgroup of sixteen waves per compute unit walks the 16-row tiles of X.  Waves 8..15 only stream:
// each owns two rows of every tile, requests them three tiles ahead, quantizes them in registers and writes the
// bytes to Xq and to a two-slot LDS ring.  Waves 0..7 only multiply and store: each keeps the B fragments of two
// column tiles in registers for the whole launch (fragment-order packing: one contiguous KB per fragment), reads
// the A fragments of the tile from the ring and stores a 16 x 32 piece of Y.  gemm_fq_kernel runs these phases
// one after the other inside a workgroup of four waves; here the stream of X never pauses for the MFMAs or the
// Y stores, and the sixteen rows of a tile reach Y (and Xq) together.  One barrier per tile hands a slot over.
template <int KSTEPS, int XV, int MODE>
__global__ __launch_bounds__(1024) void gemm_fqr_kernel(const FqParams p, int ntiles) {
    constexpr int IT = (KSTEPS * 64 + 255) / 256;  // 256-column chunks of a row a lane loads from
    constexpr int D = 3;                           // tiles in flight per streaming wave
    extern __shared__ __attribute__((aligned(16))) int8_t ring[];  // 2 x ([16][pitch] + 64), then 256 floats of bias
    const int pitch = p.pitch;
    const int slot_bytes = 16 * pitch + 64;
    float* bias_lds = reinterpret_cast<float*>(ring + 2 * slot_bytes);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
    const int stride = static_cast<int>(gridDim.x);
    const int t0 = static_cast<int>(blockIdx.x);
    const int rounds = t0 < ntiles ? (ntiles - t0 + stride - 1) / stride : 0;  // the same for every wave
    auto hand_over = [] { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    if (threadIdx.x < 256) bias_lds[threadIdx.x] = (p.bias && threadIdx.x < p.N) ? p.bias[threadIdx.x] : 0.0f;

    if (wave >= 8) {  // ---- streaming waves: rows 2 (wave - 8) and 2 (wave - 8) + 1 of every tile
        const int lr0 = 2 * (wave - 8);
        const float rs = rscale_of(p.sA[0]);
        // lane owns columns 4 (lane + 64 it) .. + 3 of its rows, read in pieces of XV floats; K is a multiple of XV
        // (host), so a piece is either inside a row or past its end
        bool in[IT][4 / XV];
#pragma unroll
        for (int it = 0; it < IT; ++it)
#pragma unroll
            for (int h = 0; h < 4 / XV; ++h) in[it][h] = ((lane + 64 * it) << 2) + XV * h < p.K;
        const int last_piece = static_cast<int>(p.K) - XV;  // where the pieces past a row's end read instead
        // Every load is issued unconditionally (a piece past the end of a row reads the row's last piece again:
        // the same 64 bytes as its neighbour lanes in the same instruction, so no request is added; a row
        // past the end of X reads the last row, a tile past the last one reads the last one again) and what must
        // not count is replaced afterwards: the number of loads between a request and its use is then fixed, and
        // the wait for a register set waits for that set only, not for the younger requests
        const int t_last = t0 + (rounds - 1) * stride;
        auto fetch = [&](float (*f)[IT][4], float* rm, int t) {
            if (t > t_last) t = t_last;
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                int64_t row = static_cast<int64_t>(t) * 16 + lr0 + b;
                if (row >= p.M) row = p.M - 1;  // last tile only; these rows are not stored
                const float* xr = p.X + row * p.ldx;
                const float* rp = p.x_row_mul ? p.x_row_mul + row : p.sA;
                rm[b] = *rp;
#pragma unroll
                for (int it = 0; it < IT; ++it) {
                    if (XV == 4) {
                        const f32x4 v = __builtin_nontemporal_load(
                            reinterpret_cast<const f32x4*>(xr + (in[it][0] ? (lane << 2) + 256 * it : last_piece)));
                        f[b][it][0] = v.x; f[b][it][1] = v.y; f[b][it][2] = v.z; f[b][it][3] = v.w;
                    } else {
                        typedef float f32x2 __attribute__((ext_vector_type(2)));
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            const f32x2 v = __builtin_nontemporal_load(
                                reinterpret_cast<const f32x2*>(xr + (in[it][h] ? (lane << 2) + 256 * it + 2 * h : last_piece)));
                            f[b][it][2 * h] = v.x;
                            f[b][it][2 * h + 1] = v.y;
                        }
                    }
                }
            }
        };
        auto emit = [&](float (*f)[IT][4], const float* rm, int slot) {
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                int8_t* dst = ring + slot * slot_bytes + (lr0 + b) * pitch + (lane << 2);
#pragma unroll
                for (int it = 0; it < IT; ++it) {
                    const int c0 = (lane + 64 * it) << 2;
                    if (c0 < pitch) {  // the columns between K and the pitch take zeros
                        constexpr int H = 4 / XV;  // pieces per four floats
                        float x0 = f[b][it][0], x1 = f[b][it][1], x2 = f[b][it][2], x3 = f[b][it][3];
                        if (it == IT - 1) {  // K > 256 (IT - 1) (host): only the last chunk can reach past the row
                            x0 = in[it][0] ? x0 : 0.0f; x1 = in[it][0] ? x1 : 0.0f;
                            x2 = in[it][H - 1] ? x2 : 0.0f; x3 = in[it][H - 1] ? x3 : 0.0f;
                        }
                        if (p.x_row_mul) { x0 = x0 * rm[b]; x1 = x1 * rm[b]; x2 = x2 * rm[b]; x3 = x3 * rm[b]; }
                        *reinterpret_cast<uint32_t*>(dst + 256 * it) =
                            pack4(quant_one<MODE>(x0, rs, 0.f), quant_one<MODE>(x1, rs, 0.f),
                                  quant_one<MODE>(x2, rs, 0.f), quant_one<MODE>(x3, rs, 0.f));
                    }
                }
            }
        };
        // the register sets take turns by unrolling, so that no set is copied while its loads are in flight
        float f[D][2][IT][4];
        float rm[D][2];
#pragma unroll
        for (int u = 0; u < D; ++u) fetch(f[u], rm[u], t0 + u * stride);  // rounds >= 1 (host)
        emit(f[0], rm[0], 0);
        fetch(f[0], rm[0], t0 + D * stride);
        hand_over();  // slot 0 holds the first tile
        // round k: the tile of round k + 1 goes to slot (k + 1) % 2 while waves 0..7 read slot k % 2
        for (int kb = 0; kb < rounds; kb += D) {
#pragma unroll
            for (int u = 0; u < D; ++u) {
                const int k = kb + u;
                if (k >= rounds) break;
                const int set = (u + 1) % D;
                emit(f[set], rm[set], (k + 1) & 1);  // past the last round: the last tile again, read by nobody
                fetch(f[set], rm[set], t0 + (k + 1 + D) * stride);
                hand_over();
            }
        }
        if (p.absmax_out) block_absmax_to_global(0.0f, p.absmax_out);
        return;
    }

    // ---- multiplying waves: column tiles 2 wave and 2 wave + 1
    const int g = lane >> 4, r16 = lane & 15;
    const int n0 = 32 * wave;
    i32x4 b[2][KSTEPS];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const bool tile_ok = n0 + 16 * j < p.N;  // tiles past the last column multiply zeros and store nothing
        const int8_t* pb = p.B + ((static_cast<int64_t>(tile_ok ? 2 * wave + j : 0) * KSTEPS) << 10) + lane * 16;
#pragma unroll
        for (int st = 0; st < KSTEPS; ++st) {
            b[j][st] = i32x4{0, 0, 0, 0};
            if (tile_ok) b[j][st] = *reinterpret_cast<const i32x4*>(pb + (st << 10));
        }
    }
    const float s = p.sA[0] * p.sB[0];
    const uintptr_t ca = reinterpret_cast<uintptr_t>(p.C);
    const int wide = ((ca & 15) == 0 && (p.ldc & 3) == 0) ? 4 : ((ca & 7) == 0 && (p.ldc & 1) == 0) ? 2 : 1;
    const int frag0 = r16 * pitch + g * 16;
    const bool plain = !p.bias && wide == 4 && n0 + 32 <= p.N;
    // Xq leaves through these waves too, 16 bytes per lane straight from the ring (a row of Xq is ldxq / 16 <= pitch / 16
    // pieces; the bytes past K are the zeros the streaming waves wrote): the streaming waves hold 4 bytes per lane
    // and row, and a store of 256 bytes per instruction costs as much issue time as one of 1 KB
    const int cpr = static_cast<int>(p.ldxq >> 4);
    int q_lds[2], q_row[2];
    int64_t q_glb[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int id = i * 512 + wave * 64 + lane;
        const int r = id / cpr, c = id - r * cpr;
        q_row[i] = r < 16 ? r : -1;
        q_lds[i] = r * pitch + c * 16;
        q_glb[i] = static_cast<int64_t>(r) * p.ldxq + c * 16;
    }
    float m = 0.0f;
    hand_over();
    for (int k = 0; k < rounds; ++k) {
        const int8_t* slot = ring + (k & 1) * slot_bytes + frag0;
        i32x4 acc[2] = {i32x4{0, 0, 0, 0}, i32x4{0, 0, 0, 0}};
#pragma unroll
        for (int st = 0; st < KSTEPS; ++st) {
            const i32x4 a = *reinterpret_cast<const i32x4*>(slot + st * 64);
            acc[0] = mfma_16x16x64(b[0][st], a, acc[0]);  // operands swapped, see gemm_nt_kernel
            acc[1] = mfma_16x16x64(b[1][st], a, acc[1]);
        }
        const int64_t row0 = static_cast<int64_t>(t0 + k * stride) * 16;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            if (q_row[i] >= 0 && row0 + q_row[i] < p.M)
                *reinterpret_cast<i32x4*>(p.Xq + row0 * p.ldxq + q_glb[i]) =
                    *reinterpret_cast<const i32x4*>(ring + (k & 1) * slot_bytes + q_lds[i]);
        }
        const int64_t row = row0 + r16;
        if (row < p.M && plain) {  // whole tiles, 16-byte stores, no bias: nothing to test per tile
            f32x4* cp = reinterpret_cast<f32x4*>(p.C + row * p.ldc + n0 + 4 * g);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const f32x4 y{s * static_cast<float>(acc[j][0]), s * static_cast<float>(acc[j][1]),
                              s * static_cast<float>(acc[j][2]), s * static_cast<float>(acc[j][3])};
                m = fmaxf(fmaxf(m, fmaxf(fabsf(y[0]), fabsf(y[1]))), fmaxf(fabsf(y[2]), fabsf(y[3])));
                cp[4 * j] = y;
            }
        } else if (row < p.M) {
            float* crow = p.C + row * p.ldc;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int col = n0 + 16 * j + 4 * g;
                if (col >= p.N) continue;
                float y[4];
                const f32x4 bv = *reinterpret_cast<const f32x4*>(bias_lds + col);
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    y[v] = s * static_cast<float>(acc[j][v]);
                    if (p.bias) y[v] = bv[v] + y[v];
                    if (col + v < p.N) m = fmaxf(m, fabsf(y[v]));
                }
                if (col + 4 <= p.N && wide == 4) {
                    *reinterpret_cast<f32x4*>(crow + col) = f32x4{y[0], y[1], y[2], y[3]};
                } else if (col + 4 <= p.N && wide == 2) {
                    typedef float f32x2 __attribute__((ext_vector_type(2)));
                    *reinterpret_cast<f32x2*>(crow + col) = f32x2{y[0], y[1]};
                    *reinterpret_cast<f32x2*>(crow + col + 2) = f32x2{y[2], y[3]};
                } else {
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        if (col + v < p.N) crow[col + v] = y[v];
                }
            }
        }
        hand_over();  // the slot just read may be refilled, the other one is complete
    }
    if (p.absmax_out) block_absmax_to_global(m / 127.0f, p.absmax_out);
}

// W-stationary forward for tall X and narrow outputs (N <= 32): one persistent 12-wave workgroup per
// CU keeps the whole packed W in LDS; the 16-row blocks of X are dealt round-robin over the waves of
// the launch and a wave owns ALL N columns of its block.  A lane loads floats of X that belong to
// its row's MFMA A-fragment, quantizes them in registers, the four lanes of a row exchange dwords,
// the 16 bytes go to Xq (the backward cache) and straight into the MFMAs: X never passes through
// LDS, there is no barrier after the W load, and the HBM reads run three k-steps ahead, so loads,
// MFMAs and the Y stores of different waves overlap.  NT = 16-column tiles (N <= 16 NT).
// (For wide outputs the accumulators of all N columns leave too few registers for the prefetch
// and gemm_fq_kernel's LDS-staged form is faster: 0.30 ms against 0.49 ms at 232,965 x 602 x 256.)
template <int NT, int XV, int MODE, int THREADS>
__global__ __launch_bounds__(THREADS) void gemm_ws_kernel(const FqParams p, int nblocks, int pitch, int kq) {
    extern __shared__ __attribute__((aligned(16))) int8_t w_lds[];  // [16 NT][pitch]
    constexpr int RT = 1;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int g = lane >> 4, r16 = lane & 15;

    // ---- W -> LDS, rows beyond N and chunks beyond kq zero-filled
    {
        const int cpr = pitch >> 4;  // 16-byte chunks per LDS row
        for (int idx = tid; idx < 16 * NT * cpr; idx += THREADS) {
            const int n = idx / cpr, c = idx - n * cpr;
            i32x4 v{0, 0, 0, 0};
            if (n < p.N && c * 16 < kq) v = *reinterpret_cast<const i32x4*>(p.B + static_cast<int64_t>(n) * p.ldb + c * 16);
            *reinterpret_cast<i32x4*>(w_lds + n * pitch + c * 16) = v;
        }
    }
    __syncthreads();

    const float rs = rscale_of(p.sA[0]);
    const float s = p.sA[0] * p.sB[0];
    const int ksteps = (static_cast<int>(p.K) + 63) >> 6;
    const uintptr_t ca = reinterpret_cast<uintptr_t>(p.C);
    const int wide = ((ca & 15) == 0 && (p.ldc & 3) == 0) ? 4 : ((ca & 7) == 0 && (p.ldc & 1) == 0) ? 2 : 1;
    float m = 0.0f;

    // raw[i][4 w + c] = X[row0 + 16 i + r16][64 step + 16 w + 4 g + c]: in load w the four lanes of a row
    // (g = 0..3) read 64 contiguous bytes, so a wave-wide load covers 16 rows x 64 B instead of 64
    // scattered 16-byte pieces; the lanes of a row exchange dwords after quantization (below).
    auto load_raw = [&](float (*raw)[16], int64_t row0, int step) {
        const int64_t kbase = static_cast<int64_t>(step) * 64 + g * 4;
#pragma unroll
        for (int i = 0; i < RT; ++i) {
            const int64_t row = row0 + 16 * i + r16;
            const float* xr = p.X + row * p.ldx + kbase;
            if (row < p.M && static_cast<int64_t>(step) * 64 + 64 <= p.K) {
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    if (XV == 4) {
                        const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(xr + 16 * w));
                        raw[i][4 * w] = v.x; raw[i][4 * w + 1] = v.y; raw[i][4 * w + 2] = v.z; raw[i][4 * w + 3] = v.w;
                    } else {
                        typedef float f32x2 __attribute__((ext_vector_type(2)));
                        const f32x2 v0 = __builtin_nontemporal_load(reinterpret_cast<const f32x2*>(xr + 16 * w));
                        const f32x2 v1 = __builtin_nontemporal_load(reinterpret_cast<const f32x2*>(xr + 16 * w + 2));
                        raw[i][4 * w] = v0.x; raw[i][4 * w + 1] = v0.y; raw[i][4 * w + 2] = v1.x; raw[i][4 * w + 3] = v1.y;
                    }
                }
            } else {  // the last, partial k-step and rows past M
#pragma unroll
                for (int w = 0; w < 4; ++w)
#pragma unroll
                    for (int c = 0; c < 4; ++c)
                        raw[i][4 * w + c] = (row < p.M && kbase + 16 * w + c < p.K) ? xr[16 * w + c] : 0.0f;
            }
        }
    };
    // quantize raw into the A fragments of this step, store them to Xq, run the step's MFMAs
    auto step_mma = [&](float (*raw)[16], int64_t row0, int step, i32x4 (*acc)[NT]) {
        const int64_t k0 = static_cast<int64_t>(step) * 64 + g * 16;
        const bool chunk_ok = k0 < kq;
        i32x4 a[RT];
#pragma unroll
        for (int i = 0; i < RT; ++i) {
            const int64_t row = row0 + 16 * i + r16;
            const float rm = (p.x_row_mul && row < p.M) ? p.x_row_mul[row] : 1.0f;
            uint32_t q[4];  // q[w]: the bytes of columns 64 step + 16 w + 4 g .. + 3
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                float x0 = raw[i][4 * w], x1 = raw[i][4 * w + 1], x2 = raw[i][4 * w + 2], x3 = raw[i][4 * w + 3];
                if (p.x_row_mul) { x0 = x0 * rm; x1 = x1 * rm; x2 = x2 * rm; x3 = x3 * rm; }
                q[w] = pack4(quant_one<MODE>(x0, rs, 0.f), quant_one<MODE>(x1, rs, 0.f),
                             quant_one<MODE>(x2, rs, 0.f), quant_one<MODE>(x3, rs, 0.f));
            }
            // 4 x 4 dword transpose over the four lanes of the row (lanes r16 + 16 g): afterwards this lane holds
            // columns 64 step + 16 g .. + 15 in order, i.e. its MFMA fragment.  Round k: lane g pulls from lane
            // (g + k) & 3 the dword that lane holds for w = g, which is that lane's register (its g - k) & 3.
            uint32_t f[4] = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int give = (g - k) & 3;
                const uint32_t present = give == 0 ? q[0] : give == 1 ? q[1] : give == 2 ? q[2] : q[3];
                const int from = (g + k) & 3;
                const uint32_t got = static_cast<uint32_t>(__shfl(static_cast<int>(present), from * 16 + r16, kWave));
#pragma unroll
                for (int d = 0; d < 4; ++d)
                    if (from == d) f[d] = got;
            }
            a[i] = i32x4{static_cast<int>(f[0]), static_cast<int>(f[1]), static_cast<int>(f[2]), static_cast<int>(f[3])};
            if (chunk_ok && row < p.M)
                __builtin_nontemporal_store(a[i], reinterpret_cast<i32x4*>(p.Xq + row * p.ldxq + k0));
        }
        const int kb = chunk_ok ? static_cast<int>(k0) : 0;  // a is all zero for chunks past kq: any in-range B will do
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const i32x4 b = *reinterpret_cast<const i32x4*>(w_lds + (16 * j + r16) * pitch + kb);
#pragma unroll
            for (int i = 0; i < RT; ++i) acc[i][j] = mfma_16x16x64(b, a[i], acc[i][j]);
        }
    };

    // blocks are dealt round-robin over all waves of the launch (a shared ticket counter serialises:
    // one device-scope atomic per block on a single address, ~15 ns each, costs more than the block)
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int waves = static_cast<int>(gridDim.x) * (static_cast<int>(blockDim.x) >> 6);
    for (int t = static_cast<int>(blockIdx.x) * (static_cast<int>(blockDim.x) >> 6) + wave; t < nblocks; t += waves) {
        const int64_t row0 = static_cast<int64_t>(t) * (16 * RT);
        i32x4 acc[RT][NT];
#pragma unroll
        for (int i = 0; i < RT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j) acc[i][j] = i32x4{0, 0, 0, 0};
        // the X loads run three k-steps ahead of the MFMAs that consume them
        float r0[RT][16], r1[RT][16], r2[RT][16], r3[RT][16];
        load_raw(r0, row0, 0);
        if (1 < ksteps) load_raw(r1, row0, 1);
        if (2 < ksteps) load_raw(r2, row0, 2);
        for (int step = 0; step < ksteps; step += 4) {
            if (step + 3 < ksteps) load_raw(r3, row0, step + 3);
            step_mma(r0, row0, step, acc);
            if (step + 1 < ksteps) {
                if (step + 4 < ksteps) load_raw(r0, row0, step + 4);
                step_mma(r1, row0, step + 1, acc);
            }
            if (step + 2 < ksteps) {
                if (step + 5 < ksteps) load_raw(r1, row0, step + 5);
                step_mma(r2, row0, step + 2, acc);
            }
            if (step + 3 < ksteps) {
                if (step + 6 < ksteps) load_raw(r2, row0, step + 6);
                step_mma(r3, row0, step + 3, acc);
            }
        }
        // lane holds C[row0 + 16 i + r16][16 j + 4 g + v]
#pragma unroll
        for (int i = 0; i < RT; ++i) {
            const int64_t row = row0 + i * 16 + r16;
            if (row < p.M) {
                float* crow = p.C + row * p.ldc;
#pragma unroll
                for (int j = 0; j < NT; ++j) {
                    const int64_t col = j * 16 + g * 4;
                    float y[4];
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        y[v] = s * static_cast<float>(acc[i][j][v]);
                        if (p.bias && col + v < p.N) y[v] = p.bias[col + v] + y[v];
                        if (col + v < p.N) m = fmaxf(m, fabsf(y[v]));
                    }
                    if (col + 4 <= p.N && wide == 4) {
                        *reinterpret_cast<f32x4*>(crow + col) = f32x4{y[0], y[1], y[2], y[3]};
                    } else if (col + 4 <= p.N && wide == 2) {
                        typedef float f32x2 __attribute__((ext_vector_type(2)));
                        *reinterpret_cast<f32x2*>(crow + col) = f32x2{y[0], y[1]};
                        *reinterpret_cast<f32x2*>(crow + col + 2) = f32x2{y[2], y[3]};
                    } else {
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            if (col + v < p.N) crow[col + v] = y[v];
                    }
                }
            }
        }
    }
    if (p.absmax_out) block_absmax_to_global(m / 127.0f, p.absmax_out);
}

// ------------------------------------------------------- operand packing
// dst[r, 0..ldd) = src[r, 0..cols) zero-filled, for r < rows (src row stride lds).
__global__ __launch_bounds__(256) void pack_rows_i8_kernel(int8_t* __restrict__ dst, int64_t ldd,
                                                           const int8_t* __restrict__ src, int64_t lds,
                                                           int64_t rows, int64_t cols) {
    const int64_t total = rows * ldd;
    const int64_t nthr = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += nthr) {
        const int64_t r = i / ldd, c = i - r * ldd;
        dst[i] = c < cols ? src[r * lds + c] : static_cast<int8_t>(0);
    }
}

// The weight operand of the forward GEMM in one pass: Wq[n, k] = quantize(W[n, k]) (the cache the
// backward reads) and the same bytes in the packed form the MFMA loop reads, rows of ldp bytes,
// zero-filled.  Thread 0 also zeroes the slot the GEMM's epilogue maxes the output scale into.
template <int MODE>
__global__ __launch_bounds__(256) void quantize_pack_w_kernel(const float* __restrict__ W, int64_t ldw,
                                                              const float* __restrict__ scale,
                                                              int8_t* __restrict__ Wq, int8_t* __restrict__ packed,
                                                              int64_t ldp, int64_t N, int64_t K,
                                                              float* __restrict__ zero_slot, int frag) {
    if (zero_slot && blockIdx.x == 0 && threadIdx.x == 0) zero_slot[0] = 0.0f;
    const float r = rscale_of(scale[0]);
    // frag: the packed copy is laid out in MFMA fragment order instead of rows (ldp is a multiple of 64): the 16
    // bytes that lane 16 g + r feeds the MFMA of column tile j at k-step st (row 16 j + r, columns 64 st + 16 g ..)
    // stand at ((j ldp / 64 + st) 64 + 16 g + r) 16, so that a wave fetches a fragment as one contiguous KB; rows
    // up to the next multiple of 16 are zero-filled
    const int64_t rows = frag ? (N + 15) / 16 * 16 : N;
    const int64_t total = rows * ldp;
    const int64_t nthr = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += nthr) {
        const int64_t n = i / ldp, k = i - n * ldp;
        int8_t q = 0;
        if (k < K && n < N) {
            q = static_cast<int8_t>(quant_one<MODE>(W[n * ldw + k], r, 0.0f));
            Wq[n * K + k] = q;
        }
        int64_t at = i;
        if (frag) at = ((((n >> 4) * (ldp >> 6) + (k >> 6)) << 6) + (((k >> 4) & 3) << 4) + (n & 15)) * 16 + (k & 15);
        packed[at] = q;
    }
}

// dst[c, 0..ldd) = src[0..rows, c] zero-filled, for c < cols: dst is [cols, ldd].
__global__ __launch_bounds__(256) void transpose_pack_i8_kernel(int8_t* __restrict__ dst, int64_t ldd,
                                                                const int8_t* __restrict__ src,
                                                                int64_t lds, int64_t rows, int64_t cols) {
    const int64_t total = cols * ldd;
    const int64_t nthr = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += nthr) {
        const int64_t c = i / ldd, r = i - c * ldd;
        dst[i] = r < rows ? src[r * lds + c] : static_cast<int8_t>(0);
    }
}

// ------------------------------------------------------------- TN kernel
struct TnParams {
    int* acc;          // [splits, N, Kp] int32 partial sums, one slab per split of M (Kp = K rounded up to 4)
    int64_t Kp;
    const int8_t* A;   // dY [M, N] int8, row stride lda
    const int8_t* B;   // X  [M, K] int8, row stride ldb
    int64_t M, N, K;
    int64_t lda, ldb;
    int64_t a_row_bytes, b_row_bytes;  // readable bytes per row
    int64_t chunk;     // rows of M per split (multiple of 64)
    int tiles_n, tiles_k, splits;
};

// Workgroup tile: 128 (n) x 128 (k), reduction in steps of 64 rows of M.
// Waves 2 x 2, each 64 x 64.  Fragment row r16 of sub-tile j maps to column
// 4 * r16 + j of the wave's 64-wide range (the order the register transpose
// produces); the output indexing below undoes it.
template <int VEC>
__global__ __launch_bounds__(256, 2) void gemm_tn_kernel(const TnParams p) {
    constexpr int PITCH = 33;  // dwords per LDS row: 128 bytes + 4, odd so that row groups spread over banks
    __shared__ uint32_t ldsA[64 * PITCH];
    __shared__ uint32_t ldsB[64 * PITCH];

    // consecutive launch ids land on different XCDs; give each XCD a contiguous range of tiles
    // so that the tiles sharing one M-chunk run on the same L2
    const int nblk = gridDim.x;
    int bid = blockIdx.x;
    if ((nblk & 7) == 0) bid = (bid & 7) * (nblk >> 3) + (bid >> 3);
    const int tiles = p.tiles_n * p.tiles_k;
    const int split = bid / tiles;
    const int tile = bid - split * tiles;
    const int tn = tile / p.tiles_k, tk = tile - tn * p.tiles_k;
    const int64_t n0 = static_cast<int64_t>(tn) * 128, k0 = static_cast<int64_t>(tk) * 128;
    const int64_t m_begin = static_cast<int64_t>(split) * p.chunk;
    const int64_t m_end = (m_begin + p.chunk < p.M) ? m_begin + p.chunk : p.M;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave >> 1, wk = wave & 1;
    const int g = lane >> 4, r16 = lane & 15;

    // staging: a tile is 64 rows x 8 chunks of 16 bytes = 512 chunks, 2 per thread per operand
    const int srow = tid >> 3, scol = tid & 7;  // rows srow and srow + 32, chunk scol

    i32x4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = i32x4{0, 0, 0, 0};

    auto fetch = [&](i32x4* ra, i32x4* rb, int64_t m0) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int64_t m = m0 + srow + 32 * h;
            const bool mok = m < m_end;
            const int64_t ca = n0 + scol * 16, cb = k0 + scol * 16;
            ra[h] = load16<VEC>(p.A + m * p.lda + ca, (mok && ca < p.N) ? p.a_row_bytes - ca : 0);
            rb[h] = load16<VEC>(p.B + m * p.ldb + cb, (mok && cb < p.K) ? p.b_row_bytes - cb : 0);
        }
    };
    auto stage = [&](const i32x4* ra, const i32x4* rb) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            uint32_t* da = ldsA + (srow + 32 * h) * PITCH + scol * 4;
            uint32_t* db = ldsB + (srow + 32 * h) * PITCH + scol * 4;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                da[q] = static_cast<uint32_t>(ra[h][q]);
                db[q] = static_cast<uint32_t>(rb[h][q]);
            }
        }
    };
    // four fragments (sub-tiles j = 0..3) of the wave's 64 columns starting at dword column c0
    auto frags = [&](const uint32_t* lds, int c0, i32x4* out) {
        uint32_t col[4][4];  // [m-block][j]
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) {
            const uint32_t* base = lds + (g * 16 + mb * 4) * PITCH + c0 + r16;
            transpose4x4(base[0], base[PITCH], base[2 * PITCH], base[3 * PITCH], col[mb]);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
            out[j] = i32x4{static_cast<int>(col[0][j]), static_cast<int>(col[1][j]),
                           static_cast<int>(col[2][j]), static_cast<int>(col[3][j])};
    };

    i32x4 ra[2], rb[2];
    fetch(ra, rb, m_begin);
    for (int64_t m0 = m_begin; m0 < m_end; m0 += 64) {
        __syncthreads();  // previous step's fragments are consumed
        stage(ra, rb);
        __syncthreads();
        fetch(ra, rb, m0 + 64);  // rows beyond m_end come back as zeros
        i32x4 fa[4], fb[4];
        frags(ldsA, wn * 16, fa);
        frags(ldsB, wk * 16, fb);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = mfma_16x16x64(fa[i], fb[j], acc[i][j]);
    }

    // acc[i][j][v] at lane (g, r16): n = n0 + 64 wn + 4 (4 g + v) + i, k = k0 + 64 wk + 4 r16 + j.
    // Every (split, n, k) belongs to exactly one workgroup, so the slab is written with plain
    // 16-byte stores (j = 0..3 are adjacent columns) and needs no zero fill.
    int* slab = p.acc + static_cast<int64_t>(split) * p.N * p.Kp;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int64_t n = n0 + wn * 64 + 4 * (4 * g + v) + i;
            const int64_t k = k0 + wk * 64 + 4 * r16;
            if (n < p.N && k < p.Kp)
                *reinterpret_cast<i32x4*>(slab + n * p.Kp + k) =
                    i32x4{acc[i][0][v], acc[i][1][v], acc[i][2][v], acc[i][3][v]};
        }
}

// 64 lanes x 16 bytes from the lanes' global addresses to 1 KB of LDS starting at a wave-uniform address.  As
// assembly, not as the compiler's builtin: the compiler makes every later LDS read of the kernel wait for all such
// loads in flight at some joins of the loop (it cannot tell the ring's stages apart there), which would undo the
// ring; the kernel's own s_waitcnt instructions order these loads instead.  M0 carries the LDS address and is not
// used by anything else in the kernel.
__device__ __forceinline__ void load_to_lds_16(const void* gptr, void* lds_wave_base) {
    const unsigned lds = static_cast<unsigned>(
        reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)lds_wave_base));  // generic -> LDS offset
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds), "v"(gptr) : "memory");
}

// The same tile and slab layout as gemm_tn_kernel for rows readable in aligned 16-byte chunks, built around three
// things that kernel lacks.  (1) The operands are staged by global-to-LDS loads into a ring of four 64-row steps:
// gemm_tn_kernel pays one memory round trip per step (its loads are asked for one step ahead, land in registers
// and go through LDS store instructions and a second barrier); here a step's 16 KB are asked for three steps ahead
// and land in LDS by themselves, and a step is: wait for the loads of steps s and s + 1 (s_waitcnt vmcnt(4): the
// youngest step stays in flight), one bare barrier (__syncthreads() carries a release fence that waits for every
// load in flight, which is exactly what the ring is there to avoid), ask for step s + 3 into the stage that step
// s - 1 left, read the operands of step s + 1, multiply step s.  Each stage is an LDS object of its own.
// (2) The operands are read by the transposing LDS read, no byte transposes in registers.  ds_read_b64_tr_b8: within
// sixteen lanes, lane j gives the address of an 8-byte block and lane i receives byte i % 8 of the blocks of lanes
// i / 8, i / 8 + 2, ..., i / 8 + 14; with lane j pointing at row j / 2, bytes 8 (j % 2) .. of a 16-column strip, lane i
// gets column i of eight consecutive rows: eight consecutive m of one n (or k), which is what a matrix operand
// wants of a tile stored [m][n].  Two such reads are a lane's sixteen bytes of an operand of
// (3) v_mfma_i32_32x32x32_i8 (lane l: row l % 32, reduction indices 16 (l / 32) .. + 15), which runs at 1.7 times the
// rate of the 16 x 16 x 64 instruction on this device.
// LDS rows have a pitch of exactly 128 bytes (a wave's load instruction lands 64 x 16 bytes back to back); the
// 16-byte chunk index is XORed with row % 8, so that the eight rows of a transposing read sit in eight different
// chunks (all 32 banks): lane L of a load instruction fills LDS chunk L, so it asks global memory for the chunk that
// belongs there.  232,965 x 256 x 602: 48 us (gemm_tn_kernel 69, the ring with byte transposes and 16 x 16 x 64: 64).
__global__ __launch_bounds__(256, 2) void gemm_tn_tr_kernel(const TnParams p) {
    typedef int v2i32 __attribute__((ext_vector_type(2)));
    typedef int i32x16t __attribute__((ext_vector_type(16)));
    // a stage: the A tile, then the B tile, [64 rows][128 bytes] each
    __shared__ uint32_t st0[4096], st1[4096], st2[4096], st3[4096];
    uint32_t* const sA0 = st0; uint32_t* const sB0 = st0 + 2048;
    uint32_t* const sA1 = st1; uint32_t* const sB1 = st1 + 2048;
    uint32_t* const sA2 = st2; uint32_t* const sB2 = st2 + 2048;
    uint32_t* const sA3 = st3; uint32_t* const sB3 = st3 + 2048;

    const int nblk = gridDim.x;
    int bid = blockIdx.x;
    if ((nblk & 7) == 0) bid = (bid & 7) * (nblk >> 3) + (bid >> 3);  // tiles that share an M-chunk on one XCD
    const int tiles = p.tiles_n * p.tiles_k;
    const int split = bid / tiles;
    const int tile = bid - split * tiles;
    const int tn = tile / p.tiles_k, tk = tile - tn * p.tiles_k;
    const int64_t n0 = static_cast<int64_t>(tn) * 128, k0 = static_cast<int64_t>(tk) * 128;
    const int64_t m_begin = static_cast<int64_t>(split) * p.chunk;
    const int64_t m_end = (m_begin + p.chunk < p.M) ? m_begin + p.chunk : p.M;
    const int64_t steps = (m_end - m_begin) >> 6;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave >> 1, wk = wave & 1;

    int64_t a_off[2], b_off[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int P = tid + 256 * i, row = P >> 3;
        const int lc = (P & 7) ^ (row & 7);
        int64_t ca = n0 + 16 * lc, cb = k0 + 16 * lc;
        if (ca > p.a_row_bytes - 16) ca = p.a_row_bytes - 16;
        if (cb > p.b_row_bytes - 16) cb = p.b_row_bytes - 16;
        a_off[i] = row * p.lda + ca;
        b_off[i] = row * p.ldb + cb;
    }
    auto issue = [&](uint32_t* dA, uint32_t* dB, int64_t step) {
        const int64_t m0 = m_begin + (step < steps ? step : steps - 1) * 64;
        const int8_t* ga = p.A + m0 * p.lda;
        const int8_t* gb = p.B + m0 * p.ldb;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            load_to_lds_16(ga + a_off[i], dA + (i * 256 + wave * 64) * 4);
            load_to_lds_16(gb + b_off[i], dB + (i * 256 + wave * 64) * 4);
        }
    };

    i32x16t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

    // this lane's part of the reads: group q = lane / 16 takes column strip q % 2 of a 32-column tile and the reduction
    // half q / 2; inside the group lane j points at row j / 2 and the 8-byte half j % 2 of the strip
    const int q = lane >> 4, j16 = lane & 15;
    const int rsub = j16 >> 1, hb = j16 & 1;
    // operand (tile t, half hm): rows 32 hm + 16 (q / 2) + 8 u + rsub for u = 0, 1; logical chunk base + 2 t + q % 2
    auto read_ops = [&](const uint32_t* lds, int chunk_base, i32x4 (*op)[2]) {
        const int8_t* base = reinterpret_cast<const int8_t*>(lds);
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int hm = 0; hm < 2; ++hm) {
                v2i32 r[2];
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const int row = 32 * hm + 16 * (q >> 1) + 8 * u + rsub;
                    const int pc = (chunk_base + 2 * t + (q & 1)) ^ (row & 7);
                    r[u] = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                        (__attribute__((address_space(3))) v2i32*)(base + row * 128 + pc * 16 + 8 * hb));
                }
                op[t][hm] = i32x4{r[0][0], r[0][1], r[1][0], r[1][1]};
            }
    };
    i32x4 opA[2][2], opB[2][2], nxA[2][2], nxB[2][2];
    auto multiply = [&]() {
#pragma unroll
        for (int hm = 0; hm < 2; ++hm)
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(opA[i][hm], opB[j][hm], acc[i][j], 0, 0, 0);
    };
    auto advance = [&]() {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int hm = 0; hm < 2; ++hm) {
                opA[t][hm] = nxA[t][hm];
                opB[t][hm] = nxB[t][hm];
            }
    };

    if (steps > 0) {
        issue(sA0, sB0, 0);
        issue(sA1, sB1, 1);
        issue(sA2, sB2, 2);
        __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8): step 0 has landed
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        read_ops(sA0, wn * 4, opA);
        read_ops(sB0, wk * 4, opB);
// steps s_ and s_ + 1 have landed at vmcnt(4); ask for s_ + 3 (FA, FB: the stage step s_ - 1 left), read s_ + 1, multiply s_
#define TANGO_TN_STEP(NA, NB, FA, FB, s_)          \
        asm volatile("" ::: "memory");             \
        __builtin_amdgcn_s_waitcnt(0x0F74);        \
        __builtin_amdgcn_s_barrier();              \
        asm volatile("" ::: "memory");             \
        issue(FA, FB, (s_) + 3);                   \
        read_ops(NA, wn * 4, nxA);                 \
        read_ops(NB, wk * 4, nxB);                 \
        multiply();                                \
        advance()
        for (int64_t s = 0; s < steps; s += 4) {
            TANGO_TN_STEP(sA1, sB1, sA3, sB3, s);
            if (s + 1 >= steps) break;
            TANGO_TN_STEP(sA2, sB2, sA0, sB0, s + 1);
            if (s + 2 >= steps) break;
            TANGO_TN_STEP(sA3, sB3, sA1, sB1, s + 2);
            if (s + 3 >= steps) break;
            TANGO_TN_STEP(sA0, sB0, sA2, sB2, s + 3);
        }
#undef TANGO_TN_STEP
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
    }
    const int64_t m_tail = m_begin + steps * 64;
    if (m_tail < m_end) {  // the rows of a last partial step, through registers, zeros beyond the end
        const int srow = tid >> 3, scol = tid & 7;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int row = srow + 32 * h;
            const int64_t m = m_tail + row;
            const bool mok = m < m_end;
            const int64_t ca = n0 + scol * 16, cb = k0 + scol * 16;
            const i32x4 ra = load16<16>(p.A + m * p.lda + ca, (mok && ca < p.N) ? p.a_row_bytes - ca : 0);
            const i32x4 rb = load16<16>(p.B + m * p.ldb + cb, (mok && cb < p.K) ? p.b_row_bytes - cb : 0);
            const int pc = scol ^ (row & 7);
            *reinterpret_cast<i32x4*>(sA0 + row * 32 + pc * 4) = ra;
            *reinterpret_cast<i32x4*>(sB0 + row * 32 + pc * 4) = rb;
        }
        __syncthreads();
        read_ops(sA0, wn * 4, opA);
        read_ops(sB0, wk * 4, opB);
        multiply();
    }

    // tile (i, j), register v, lane l: n = n0 + 64 wn + 32 i + 8 (v / 4) + 4 (l / 32) + v % 4, k = k0 + 64 wk + 32 j + l % 32:
    // a store instruction writes 128 contiguous bytes of two rows of the slab
    int* slab = p.acc + static_cast<int64_t>(split) * p.N * p.Kp;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int64_t k = k0 + wk * 64 + 32 * j + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int64_t n = n0 + wn * 64 + 32 * i + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (n < p.N && k < p.Kp) slab[n * p.Kp + k] = acc[i][j][v];
            }
        }
}

// dW[n, k] = (sA * sB) * float(sum over splits of part[split][n][k]).  A workgroup is 16 column
// quads x 16 split lanes: the split lanes add every 16th slab, LDS adds the sixteen.
__global__ __launch_bounds__(256) void tn_reduce_kernel(float* __restrict__ out, int64_t ldo,
                                                        const int* __restrict__ part, int64_t N, int64_t K,
                                                        int64_t Kp, int splits, const float* __restrict__ sA,
                                                        const float* __restrict__ sB) {
    __shared__ int red[16][16][4];
    const int vq = threadIdx.x & 15, sl = threadIdx.x >> 4;
    const int64_t quads = N * Kp / 4;
    const int64_t q = static_cast<int64_t>(blockIdx.x) * 16 + vq;
    i32x4 sum{0, 0, 0, 0};
    if (q < quads) {
        const i32x4* src = reinterpret_cast<const i32x4*>(part) + q;
        int sp = sl;
        for (; sp + 48 < splits; sp += 64) {  // four slabs in flight
            const i32x4 a = src[static_cast<int64_t>(sp) * quads], b = src[static_cast<int64_t>(sp + 16) * quads];
            const i32x4 c = src[static_cast<int64_t>(sp + 32) * quads], d = src[static_cast<int64_t>(sp + 48) * quads];
            sum += (a + b) + (c + d);
        }
        for (; sp < splits; sp += 16) sum += src[static_cast<int64_t>(sp) * quads];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) red[sl][vq][i] = sum[i];
    __syncthreads();
    if (sl == 0 && q < quads) {
        const float s = sA[0] * sB[0];
        const int64_t n = (q * 4) / Kp, k = q * 4 - n * Kp;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int t = 0;
#pragma unroll
            for (int w = 0; w < 16; ++w) t += red[w][vq][i];
            if (k + i < K) out[n * ldo + k + i] = s * static_cast<float>(t);
        }
    }
}

// ------------------------------------------------------------- host side
static int64_t round_up(int64_t v, int64_t m) { return (v + m - 1) / m * m; }

// Compute units of the current device (queried once; a fixed property of the machine).
static int compute_units() {
    static const int n = [] {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        return cus;
    }();
    return n;
}

// widest aligned access for 16-byte row pieces of an int8 matrix; `cols` bytes are meaningful
static int row_vec(const int8_t* p, int64_t ld, int64_t cols, int64_t* readable) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(p);
    if ((a & 15) == 0 && (ld & 15) == 0 && round_up(cols, 16) <= ld) {
        *readable = round_up(cols, 16);
        return 16;
    }
    if ((a & 3) == 0 && (ld & 3) == 0 && round_up(cols, 4) <= ld) {
        *readable = round_up(cols, 4);
        return 4;
    }
    *readable = cols;
    return 1;
}

constexpr size_t kLdsBytes = 160 * 1024;

// The stationary form (reduction <= 256, A rows readable in 4- or 16-byte pieces).  EPI: what the epilogue does
// with the dequantized tile (see gemm_nts_kernel).  False when the launch could not be set up.
template <int VEC, int EPI>
static bool launch_nts(const NtParams& p, hipStream_t s) {
    const int64_t n16 = ceil_div(p.N, 16);
    const int ksteps = static_cast<int>(ceil_div(p.Kr, 64));
    const int ntiles = static_cast<int>(ceil_div(p.M, 16));
    // One column block wherever the whole small operand fits the LDS (up to 38 tiles at four k-steps): a wave
    // then writes whole output rows, in two rounds of half the tiles over the A tile it holds.  Cutting the
    // columns over workgroups makes rows arrive in pieces from different compute units at different times, which
    // a store-only kernel of that shape shows at half the rate (232,960 x 608 fp32: 3.3 TB/s in three blocks of
    // 13 tiles against 6.6 TB/s for whole rows).  Wider outputs are cut into blocks of sixteen tiles, which meet
    // on 1 KB boundaries.
    const bool two_rounds = EPI == 0 && n16 > 16 && n16 <= 38 &&
                            n16 * (ksteps * 1024 + 64) + 256 <= static_cast<int64_t>(kLdsBytes);
    int ny = 1;
    int64_t nt = n16;
    if (!two_rounds && n16 > 16) {
        ny = static_cast<int>(ceil_div(n16, 16));
        nt = 16;
    }
#define TANGO_NTS(NT_, PASSES_)                                                                                 \
    do {                                                                                                        \
        constexpr int WAVES = 12;                                                                               \
        int gx = compute_units() / ny;                                                                          \
        if (gx > ceil_div(ntiles, WAVES)) gx = static_cast<int>(ceil_div(ntiles, WAVES));                       \
        if (gx < 1) gx = 1;                                                                                     \
        /* more than 64 KB of dynamic LDS has to be asked for once per kernel */                                \
        static const bool ok =                                                                                  \
            hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_nts_kernel<NT_, VEC, WAVES, EPI, PASSES_>), \
                                hipFuncAttributeMaxDynamicSharedMemorySize,                                     \
                                static_cast<int>(kLdsBytes - 256)) == hipSuccess;                               \
        if (!ok) return false;                                                                                  \
        hipLaunchKernelGGL((gemm_nts_kernel<NT_, VEC, WAVES, EPI, PASSES_>), dim3(gx, ny), dim3(64 * WAVES),    \
                           static_cast<size_t>(NT_ * PASSES_) * (ksteps * 1024 + 64), s, p, ntiles);           \
        return true;                                                                                            \
    } while (0)
    if constexpr (EPI == 3) {  // whole blocks of an even number of tiles only (the entry point admits no other shape)
        if (two_rounds || ny != 1) return false;
        if (nt == 2) TANGO_NTS(2, 1);
        else if (nt == 4) TANGO_NTS(4, 1);
        else if (nt == 8) TANGO_NTS(8, 1);
        else if (nt == 16) TANGO_NTS(16, 1);
        return false;
    } else {
    if (two_rounds) {
        if (nt <= 24) TANGO_NTS(12, (EPI == 0 ? 2 : 1));
        else if (nt <= 32) TANGO_NTS(16, (EPI == 0 ? 2 : 1));
        else TANGO_NTS(19, (EPI == 0 ? 2 : 1));
    }
    if (nt <= 2) TANGO_NTS(2, 1);
    else if (nt <= 4) TANGO_NTS(4, 1);
    else if (nt <= 8) TANGO_NTS(8, 1);
    else if (nt <= 13) TANGO_NTS(13, 1);
    else TANGO_NTS(16, 1);
    }
#undef TANGO_NTS
}

// The register-stationary form: fp32 output of 257 .. 960 columns (at most fifteen computing waves and the
// fetching one) with the plain epilogue, reduction <= 256, and
// enough row tiles to keep every compute unit busy for many rounds.
static bool launch_ntr(const NtParams& p, hipStream_t s) {
    const int64_t n16 = ceil_div(p.N, 16);
    const int64_t ntiles = ceil_div(p.M, 16);
    const uintptr_t ca = reinterpret_cast<uintptr_t>(p.C);
    if (n16 <= 16 || n16 > 60 || p.Kr > 256 || p.bias || p.accumulate || (ca & 15) != 0 || (p.ldc & 3) != 0 ||
        ntiles < 8 * compute_units() || ntiles > INT32_MAX)
        return false;
    // One workgroup per compute unit, the whole output row in it: cutting the columns over two to four workgroups
    // (more, smaller barrier groups per compute unit) was measured at 0.18 to 0.21 ms against 0.16 ms at
    // 232,965 x 256 -> 602, because the pieces of a row then reach memory at different times.
    const int waves = static_cast<int>(ceil_div(n16, 4)) + 1;  // the last one fetches
    const int gx = compute_units();
    if (p.Kr <= 128)
        hipLaunchKernelGGL((gemm_ntr_kernel<2>), dim3(gx), dim3(64 * waves), 0, s, p, static_cast<int>(ntiles));
    else
        hipLaunchKernelGGL((gemm_ntr_kernel<4>), dim3(gx), dim3(64 * waves), 0, s, p, static_cast<int>(ntiles));
    return true;
}

// False when the masked maximum was asked for and the stationary kernel, the only one that finds it, could not run.
template <int VEC>
static bool launch_nt_vec(const NtParams& p, hipStream_t s) {
    const int64_t n16 = ceil_div(p.N, 16);
    const unsigned gx = static_cast<unsigned>(ceil_div(p.M, 128));
    if (p.masked_absmax_out) return p.Kr <= 256 && VEC != 1 && launch_nts<VEC == 1 ? 4 : VEC, 3>(p, s);
    if (VEC == 16 && launch_ntr(p, s)) return true;  // A rows in aligned 16-byte pieces
#define TANGO_NT(NT_)                                                                             \
    hipLaunchKernelGGL((gemm_nt_kernel<NT_, VEC>), dim3(gx, static_cast<unsigned>(ceil_div(n16, NT_))), \
                       dim3(256), 0, s, p)
    if (p.Kr <= 256 && VEC != 1) {  // the small operand fits LDS: the stationary form
        if (launch_nts<VEC == 1 ? 4 : VEC, 0>(p, s)) return true;
    }
    if (n16 <= 1) TANGO_NT(1);
    else if (n16 <= 2) TANGO_NT(2);
    else if (n16 <= 3) TANGO_NT(3);
    else if (n16 <= 4) TANGO_NT(4);
    else if (n16 <= 8) TANGO_NT(8);
    else TANGO_NT(16);
#undef TANGO_NT
    return true;
}

// B must already be packed (16-byte aligned rows, zero-filled to a multiple of 64 columns).
// slot_zeroed: the caller has already zeroed absmax_out on this stream
static int launch_nt(NtParams p, hipStream_t s, bool slot_zeroed = false) {
    if (p.M == 0 || p.N == 0) return TANGO_OK;
    if (ceil_div(p.M, 128) > INT32_MAX) return TANGO_ERR_UNSUPPORTED;
    if (p.absmax_out && !slot_zeroed) fill_u32(p.absmax_out, 0u, 1, s);
    int64_t readable = 0;
    const int vec = row_vec(p.A, p.lda, p.Kr, &readable);
    p.a_row_bytes = readable;
    const bool done = vec == 16 ? launch_nt_vec<16>(p, s) : vec == 4 ? launch_nt_vec<4>(p, s) : launch_nt_vec<1>(p, s);
    return done ? launch_status() : TANGO_ERR_LAUNCH;
}

// The fused forward needs: a deterministic rounding mode, K <= 768 (the 64 x K int8 block and
// the per-lane staging registers are sized for it), Xq rows that are 16-byte aligned and cover
// round_up(K, 16) bytes, and X rows that are at least 8-byte aligned.
static bool fq_applicable(const float* X, int64_t ldx, const int8_t* Xq, int64_t ldxq, int64_t K,
                          int round_mode) {
    if (round_mode != TANGO_ROUND_RNE && round_mode != TANGO_ROUND_TRUNC) return false;
    if (K < 1 || K > 768) return false;
    if ((reinterpret_cast<uintptr_t>(Xq) & 15) != 0 || (ldxq & 15) != 0 || ldxq < round_up(K, 16)) return false;
    if ((reinterpret_cast<uintptr_t>(X) & 7) != 0 || (ldx & 1) != 0) return false;
    return true;
}

template <int NT, int XV, int MODE, int THREADS>
static bool launch_ws_nt(const FqParams& p, hipStream_t s) {
    const int kq = static_cast<int>(round_up(p.K, 16));
    int pitch = kq + 16;  // the extra chunk spreads the rows of a fragment read over the LDS banks
    if ((pitch >> 4) % 2 == 0) pitch += 16;  // an odd number of 16-byte units per row
    const size_t lds = static_cast<size_t>(16 * NT) * pitch;
    if (lds + 256 > kLdsBytes) return false;
    static const bool ok = [] {  // more than 64 KB of dynamic LDS has to be asked for once per kernel
        return hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_ws_kernel<NT, XV, MODE, THREADS>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize,
                                   static_cast<int>(kLdsBytes - 256)) == hipSuccess;
    }();
    if (!ok) return false;
    constexpr int WAVES = THREADS / 64;
    const int64_t nblocks = ceil_div(p.M, 16);
    const int64_t wgs = ceil_div(nblocks, WAVES) < compute_units() ? ceil_div(nblocks, WAVES) : compute_units();
    hipLaunchKernelGGL((gemm_ws_kernel<NT, XV, MODE, THREADS>), dim3(static_cast<unsigned>(wgs)), dim3(THREADS), lds, s, p,
                       static_cast<int>(nblocks), pitch, kq);
    return true;
}

// W-stationary form when X is tall (at least one 16-row block per wave of the machine) and N <= 32.  (Wider
// outputs were measured with this kernel too, eight or twelve waves per compute unit and 4 NT accumulator
// registers per lane: 232,965 x 602 x 256 0.336 ms against 0.29 ms for gemm_fq_kernel, x 256 x 41 0.098 against
// 0.080 ms.)
static bool ws_shape(int64_t M, int64_t N) {
    return N <= 32 && ceil_div(M, 16) >= 12LL * compute_units() && ceil_div(M, 16) <= INT32_MAX;
}

template <int XV, int MODE>
static bool launch_ws(const FqParams& p, hipStream_t s) {
    if (!ws_shape(p.M, p.N)) return false;
    if (p.N <= 16) return launch_ws_nt<1, XV, MODE, 768>(p, s);
    return launch_ws_nt<2, XV, MODE, 768>(p, s);
}

// Row pitch of the forward kernel's LDS block: K rounded up to an odd number of 16-byte units, so that the
// sixteen rows of a fragment read start in sixteen different bank quads.  The last k-step may read past a
// row's end (into the next row, or the 64 spare bytes after the block): those bytes meet the zero padding of
// the packed small operand, and any int8 times zero is zero.
static int fq_pitch(int64_t K) {
    const int64_t units = ceil_div(K, 16);
    return static_cast<int>(16 * (units | 1));
}

template <int XV, int MODE>
static void launch_fq_mode(const FqParams& p, hipStream_t s) {
    constexpr int RT = 4;  // 64 rows per workgroup measured faster than 32 at every benchmark shape
    if (!p.b_frag && launch_ws<XV, MODE>(p, s)) return;
    if (p.b_frag && p.N > 128 && p.N <= 256 && (p.kp == 640 || p.kp == 256) && p.ldxq <= p.pitch && p.K % 2 == 0 &&
        p.K > (p.kp == 640 ? 512 : 0) && ceil_div(p.M, 16) >= 8LL * compute_units() && ceil_div(p.M, 16) <= INT32_MAX) {
        const size_t lds = 2 * (static_cast<size_t>(16) * p.pitch + 64) + 256 * sizeof(float);
        const int nt = static_cast<int>(ceil_div(p.M, 16));
        const bool v4 = XV == 4 && p.K % 4 == 0;
#define TANGO_FQR(KS_)                                                                                              \
    do {                                                                                                            \
        if (v4) hipLaunchKernelGGL((gemm_fqr_kernel<KS_, 4, MODE>), dim3(compute_units()), dim3(1024), lds, s, p, nt); \
        else hipLaunchKernelGGL((gemm_fqr_kernel<KS_, 2, MODE>), dim3(compute_units()), dim3(1024), lds, s, p, nt);  \
    } while (0)
        if (p.kp == 640) TANGO_FQR(10);
        else TANGO_FQR(4);
#undef TANGO_FQR
        return;
    }
    const size_t lds = static_cast<size_t>(16 * RT) * p.pitch + 64 + 256 * sizeof(float);
    const unsigned gx = static_cast<unsigned>(ceil_div(p.M, 16 * RT));
#define TANGO_FQ_IT(TPW_, IT_)                                                                   \
    hipLaunchKernelGGL((gemm_fq_kernel<TPW_, XV, MODE, RT, IT_>),                                \
                       dim3(gx, static_cast<unsigned>(ceil_div(p.N, 64 * TPW_))), dim3(256), lds, s, p)
#define TANGO_FQ(TPW_)                                                   \
    do {                                                                 \
        if (p.kp <= 256) TANGO_FQ_IT(TPW_, 1);                           \
        else TANGO_FQ_IT(TPW_, 3);                                       \
    } while (0)
    if (p.N <= 64) TANGO_FQ(1);
    else if (p.N <= 128) TANGO_FQ(2);
    else TANGO_FQ(4);
#undef TANGO_FQ
#undef TANGO_FQ_IT
}

static int launch_fq(const FqParams& p, int round_mode, hipStream_t s, bool slot_zeroed = false) {
    if (ceil_div(p.M, 64) > INT32_MAX || ceil_div(p.N, 64) > 65535) return TANGO_ERR_UNSUPPORTED;
    if (p.absmax_out && !slot_zeroed) fill_u32(p.absmax_out, 0u, 1, s);
    const bool v4 = (reinterpret_cast<uintptr_t>(p.X) & 15) == 0 && (p.ldx & 3) == 0;
    if (round_mode == TANGO_ROUND_RNE) {
        if (v4) launch_fq_mode<4, TANGO_ROUND_RNE>(p, s); else launch_fq_mode<2, TANGO_ROUND_RNE>(p, s);
    } else {
        if (v4) launch_fq_mode<4, TANGO_ROUND_TRUNC>(p, s); else launch_fq_mode<2, TANGO_ROUND_TRUNC>(p, s);
    }
    return launch_status();
}

}  // namespace tango

using namespace tango;

// declared in quantize.hip
extern "C" int tango_quantize_rows_f32_i8(const float*, int64_t, int64_t, int64_t, const float*, int,
                                          int8_t*, int64_t, int, const float*, uint64_t, uint64_t,
                                          tango_stream_t);
extern "C" int tango_quantize_rows_ex_f32_i8(const float*, int64_t, int64_t, int64_t, const float*,
                                             const void*, int64_t, int, const float*, int, int8_t*, int64_t,
                                             int, const float*, uint64_t, uint64_t, const uint64_t*, tango_stream_t);
extern "C" int tango_absmax_f32(const float*, int64_t, float*, tango_stream_t);
extern "C" int tango_quantize_f32_i8(const float*, int64_t, const float*, int8_t*, int, const float*, uint64_t,
                                     uint64_t, const uint64_t*, tango_stream_t);

extern "C" {

size_t tango_qgemm_fwd_workspace(int64_t M, int64_t N, int64_t K) {
    (void)M;
    if (N <= 0 || K <= 0) return 0;
    return static_cast<size_t>(round_up(N, 16) * round_up(K, 64));  // rows to a multiple of 16: the fragment-order form
}

int tango_qgemm_fwd_ex(float* Y, int64_t ldy, const float* X, int64_t ldx, const float* x_row_mul, int8_t* Xq, int64_t ldxq,
                    const float* W, int64_t ldw, int8_t* Wq, const float* bias, float* scaleY,
                    const float* scaleX, const float* scaleW, int64_t M, int64_t N, int64_t K,
                    int round_mode, void* workspace, size_t workspace_bytes,
                    tango_stream_t stream) {
    if (M < 0 || N < 0 || K < 0 || !scaleX || !scaleW || ldy < N || (X && ldx < K) || ldw < K || ldxq < K)
        return TANGO_ERR_INVALID_ARG;
    if (M * N > 0 && !Y) return TANGO_ERR_INVALID_ARG;
    const bool cached = X == nullptr;  // Xq is an input: the caller has quantized X already
    if (M * K > 0 && !Xq) return TANGO_ERR_INVALID_ARG;
    if (cached && x_row_mul) return TANGO_ERR_INVALID_ARG;
    if (N * K > 0 && (!W || !Wq)) return TANGO_ERR_INVALID_ARG;
    // no seed / noise argument exists here, so stochastic rounding cannot be honoured: refuse it
    if (round_mode != TANGO_ROUND_RNE && round_mode != TANGO_ROUND_TRUNC) return TANGO_ERR_UNSUPPORTED;
    const size_t need = tango_qgemm_fwd_workspace(M, N, K);
    if (need > 0 && (!workspace || workspace_bytes < need)) return TANGO_ERR_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(workspace) & 15) != 0) return TANGO_ERR_INVALID_ARG;
    hipStream_t s = as_stream(stream);
    const bool fused = !cached && M > 0 && N > 0 && fq_applicable(X, ldx, Xq, ldxq, K, round_mode);
    int rc = TANGO_OK;
    if (!fused && !cached) {
        rc = tango_quantize_rows_ex_f32_i8(X, M, K, ldx, x_row_mul, nullptr, 0, 0, scaleX, 0, Xq, ldxq, round_mode,
                                           nullptr, 0, 0, nullptr, stream);
        if (rc != TANGO_OK) return rc;
    }
    int8_t* Bp = static_cast<int8_t*>(workspace);
    const int64_t ldb = round_up(K, 64);
    // the fused kernel reads the small operand fragment by fragment; the W-stationary one (narrow outputs) and the
    // kernels for an int8 X stage its rows through LDS
    const int frag = fused && !ws_shape(M, N);
    if (N > 0 && K > 0) {  // W -> Wq and its packed copy, and the zeroing of scaleY, in one launch
        const dim3 wgrid(grid_for(round_up(N, 16) * ldb, 256));
        if (round_mode == TANGO_ROUND_RNE)
            hipLaunchKernelGGL(quantize_pack_w_kernel<TANGO_ROUND_RNE>, wgrid, dim3(256), 0, s, W, ldw, scaleW, Wq, Bp,
                               ldb, N, K, scaleY, frag);
        else
            hipLaunchKernelGGL(quantize_pack_w_kernel<TANGO_ROUND_TRUNC>, wgrid, dim3(256), 0, s, W, ldw, scaleW, Wq, Bp,
                               ldb, N, K, scaleY, frag);
    } else if (scaleY) {
        fill_u32(scaleY, 0u, 1, s);
    }
    if (M == 0 || N == 0) return launch_status();
    if (fused) {
        FqParams q{};
        q.C = Y; q.X = X; q.Xq = Xq; q.B = Bp; q.bias = bias; q.x_row_mul = x_row_mul; q.absmax_out = scaleY;
        q.sA = scaleX; q.sB = scaleW; q.M = M; q.N = N; q.K = K; q.ldx = ldx; q.ldxq = ldxq; q.ldb = ldb;
        q.ldc = ldy; q.kp = static_cast<int>(ldb); q.pitch = fq_pitch(K); q.b_frag = frag;
        return launch_fq(q, round_mode, s, true);
    }
    NtParams p{};
    p.C = Y; p.A = Xq; p.B = Bp; p.bias = bias; p.absmax_out = scaleY; p.sA = scaleX; p.sB = scaleW;
    p.M = M; p.N = N; p.Kr = K; p.lda = ldxq; p.ldb = ldb; p.ldc = ldy;
    return launch_nt(p, s, true);
}

int tango_qgemm_fwd_q8(int8_t* Yq, int64_t ldyq, float* scaleY, const int8_t* Xq, int64_t ldxq, const float* W,
                       int64_t ldw, int8_t* Wq, const float* bias, const float* scaleX, const float* scaleW,
                       int64_t M, int64_t N, int64_t K, int round_mode, void* workspace, size_t workspace_bytes,
                       tango_stream_t stream) {
    if (M < 0 || N < 0 || K < 0 || !scaleX || !scaleW || !scaleY || ldyq < N || ldw < K || ldxq < K)
        return TANGO_ERR_INVALID_ARG;
    if ((M * N > 0 && !Yq) || (M * K > 0 && !Xq) || (N * K > 0 && (!W || !Wq))) return TANGO_ERR_INVALID_ARG;
    if (round_mode != TANGO_ROUND_RNE && round_mode != TANGO_ROUND_TRUNC) return TANGO_ERR_UNSUPPORTED;
    if (K < 1 || K > 256 || ceil_div(M, 16) > INT32_MAX) return TANGO_ERR_UNSUPPORTED;  // the stationary form only
    int64_t readable = 0;
    if (M > 0 && row_vec(Xq, ldxq, K, &readable) != 16) return TANGO_ERR_UNSUPPORTED;
    const size_t need = tango_qgemm_fwd_workspace(M, N, K);
    if (need > 0 && (!workspace || workspace_bytes < need)) return TANGO_ERR_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(workspace) & 15) != 0) return TANGO_ERR_INVALID_ARG;
    hipStream_t s = as_stream(stream);
    int8_t* Bp = static_cast<int8_t*>(workspace);
    const int64_t ldb = round_up(K, 64);
    if (N > 0) {  // W -> Wq and its packed copy, and the zeroing of scaleY, in one launch
        const dim3 wgrid(grid_for(N * ldb, 256));
        if (round_mode == TANGO_ROUND_RNE)
            hipLaunchKernelGGL(quantize_pack_w_kernel<TANGO_ROUND_RNE>, wgrid, dim3(256), 0, s, W, ldw, scaleW, Wq, Bp,
                               ldb, N, K, scaleY, 0);
        else
            hipLaunchKernelGGL(quantize_pack_w_kernel<TANGO_ROUND_TRUNC>, wgrid, dim3(256), 0, s, W, ldw, scaleW, Wq, Bp,
                               ldb, N, K, scaleY, 0);
    } else {
        fill_u32(scaleY, 0u, 1, s);
    }
    if (M == 0 || N == 0) return launch_status();
    NtParams p{};
    p.A = Xq; p.B = Bp; p.bias = bias; p.absmax_out = scaleY; p.sA = scaleX; p.sB = scaleW;
    p.M = M; p.N = N; p.Kr = K; p.lda = ldxq; p.ldb = ldb; p.a_row_bytes = readable;
    // the product twice: first only its absmax, then, with the scale known, rounded straight to int8
    if (!launch_nts<16, 1>(p, s)) return TANGO_ERR_UNSUPPORTED;
    p.absmax_out = nullptr; p.Cq = Yq; p.ldcq = ldyq; p.q_scale = scaleY; p.q_mode = round_mode;
    if (!launch_nts<16, 2>(p, s)) return TANGO_ERR_UNSUPPORTED;
    return launch_status();
}

int tango_qgemm_fwd(float* Y, int64_t ldy, const float* X, int64_t ldx, int8_t* Xq, int64_t ldxq,
                    const float* W, int64_t ldw, int8_t* Wq, const float* bias, float* scaleY,
                    const float* scaleX, const float* scaleW, int64_t M, int64_t N, int64_t K,
                    int round_mode, void* workspace, size_t workspace_bytes,
                    tango_stream_t stream) {
    return tango_qgemm_fwd_ex(Y, ldy, X, ldx, nullptr, Xq, ldxq, W, ldw, Wq, bias, scaleY, scaleX, scaleW, M, N,
                              K, round_mode, workspace, workspace_bytes, stream);
}

size_t tango_qgemm_i8_nt_workspace(int64_t M, int64_t N, int64_t K) {
    return tango_qgemm_fwd_workspace(M, N, K);
}

int tango_qgemm_i8_nt(float* Y, int64_t ldy, const int8_t* A, int64_t lda, const int8_t* B,
                      int64_t ldb, const float* bias, float* scaleY, const float* sA,
                      const float* sB, int64_t M, int64_t N, int64_t K, void* workspace,
                      size_t workspace_bytes, tango_stream_t stream) {
    if (M < 0 || N < 0 || K < 0 || !sA || !sB || ldy < N || lda < K || ldb < K)
        return TANGO_ERR_INVALID_ARG;
    if ((M * N > 0 && !Y) || (M * K > 0 && !A) || (N * K > 0 && !B)) return TANGO_ERR_INVALID_ARG;
    if (M == 0 || N == 0) return TANGO_OK;
    hipStream_t s = as_stream(stream);
    NtParams p{};
    p.C = Y; p.A = A; p.bias = bias; p.absmax_out = scaleY; p.sA = sA; p.sB = sB;
    p.M = M; p.N = N; p.Kr = K; p.lda = lda; p.ldc = ldy;
    const size_t need = tango_qgemm_fwd_workspace(M, N, K);
    if (need > 0 && (!workspace || workspace_bytes < need)) return TANGO_ERR_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(workspace) & 15) != 0) return TANGO_ERR_INVALID_ARG;
    int8_t* Bp = static_cast<int8_t*>(workspace);
    const int64_t ldp = round_up(K, 64);
    if (K > 0)
        hipLaunchKernelGGL(pack_rows_i8_kernel, dim3(grid_for(N * ldp, 256)), dim3(256), 0, s, Bp, ldp,
                           B, ldb, N, K);
    p.B = Bp; p.ldb = ldp;
    return launch_nt(p, s);
}

size_t tango_qgemm_bwd_dx_workspace(int64_t M, int64_t N, int64_t K) {
    (void)M;
    if (N <= 0 || K <= 0) return 0;
    return static_cast<size_t>(K * round_up(N, 64));
}

int tango_qgemm_bwd_dx_ex(float* dX, int64_t lddx, const int8_t* dYq, int64_t lddy,
                          const int8_t* Wq, int64_t ldw, const float* s_dY, const float* s_W,
                          const float* row_scale, int accumulate,
                       int64_t M, int64_t N, int64_t K, void* workspace, size_t workspace_bytes,
                       tango_stream_t stream) {
    if (M < 0 || N < 0 || K < 0 || !s_dY || !s_W || lddx < K || lddy < N || ldw < K)
        return TANGO_ERR_INVALID_ARG;
    if ((M * K > 0 && !dX) || (M * N > 0 && !dYq) || (N * K > 0 && !Wq)) return TANGO_ERR_INVALID_ARG;
    if (M == 0 || K == 0) return TANGO_OK;
    const size_t need = tango_qgemm_bwd_dx_workspace(M, N, K);
    if (need > 0 && (!workspace || workspace_bytes < need)) return TANGO_ERR_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(workspace) & 15) != 0) return TANGO_ERR_INVALID_ARG;
    hipStream_t s = as_stream(stream);
    // W^T packed as [K, N padded to 64]: the small operand of an NT product with reduction N
    int8_t* Wt = static_cast<int8_t*>(workspace);
    const int64_t ldt = round_up(N, 64);
    if (N > 0)
        hipLaunchKernelGGL(transpose_pack_i8_kernel, dim3(grid_for(K * ldt, 256)), dim3(256), 0, s, Wt,
                           ldt, Wq, ldw, N, K);
    NtParams p{};
    p.C = dX; p.A = dYq; p.B = Wt; p.sA = s_dY; p.sB = s_W; p.row_scale = row_scale; p.accumulate = accumulate;
    p.M = M; p.N = K; p.Kr = N; p.lda = lddy; p.ldb = ldt; p.ldc = lddx;
    return launch_nt(p, s);
}

int tango_qgemm_bwd_dx_masked(float* dX, int64_t lddx, const int8_t* dYq, int64_t lddy, const int8_t* Wq,
                              int64_t ldw, const float* s_dY, const float* s_W, const float* row_scale,
                              const uint16_t* mask_bits, int64_t ldmask, const float* mask_mul,
                              float* masked_scale_out, int64_t M, int64_t N, int64_t K, void* workspace,
                              size_t workspace_bytes, tango_stream_t stream) {
    if (M < 0 || N < 0 || K < 0 || !s_dY || !s_W || lddx < K || lddy < N || ldw < K || !mask_bits ||
        !masked_scale_out || ldmask < K / 16)
        return TANGO_ERR_INVALID_ARG;
    if ((M * K > 0 && !dX) || (M * N > 0 && !dYq) || (N * K > 0 && !Wq)) return TANGO_ERR_INVALID_ARG;
    // the shapes whose launch is the stationary kernel over whole blocks of an even number of 16-column tiles
    int64_t readable = 0;
    const bool ok = (K == 32 || K == 64 || K == 128 || K == 256) && N >= 1 && N <= 256 && M > 0 &&
                    row_vec(dYq, lddy, N, &readable) != 1 && (reinterpret_cast<uintptr_t>(dX) & 15) == 0 &&
                    (lddx & 3) == 0 && (ldmask & 1) == 0 && (reinterpret_cast<uintptr_t>(mask_bits) & 3) == 0;
    if (!ok) return TANGO_ERR_UNSUPPORTED;
    const size_t need = tango_qgemm_bwd_dx_workspace(M, N, K);
    if (need > 0 && (!workspace || workspace_bytes < need)) return TANGO_ERR_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(workspace) & 15) != 0) return TANGO_ERR_INVALID_ARG;
    hipStream_t s = as_stream(stream);
    int8_t* Wt = static_cast<int8_t*>(workspace);
    const int64_t ldt = round_up(N, 64);
    hipLaunchKernelGGL(transpose_pack_i8_kernel, dim3(grid_for(K * ldt, 256)), dim3(256), 0, s, Wt, ldt, Wq, ldw, N, K);
    fill_u32(masked_scale_out, 0u, 1, s);
    NtParams p{};
    p.C = dX; p.A = dYq; p.B = Wt; p.sA = s_dY; p.sB = s_W; p.row_scale = row_scale;
    p.M = M; p.N = K; p.Kr = N; p.lda = lddy; p.ldb = ldt; p.ldc = lddx;
    p.mask_bits = mask_bits; p.ldmask = ldmask; p.mask_mul = mask_mul; p.masked_absmax_out = masked_scale_out;
    return launch_nt(p, s);
}

int tango_qgemm_bwd_dx(float* dX, int64_t lddx, const int8_t* dYq, int64_t lddy,
                       const int8_t* Wq, int64_t ldw, const float* s_dY, const float* s_W,
                       int64_t M, int64_t N, int64_t K, void* workspace, size_t workspace_bytes,
                       tango_stream_t stream) {
    return tango_qgemm_bwd_dx_ex(dX, lddx, dYq, lddy, Wq, ldw, s_dY, s_W, nullptr, 0, M, N, K, workspace,
                                 workspace_bytes, stream);
}

// How the reduction over M is cut: `splits` chunks of `chunk` rows (a multiple of 64).
struct TnPlan {
    int tiles_n, tiles_k;
    int64_t splits, chunk, Kp;
};

static TnPlan tn_plan(int64_t M, int64_t N, int64_t K, int64_t workgroups = 768) {
    TnPlan t{};
    t.tiles_n = static_cast<int>(ceil_div(N, 128));
    t.tiles_k = static_cast<int>(ceil_div(K, 128));
    t.Kp = round_up(K, 4);
    const int64_t tiles = static_cast<int64_t>(t.tiles_n) * t.tiles_k;
    // enough workgroups for `workgroups` / 256 per CU, each with at least 4 reduction steps ...
    int64_t splits = workgroups == 768 ? ceil_div(workgroups, tiles) : workgroups / tiles;  // the ring kernel: no partial second round
    const int64_t max_splits = ceil_div(M, 256);
    if (splits > max_splits) splits = max_splits;
    // ... but the slabs (written once, read once, 4 bytes each way) stay below the operand bytes
    const int64_t by_traffic = M * (N + K) / (8 * N * t.Kp);
    if (splits > by_traffic) splits = by_traffic;
    if (splits < 1) splits = 1;
    if (workgroups != 768) {
        // A number of workgroups that is a multiple of eight: the kernel then gives each XCD a contiguous range of
        // them, so that the tiles that share a chunk of rows meet in one L2 (232,965 x 256 x 602: 71 us with 480
        // workgroups, 128 us with 510)
        int64_t s8 = splits;
        while (s8 > 1 && (s8 * tiles) % 8 != 0) --s8;
        if ((s8 * tiles) % 8 == 0) splits = s8;
    }
    t.chunk = round_up(ceil_div(M, splits), 64);
    t.splits = M > 0 ? ceil_div(M, t.chunk) : 0;
    return t;
}

size_t tango_qgemm_bwd_dw_workspace(int64_t M, int64_t N, int64_t K) {
    if (N <= 0 || K <= 0 || M < 0) return 0;
    const TnPlan t = tn_plan(M, N, K);
    return static_cast<size_t>((t.splits > 0 ? t.splits : 1) * N * t.Kp) * sizeof(int);
}

int tango_qgemm_bwd_dw(float* dW, int64_t lddw, const int8_t* dYq, int64_t lddy,
                       const int8_t* Xq, int64_t ldx, const float* s_dY, const float* s_X,
                       int64_t M, int64_t N, int64_t K, void* workspace, size_t workspace_bytes,
                       tango_stream_t stream) {
    if (M < 0 || N < 0 || K < 0 || !s_dY || !s_X || lddw < K || lddy < N || ldx < K)
        return TANGO_ERR_INVALID_ARG;
    if ((N * K > 0 && !dW) || (M * N > 0 && !dYq) || (M * K > 0 && !Xq)) return TANGO_ERR_INVALID_ARG;
    if (N == 0 || K == 0) return TANGO_OK;
    const size_t need = tango_qgemm_bwd_dw_workspace(M, N, K);
    if (!workspace || workspace_bytes < need) return TANGO_ERR_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(workspace) & 15) != 0) return TANGO_ERR_INVALID_ARG;
    hipStream_t s = as_stream(stream);
    int* acc = static_cast<int*>(workspace);
    int64_t ra = 0, rb = 0;
    const int va = row_vec(dYq, lddy, N, &ra), vb = row_vec(Xq, ldx, K, &rb);
    const int vec = va < vb ? va : vb;
    // the ring kernel holds 64 KB of LDS per workgroup, two per CU: fewer, longer splits than the workspace was
    // sized for (never more)
    const TnPlan t = vec == 16 ? tn_plan(M, N, K, 512) : tn_plan(M, N, K);
    if (M > 0) {
        TnParams p{};
        p.acc = acc; p.Kp = t.Kp; p.A = dYq; p.B = Xq; p.M = M; p.N = N; p.K = K; p.lda = lddy; p.ldb = ldx;
        p.tiles_n = t.tiles_n;
        p.tiles_k = t.tiles_k;
        const int64_t tiles = static_cast<int64_t>(p.tiles_n) * p.tiles_k;
        p.chunk = t.chunk;
        p.splits = static_cast<int>(t.splits);
        if (tiles * t.splits > INT32_MAX) return TANGO_ERR_UNSUPPORTED;
        p.a_row_bytes = (vec == 16) ? round_up(N, 16) : (vec == 4 ? round_up(N, 4) : N);
        p.b_row_bytes = (vec == 16) ? round_up(K, 16) : (vec == 4 ? round_up(K, 4) : K);
        const dim3 grid(static_cast<unsigned>(tiles * t.splits));
        if (vec == 16) hipLaunchKernelGGL(gemm_tn_tr_kernel, grid, dim3(256), 0, s, p);
        else if (vec == 4) hipLaunchKernelGGL(gemm_tn_kernel<4>, grid, dim3(256), 0, s, p);
        else hipLaunchKernelGGL(gemm_tn_kernel<1>, grid, dim3(256), 0, s, p);
    }
    const int64_t quads = N * t.Kp / 4;
    hipLaunchKernelGGL(tn_reduce_kernel, dim3(static_cast<unsigned>(ceil_div(quads, 16))), dim3(256), 0, s, dW, lddw,
                       acc, N, K, t.Kp, static_cast<int>(t.splits), s_dY, s_X);
    return launch_status();
}

// Workspace layout of the legacy path: two scales (16 bytes), Aq packed [m, k64], Bq packed [n, k64],
// and a dense staging copy of the larger quantized operand before packing / transposing.
size_t tango_qgemm_legacy_workspace(int64_t m, int64_t n, int64_t k) {
    if (m <= 0 || n <= 0 || k <= 0) return 16;
    const int64_t k64 = round_up(k, 64);
    const int64_t big = (m > n ? m : n) * k;
    return static_cast<size_t>(16 + round_up(m * k64, 16) + round_up(n * k64, 16) + round_up(big, 16));
}

int tango_qgemm_legacy(float* C, const float* A, const float* B, int64_t m, int64_t n, int64_t k,
                       int trans_a, int trans_b, void* workspace, size_t workspace_bytes,
                       tango_stream_t stream) {
    if (m < 0 || n < 0 || k < 0) return TANGO_ERR_INVALID_ARG;
    if (m * n == 0) return TANGO_OK;
    if (!C || (k > 0 && (!A || !B))) return TANGO_ERR_INVALID_ARG;
    const size_t need = tango_qgemm_legacy_workspace(m, n, k);
    if (!workspace || workspace_bytes < need) return TANGO_ERR_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(workspace) & 15) != 0) return TANGO_ERR_INVALID_ARG;
    hipStream_t s = as_stream(stream);
    const int64_t k64 = round_up(k, 64);
    int8_t* base = static_cast<int8_t*>(workspace);
    float* scales = reinterpret_cast<float*>(base);
    int8_t* Ap = base + 16;
    int8_t* Bp = Ap + round_up(m * k64, 16);
    int8_t* tmp = Bp + round_up(n * k64, 16);
    int rc;
    if ((rc = tango_absmax_f32(A, m * k, scales, stream)) != TANGO_OK) return rc;
    if ((rc = tango_absmax_f32(B, n * k, scales + 1, stream)) != TANGO_OK) return rc;
    // A as stored is [m,k] (or [k,m]); quantize densely, then pack (or transpose-pack) to [m, k64]
    rc = tango_quantize_f32_i8(A, m * k, scales, tmp, TANGO_ROUND_RNE, nullptr, 0, 0, nullptr, stream);
    if (rc != TANGO_OK) return rc;
    if (trans_a)
        hipLaunchKernelGGL(transpose_pack_i8_kernel, dim3(grid_for(m * k64, 256)), dim3(256), 0, s, Ap, k64, tmp, m, k, m);
    else
        hipLaunchKernelGGL(pack_rows_i8_kernel, dim3(grid_for(m * k64, 256)), dim3(256), 0, s, Ap, k64, tmp, k, m, k);
    rc = tango_quantize_f32_i8(B, n * k, scales + 1, tmp, TANGO_ROUND_RNE, nullptr, 0, 0, nullptr, stream);
    if (rc != TANGO_OK) return rc;
    if (trans_b)  // stored [n,k]
        hipLaunchKernelGGL(pack_rows_i8_kernel, dim3(grid_for(n * k64, 256)), dim3(256), 0, s, Bp, k64, tmp, k, n, k);
    else  // stored [k,n]
        hipLaunchKernelGGL(transpose_pack_i8_kernel, dim3(grid_for(n * k64, 256)), dim3(256), 0, s, Bp, k64, tmp, n, k, n);
    NtParams p{};
    p.C = C; p.A = Ap; p.B = Bp; p.sA = scales; p.sB = scales + 1;
    p.M = m; p.N = n; p.Kr = k; p.lda = k64; p.ldb = k64; p.ldc = n;
    return launch_nt(p, s);
}

}  // extern "C"
