// Dense blocks of a power-law adjacency on the CDNA4 matrix cores (v_mfma_i32_32x32x32_i8).
//
// With rows and columns ranked by falling slot count, the cells (row rank i, column rank j) whose
// expected density deg(i) * cnt(j) / nnz is above about one per cent form a staircase in the corner of the
// adjacency that holds a third to a half of all edges of such a graph.  There one bit per cell and a
// 0/1-byte x int8 matrix product cost less than one gathered 128-byte line per edge.  Per launch:
//   dense_stage_kernel   gathers the ranked columns' feature rows and writes them transposed, in the
//                        order the matrix instruction's second operand wants them (one KB per fragment);
//                        its last workgroups zero the partial sums of row blocks that several workgroups add into;
//   dense_block_kernel   two persistent 4-wave workgroups per CU walk their segments (row block, range of
//                        256-column units): a unit's staged features go from global memory straight into one
//                        of two LDS chunks, the mask bits come straight from memory (one dword per lane and
//                        k-step = two operand fragments after a shift and an AND per dword), a wave owns a
//                        128 x 64 (narrow features: 64 x 64) tile in accumulator registers and leaves it as
//                        int32 partial sums.
// The gather kernels of spmm.hip then add those partial sums in their epilogue.  Integer arithmetic
// throughout: the result does not depend on how the adjacency was split.
#include "spmm_dense.hpp"

namespace tango {

typedef int i32x16v __attribute__((ext_vector_type(16)));

struct DenseParams {
    const uint32_t* mask;
    const int64_t* mask_off;
    const int32_t* seg_ptr;
    const int32_t* segs;
    const int32_t* shared_blocks;
    const int32_t* col_ids;
    const int8_t* feat;
    int64_t ldf;
    int64_t fbytes;  // bytes of a feature row that may be read: F rounded up to 16
    int8_t* xt;      // staged features
    int* part;       // [dense_rows][npad]
    int npad;
    int64_t units;   // dense_cols / 256
    int64_t stage_groups;  // workgroups of the staging kernel that stage (64 columns each); the rest zero
};

// blockDim.x = 256; workgroup b stages mask columns 64 b .. 64 b + 63 (two k-steps of 32).
// Output order: column split q (SPLIT of them, NCTW 32-column tiles each), k-step s, tile ct of the split,
// lane l, 16 bytes: byte t of (((q * ksteps + s) * NCTW + ct) * 64 + l) * 16 is feature
// 32 (q * NCTW + ct) + l % 32 of column 32 s + 16 (l / 32) + t.
template <int NPAD, int NCTW>
__global__ __launch_bounds__(256) void dense_stage_kernel(const DenseParams p) {
    constexpr int CPR = NPAD / 16;  // 16-byte chunks per staged row
    __shared__ __attribute__((aligned(16))) uint32_t tile[64 * (NPAD / 4)];
    const int t = threadIdx.x;
    if (static_cast<int64_t>(blockIdx.x) >= p.stage_groups) {
        // the workgroups behind the staging ones zero the partial sums of the row blocks that several workgroups
        // of the block kernel add into (one launch less than a kernel of their own)
        const int64_t rb = p.shared_blocks[blockIdx.x - p.stage_groups];
        i32x4* dst = reinterpret_cast<i32x4*>(p.part + rb * kDenseRows * p.npad);
        const int n = kDenseRows * p.npad / 4;
        for (int i = t; i < n; i += 256) dst[i] = i32x4{0, 0, 0, 0};
        return;
    }
    const int64_t j0 = static_cast<int64_t>(blockIdx.x) * 64;
    const int64_t ksteps = p.stage_groups * 2;
    for (int c = t; c < 64 * CPR; c += 256) {
        const int r = c / CPR, cc = c - r * CPR;
        const int id = p.col_ids[j0 + r];
        u32x4 v{0u, 0u, 0u, 0u};
        if (id >= 0 && 16 * (cc + 1) <= p.fbytes)
            v = *reinterpret_cast<const u32x4*>(p.feat + static_cast<int64_t>(id) * p.ldf + 16 * cc);
        *reinterpret_cast<u32x4*>(&tile[r * (NPAD / 4) + 4 * cc]) = v;
    }
    __syncthreads();
    // item = (feature quad fq, group of 16 columns jg): sixteen dwords in, four 16-byte pieces out
    for (int it = t; it < NPAD; it += 256) {
        const int fq = it % (NPAD / 4), jg = it / (NPAD / 4);
        uint32_t r[16];
#pragma unroll
        for (int k = 0; k < 16; ++k) r[k] = tile[(16 * jg + k) * (NPAD / 4) + fq];
        uint32_t c[4][4];
#pragma unroll
        for (int tb = 0; tb < 4; ++tb) transpose4x4(r[4 * tb], r[4 * tb + 1], r[4 * tb + 2], r[4 * tb + 3], c[tb]);
        const int64_t s = (j0 >> 5) + (jg >> 1);
        const int g = jg & 1;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int f = 4 * fq + i;
            const int ct = f >> 5, l = (f & 31) + 32 * g;
            const int q = ct / NCTW, ctl = ct - q * NCTW;
            int8_t* dst = p.xt + (((q * ksteps + s) * NCTW + ctl) * 64 + l) * 16;
            *reinterpret_cast<u32x4*>(dst) = u32x4{c[0][i], c[1][i], c[2][i], c[3][i]};
        }
    }
}

// blockDim.x = 256 (4 waves), grid (groups, SPLIT): with one split the plan's finer table of segments is used
// (twice the groups), so that either way two workgroups per CU are in flight.  A workgroup owns 256 rows x 32 NCTW columns of a segment.
// RW = 4: wave w owns rows 128 (w / 2) .. + 127 and half of those column tiles, so that a feature fragment
// read from LDS feeds four matrix instructions; RW = 2 (narrow features): rows 64 w .. + 63 and every column
// tile, so that the bits of a mask word, which cost more instructions to expand than a fragment read, feed
// as many matrix instructions as there are column tiles.  Dynamic LDS: two chunks of 8 NCTW KB; two workgroups share a CU, so
// that one multiplies while the other waits for its next chunk.
template <int NCTW, int SPLIT, int RW>
__global__ __launch_bounds__(256, 2) void dense_block_kernel(const DenseParams p) {
    constexpr int CHUNK = 8 * NCTW * 1024;  // staged bytes of one unit and split
    constexpr int PASSES = CHUNK / (256 * 16);
    constexpr int CT = NCTW * 2 / RW;  // column tiles of a wave
    constexpr int RG = RW / 2;         // 64-row groups of a wave
    // Two chunks, as two objects: the compiler then knows that the loads that fill one do not touch the one
    // the fragment reads come from, and does not make those reads wait for the loads.
    __shared__ __attribute__((aligned(16))) int8_t chunk_a[CHUNK];
    __shared__ __attribute__((aligned(16))) int8_t chunk_b[CHUNK];
    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int rgrp = RW == 4 ? wave >> 1 : wave, cgrp = RW == 4 ? wave & 1 : 0;
    // Workgroups go to the eight XCDs round-robin by their linear id.  A column split is bound to 8 / SPLIT of them, so
    // that an XCD's L2 only has to hold that split's share of the staged features (every row block reads all of it).
    int q = blockIdx.y, grp = blockIdx.x;  // column split, group of segments
    if (SPLIT > 1 && (gridDim.x & 7) == 0) {
        constexpr int PER = 8 / SPLIT;
        const int lin = blockIdx.y * gridDim.x + blockIdx.x, xcd = lin & 7;
        q = xcd / PER;
        grp = (lin >> 3) * PER + xcd % PER;
    }
    const int sg0 = p.seg_ptr[grp], sg1 = p.seg_ptr[grp + 1];
    const u32x4* xsrc = reinterpret_cast<const u32x4*>(p.xt + static_cast<int64_t>(q) * p.units * CHUNK) + t;
    // The staged chunk of unit u goes from global memory straight into LDS (no registers, no LDS store instructions,
    // which cost this loop a third of its rate): each wave instruction lands 64 lanes x 16 bytes at a wave-uniform
    // LDS address, in the order they sit in global memory.
    auto stage = [&](int8_t* chunk, int64_t u) {
        const u32x4* x = xsrc + u * (CHUNK / 16);
#pragma unroll
        for (int i = 0; i < PASSES; ++i)
            __builtin_amdgcn_global_load_lds(x + i * 256, reinterpret_cast<u32x4*>(chunk) + i * 256 + wave * 64, 16, 0, 0);
    };
    for (int sg = sg0; sg < sg1; ++sg) {
        const int rb = p.segs[4 * sg], u0 = p.segs[4 * sg + 1], nu = p.segs[4 * sg + 2], shared = p.segs[4 * sg + 3];
        i32x16v acc[CT][RW];
#pragma unroll
        for (int c = 0; c < CT; ++c)
#pragma unroll
            for (int h = 0; h < RW; ++h)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[c][h][v] = 0;
        // this wave's mask words of unit u: two row groups of 64 rows, two 16-byte loads per lane each
        const u32x4* mrow = reinterpret_cast<const u32x4*>(p.mask + p.mask_off[rb]) + rgrp * (128 * RG) + lane;
        u32x4 mw[RG][2], mnext[RG][2];
        // first unit of the segment: every wave is past the barrier that ended the previous segment's last unit,
        // so nobody reads either chunk any more
        stage(chunk_a, u0);
#pragma unroll
        for (int g = 0; g < RG; ++g)
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) mw[g][hf] = mrow[static_cast<int64_t>(u0) * 512 + g * 128 + hf * 64];
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the chunk has landed in LDS
        __syncthreads();
        // One unit: ask for the next unit's chunk (into the chunk nobody reads now) and mask words, multiply this
        // one, wait for what was asked for (long since there), barrier.  The last unit asks for itself again: every
        // load is unconditional, so that the compiler waits for them behind the products and not at a join in front.
        auto unit = [&](const int8_t* cur, int8_t* nxt, int k) {
            const int64_t un = u0 + (k + 1 < nu ? k + 1 : k);
            stage(nxt, un);
#pragma unroll
            for (int g = 0; g < RG; ++g)
#pragma unroll
                for (int hf = 0; hf < 2; ++hf) mnext[g][hf] = mrow[un * 512 + g * 128 + hf * 64];
            __builtin_amdgcn_sched_barrier(0);  // the loads stay in front of the products, their use behind them
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                i32x4 mf[RW];
#pragma unroll
                for (int g = 0; g < RG; ++g) {
                    const uint32_t word = mw[g][s >> 2][s & 3];
#pragma unroll
                    for (int h = 0; h < 2; ++h)
#pragma unroll
                        for (int w = 0; w < 4; ++w)
                            mf[2 * g + h][w] = static_cast<int>((word >> (4 * h + w)) & 0x01010101u);
                }
#pragma unroll
                for (int c = 0; c < CT; ++c) {
                    const i32x4 ff = *reinterpret_cast<const i32x4*>(cur + ((s * NCTW + cgrp * CT + c) * 64 + lane) * 16);
#pragma unroll
                    for (int h = 0; h < RW; ++h)
                        acc[c][h] = __builtin_amdgcn_mfma_i32_32x32x32_i8(mf[h], ff, acc[c][h], 0, 0, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
#pragma unroll
            for (int g = 0; g < RG; ++g)
#pragma unroll
                for (int hf = 0; hf < 2; ++hf) mw[g][hf] = mnext[g][hf];
            __syncthreads();  // the next chunk is in place and nobody reads the current one any more
        };
        for (int k = 0; k < nu; k += 2) {
            unit(chunk_a, chunk_b, k);
            if (k + 1 < nu) unit(chunk_b, chunk_a, k + 1);
        }
        // the mask is the instruction's first operand, so accumulator v of tile (c, h) is row
        // 8 (v / 4) + 4 (lane / 32) + v % 4, column lane % 32 of the tile: a store covers 128 bytes of two rows
#pragma unroll
        for (int c = 0; c < CT; ++c)
#pragma unroll
            for (int h = 0; h < RW; ++h) {
                const int64_t row0 = static_cast<int64_t>(rb) * kDenseRows + rgrp * (32 * RW) + h * 32 + 4 * (lane >> 5);
                int* dst = p.part + row0 * p.npad + (q * NCTW + cgrp * CT + c) * 32 + (lane & 31);
                if (shared) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) atomicAdd(dst + (8 * (v >> 2) + (v & 3)) * p.npad, acc[c][h][v]);
                } else {
#pragma unroll
                    for (int v = 0; v < 16; ++v) dst[(8 * (v >> 2) + (v & 3)) * p.npad] = acc[c][h][v];
                }
            }
    }
}

// One wavefront per row of the adjacency; blockDim.x = 256.
__global__ __launch_bounds__(256) void dense_mask_build_kernel(const int64_t* indptr, const void* indices, int idx32,
                                                               int64_t rows, const int32_t* row_rank,
                                                               const int32_t* col_rank, const int32_t* extent_cols,
                                                               const int64_t* mask_off, int64_t row_blocks,
                                                               uint32_t* mask, uint8_t* keep, int32_t* kept) {
    const int lane = lane_id();
    const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int64_t start = indptr[row], end = indptr[row + 1];
    const int rr = row_rank[row];
    const int64_t rb = rr >> 8;
    const bool in_block = rb < row_blocks;
    const int ext = in_block ? extent_cols[rb] : 0;
    uint32_t* mblock = in_block ? mask + mask_off[rb] : mask;
    const int rl = rr & 255, rg = rl >> 6, h = (rl >> 5) & 1, lr = rl & 31;
    int cnt = 0;
    for (int64_t q = start + lane; q < end; q += kWave) {
        const int j = idx32 ? static_cast<const int*>(indices)[q]
                            : static_cast<int>(static_cast<const int64_t*>(indices)[q]);
        int k = 1;
        const int cr = ext > 0 ? col_rank[j] : 0;
        if (cr < ext) {
            const int u = cr >> 8, jl = cr & 255;
            const int s = jl >> 5, g = (jl >> 4) & 1, tt = jl & 15;
            const int w = tt >> 2, b = tt & 3;
            const int64_t dword = (((static_cast<int64_t>(u) * 4 + rg) * 2 + (s >> 2)) * 64 + lr + 32 * g) * 4 + (s & 3);
            const uint32_t bit = 1u << (8 * b + 4 * h + w);
            const uint32_t old = atomicOr(mblock + dword, bit);
            if (!(old & bit)) k = 0;  // a repeated edge finds its bit set and stays in the rest
        }
        keep[q] = static_cast<uint8_t>(k);
        cnt += k;
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) cnt += __shfl_xor(cnt, off, kWave);
    if (lane == 0) kept[row] = cnt;
}

// Rate probe of the int8 matrix instructions: every wavefront runs `iters` rounds of eight independent
// accumulator chains out of registers (no memory traffic); blockDim.x = 256.
template <int SHAPE>
__global__ __launch_bounds__(256) void mfma_probe_kernel(int iters, int* sink) {
    const int lane = lane_id();
    i32x4 a{lane, lane + 1, lane + 2, lane + 3}, b{3 * lane, 5 * lane, 7 * lane, 11 * lane};
    int total = 0;
    if (SHAPE == 0) {
        i32x4 acc[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[c] = i32x4{c, 0, 0, 0};
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int c = 0; c < 8; ++c) acc[c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[c], 0, 0, 0);
        }
#pragma unroll
        for (int c = 0; c < 8; ++c) total += acc[c][0] + acc[c][1] + acc[c][2] + acc[c][3];
    } else {
        i32x16v acc[8];
#pragma unroll
        for (int c = 0; c < 8; ++c)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[c][v] = c + v;
        // SHAPE 2, 3, 4: the first operand is expanded from a word of bits (a shift and an and per register, as the
        // bit-block kernel does) once per 1, 2, 4 matrix instructions: what the matrix pipes sustain beside that work
        constexpr int PER = SHAPE <= 1 ? 0 : 1 << (SHAPE - 2);
        uint32_t word = 0x9e3779b9u * static_cast<uint32_t>(lane + 1);
        for (int it = 0; it < iters; ++it) {
            if (PER) word += 0x01000193u;
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                if (PER && c % PER == 0) {
#pragma unroll
                    for (int w = 0; w < 4; ++w) a[w] = static_cast<int>((word >> ((c + w) & 7)) & 0x01010101u);
                }
                acc[c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[c], 0, 0, 0);
            }
        }
#pragma unroll
        for (int c = 0; c < 8; ++c)
#pragma unroll
            for (int v = 0; v < 16; ++v) total += acc[c][v];
    }
    if (total == 0x7fffffff) sink[0] = total;  // keeps the chains alive; practically never taken
}

// The inner loop of the bit-block kernel without its global loads (timing experiments): per round eight k-steps of
// (two fragment reads from LDS, four operand expansions, eight matrix instructions); LEVEL 1 adds the LDS writes
// and the workgroup barrier that end a unit.  blockDim.x = 256, dynamic LDS 64 KB.
template <int LEVEL>
__global__ __launch_bounds__(256, 2) void mfma_loop_probe_kernel(int iters, int* sink, const int8_t* src = nullptr) {
    extern __shared__ __attribute__((aligned(16))) int8_t ring[];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    for (int i = t; i < 4096; i += 256) reinterpret_cast<i32x4*>(ring)[i] = i32x4{i, i + 1, i + 2, i + 3};
    __syncthreads();
    i32x16v acc[2][4];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int h = 0; h < 4; ++h)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[c][h][v] = 0;
    u32x4 mw[2][2];
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) mw[g][hf] = u32x4{0x9e3779b9u * (lane + 1), 0x85ebca6bu * (lane + 3), 0xc2b2ae35u * (lane + 5), 0x27d4eb2fu * (lane + 7)};
    for (int k = 0; k < iters; ++k) {
        const int8_t* buf = ring + (k & 1) * 32768;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            i32x4 mf[4];
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                const uint32_t word = mw[g][s >> 2][s & 3] + k;
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int w = 0; w < 4; ++w) mf[2 * g + h][w] = static_cast<int>((word >> (4 * h + w)) & 0x01010101u);
            }
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const i32x4 ff = *reinterpret_cast<const i32x4*>(buf + ((s * 4 + (wave & 1) * 2 + c) * 64 + lane) * 16);
#pragma unroll
                for (int h = 0; h < 4; ++h) acc[c][h] = __builtin_amdgcn_mfma_i32_32x32x32_i8(mf[h], ff, acc[c][h], 0, 0, 0);
            }
        }
        if (LEVEL == 1) {
            int8_t* nbuf = ring + ((k + 1) & 1) * 32768;
#pragma unroll
            for (int i = 0; i < 8; ++i) *reinterpret_cast<u32x4*>(nbuf + (i * 256 + t) * 16) = mw[i & 1][(i >> 1) & 1];
        }
        if (LEVEL == 3) {  // the next chunk by global-to-LDS loads from a small (cached) buffer, as the block kernel stages
            int8_t* nbuf = ring + ((k + 1) & 1) * 32768;
            const u32x4* x = reinterpret_cast<const u32x4*>(src) + ((k & 7) * 2048 + t);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                __builtin_amdgcn_global_load_lds(x + i * 256, reinterpret_cast<u32x4*>(nbuf) + i * 256 + (t >> 6) * 64, 16, 0, 0);
            __builtin_amdgcn_s_waitcnt(0x0F70);
        }
        if (LEVEL >= 1) __syncthreads();
    }
    int total = 0;
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int h = 0; h < 4; ++h)
#pragma unroll
            for (int v = 0; v < 16; ++v) total += acc[c][h][v];
    if (total == 0x7fffffff) sink[0] = total;
}

static size_t align256(size_t v) { return (v + 255) & ~static_cast<size_t>(255); }

size_t dense_workspace_bytes(const tango_spmm_dense_plan& plan, int64_t F) {
    const int npad = dense_npad(F);
    if (!npad) return 0;
    return align256(static_cast<size_t>(plan.dense_cols) * npad) +
           align256(static_cast<size_t>(plan.dense_rows) * npad * sizeof(int));
}

int dense_partial_sums(const tango_spmm_dense_plan& plan, const int8_t* feat, int64_t ldf, int64_t F,
                       void* workspace, size_t workspace_bytes, const int** part, int* npad_out) {
    const int npad = dense_npad(F);
    if (!npad) return TANGO_ERR_UNSUPPORTED;
    if ((reinterpret_cast<uintptr_t>(feat) & 15) || (ldf & 15) || ((F + 15) & ~15LL) > ldf) return TANGO_ERR_UNSUPPORTED;
    if (!workspace || workspace_bytes < dense_workspace_bytes(plan, F) || (reinterpret_cast<uintptr_t>(workspace) & 255))
        return TANGO_ERR_WORKSPACE;
    if (plan.dense_rows != plan.row_blocks * kDenseRows || plan.dense_cols % kDenseUnit != 0 || plan.num_groups <= 0 ||
        plan.num_groups > 65535 || plan.num_groups2 <= 0 || plan.num_groups2 > 65535 || !plan.seg_ptr2 || !plan.segs2 || !plan.col_ids || !plan.mask || !plan.mask_off || !plan.seg_ptr || !plan.segs ||
        (plan.num_shared > 0 && !plan.shared_blocks))
        return TANGO_ERR_INVALID_ARG;
    *part = reinterpret_cast<const int*>(static_cast<char*>(workspace) + align256(static_cast<size_t>(plan.dense_cols) * npad));
    *npad_out = npad;
    return TANGO_OK;
}

int launch_dense_block(const tango_spmm_dense_plan& plan, const int8_t* feat, int64_t ldf, int64_t F,
                       void* workspace, size_t workspace_bytes, const int** part, int* npad_out, hipStream_t s) {
    const int checked = dense_partial_sums(plan, feat, ldf, F, workspace, workspace_bytes, part, npad_out);
    if (checked != TANGO_OK) return checked;
    const int npad = *npad_out;
    DenseParams p{};
    p.mask = plan.mask; p.mask_off = plan.mask_off; p.seg_ptr = plan.seg_ptr; p.segs = plan.segs;
    p.shared_blocks = plan.shared_blocks; p.col_ids = plan.col_ids; p.feat = feat; p.ldf = ldf;
    p.fbytes = (F + 15) & ~15LL;
    p.xt = static_cast<int8_t*>(workspace);
    p.part = const_cast<int*>(*part);
    p.npad = npad;
    p.units = plan.dense_cols / kDenseUnit;
    p.stage_groups = plan.dense_cols / 64;
    const dim3 sgrid(static_cast<unsigned>(p.stage_groups + plan.num_shared));  // staging, then zeroing workgroups
#define TANGO_DENSE(NPAD, NCTW, RW)                                                                              \
    do {                                                                                                     \
        constexpr int SPLIT = NPAD / (32 * NCTW);                                                            \
        if (SPLIT == 1) {                                                                                    \
            p.seg_ptr = plan.seg_ptr2; p.segs = plan.segs2;                                                  \
        }                                                                                                    \
        const dim3 bgrid(static_cast<unsigned>(SPLIT == 1 ? plan.num_groups2 : plan.num_groups), SPLIT);     \
        hipLaunchKernelGGL((dense_stage_kernel<NPAD, NCTW>), sgrid, dim3(256), 0, s, p);                     \
        hipLaunchKernelGGL((dense_block_kernel<NCTW, SPLIT, RW>), bgrid, dim3(256), 0, s, p);                             \
    } while (0)
    if (npad == 64) TANGO_DENSE(64, 2, 2);
    else if (npad == 128) TANGO_DENSE(128, 2, 2);
    else TANGO_DENSE(256, 4, 4);
#undef TANGO_DENSE
    return launch_status();
}

}  // namespace tango

using namespace tango;

extern "C" {

int tango_probe_mfma_i8(int shape, int iters, int blocks, int* sink, tango_stream_t stream) {
    if (shape < 0 || shape > 8 || iters < 0 || blocks <= 0 || !sink) return TANGO_ERR_INVALID_ARG;
    hipStream_t s = as_stream(stream);
    switch (shape) {
        case 0: hipLaunchKernelGGL(mfma_probe_kernel<0>, dim3(blocks), dim3(256), 0, s, iters, sink); break;
        case 1: hipLaunchKernelGGL(mfma_probe_kernel<1>, dim3(blocks), dim3(256), 0, s, iters, sink); break;
        case 2: hipLaunchKernelGGL(mfma_probe_kernel<2>, dim3(blocks), dim3(256), 0, s, iters, sink); break;
        case 3: hipLaunchKernelGGL(mfma_probe_kernel<3>, dim3(blocks), dim3(256), 0, s, iters, sink); break;
        case 4: hipLaunchKernelGGL(mfma_probe_kernel<4>, dim3(blocks), dim3(256), 0, s, iters, sink); break;
        case 5: hipLaunchKernelGGL(mfma_loop_probe_kernel<0>, dim3(blocks), dim3(256), 65536, s, iters, sink, nullptr); break;
        case 6: hipLaunchKernelGGL(mfma_loop_probe_kernel<1>, dim3(blocks), dim3(256), 65536, s, iters, sink, nullptr); break;
        case 7: hipLaunchKernelGGL(mfma_loop_probe_kernel<2>, dim3(blocks), dim3(256), 65536, s, iters, sink, nullptr); break;
        default: hipLaunchKernelGGL(mfma_loop_probe_kernel<3>, dim3(blocks), dim3(256), 65536, s, iters, sink,
                                    reinterpret_cast<const int8_t*>(sink) + 256); break;
    }
    return launch_status();
}

int tango_spmm_dense_mask_build(const int64_t* indptr, const void* indices, int idx_bits, int64_t rows,
                                const int32_t* row_rank, const int32_t* col_rank,
                                const int32_t* extent_cols, const int64_t* mask_off, int64_t row_blocks,
                                uint32_t* mask, uint8_t* keep, int32_t* kept, tango_stream_t stream) {
    if (rows < 0 || row_blocks < 0 || !indptr || (idx_bits != 32 && idx_bits != 64) ||
        (rows > 0 && (!indices || !row_rank || !col_rank || !keep || !kept)) ||
        (row_blocks > 0 && (!extent_cols || !mask_off || !mask)))
        return TANGO_ERR_INVALID_ARG;
    if (rows == 0) return TANGO_OK;
    if (ceil_div(rows, 4) > INT32_MAX) return TANGO_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(dense_mask_build_kernel, dim3(static_cast<unsigned>(ceil_div(rows, 4))), dim3(256), 0,
                       as_stream(stream), indptr, indices, idx_bits == 32 ? 1 : 0, rows, row_rank, col_rank,
                       extent_cols, mask_off, row_blocks, mask, keep, kept);
    return launch_status();
}

}  // extern "C"
