// Dense-block part of the copy_u aggregation (spmm_dense.hip), as seen by spmm.hip.
#pragma once
#include "common.hpp"

namespace tango {

constexpr int kDenseRows = 256;  // rows of a row block (one workgroup's output tile)
constexpr int kDenseUnit = 256;  // mask columns of a unit (one LDS chunk of staged features)

// Column count the staged features and the partial sums are padded to: 64, 128 or 256 (0: too wide).
inline int dense_npad(int64_t F) { return F <= 64 ? 64 : F <= 128 ? 128 : F <= 256 ? 256 : 0; }

// Bytes of workspace the dense part needs: staged features, then the int32 partial sums.
size_t dense_workspace_bytes(const tango_spmm_dense_plan& plan, int64_t F);

// Stages the plan's columns of feat, multiplies the plan's bit blocks with them on the matrix cores and
// leaves sum over the block's edges of feat[src, c] as int32 at part[row_slot[r] * npad + c].
// Returns a status code; *part receives the partial sums' address inside the workspace.
int launch_dense_block(const tango_spmm_dense_plan& plan, const int8_t* feat, int64_t ldf, int64_t F,
                       void* workspace, size_t workspace_bytes, const int** part, int* npad, hipStream_t s);

// Where launch_dense_block leaves its partial sums for this plan, width and workspace, with its argument checks and
// no launch.
int dense_partial_sums(const tango_spmm_dense_plan& plan, const int8_t* feat, int64_t ldf, int64_t F,
                       void* workspace, size_t workspace_bytes, const int** part, int* npad);

}  // namespace tango
