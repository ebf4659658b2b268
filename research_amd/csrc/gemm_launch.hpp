// Launchers of the two grouped GEMM forms of the backward pass (grouped_gemm_bwd.hip),
// callable from the entry points in backward.hip.  Both pick the LDS-DMA bf16 kernels when
// shape and alignment allow and an element-wise staged kernel (any dtype, any shape) otherwise.
#pragma once

#include "common.hpp"

namespace jtmoe {

// C[rows of group e, :] = sum over s < segs of A_s[rows of e, :] @ B_s[e]^T
//   A_s: [rows, Kdim], or [a_rows, Kdim] read through row_map (row j -> row_map[j] / row_div)
//   B_s: [E, N, Kdim]      C: [rows, N]      group_sizes == nullptr: one group holding every row
int launch_gemm_nt(int dtype, const void* a0, const void* a1, const void* b0, const void* b1, void* c,
                   const int32_t* group_sizes, const int32_t* offsets, int64_t rows, int64_t Kdim, int64_t N,
                   int64_t E, const int32_t* row_map, int row_div, int64_t a_rows, int segs, hipStream_t stream);

// C_i[e] = P[rows of group e, :]^T @ D_i[rows of group e, :]     (i = 0, and 1 if d1 is given)
//   P: [rows, KA], D_i: [rows, N]; either may instead be [gathered_rows, .] read through row_map
//   C_i: [E, KA, N]; an empty group yields zeros
//   split_ws: scratch of gemm_tn_split_bytes(...) bytes, or nullptr.  With it, a one-group call whose
//   output has too few tiles to fill the chip is run as partial sums over runs of rows (float32, in
//   split_ws) that a second kernel adds up in a fixed order.
int launch_gemm_tn(int dtype, const void* p, const void* d0, const void* d1, void* c0, void* c1,
                   const int32_t* group_sizes, const int32_t* offsets, int64_t rows, int64_t KA, int64_t N, int64_t E,
                   const int32_t* row_map, int row_div, bool p_gather, bool d_gather, int64_t gathered_rows,
                   hipStream_t stream, void* split_ws = nullptr);
size_t gemm_tn_split_bytes(int dtype, int64_t rows, int64_t KA, int64_t N, bool dual);

}  // namespace jtmoe
