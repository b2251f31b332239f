// Packed expert rows in one launch: the body of a workgroup of the row compaction, shared by
// vmoe_compact_rows (route_assign.hip) and vmoe_compact_rows_planned (expert_mlp.hip).
#ifndef VMOE_COMPACT_ROWS_H_
#define VMOE_COMPACT_ROWS_H_
#include "vmoe_common.h"

namespace vmoe {

// Groups that one block of 256 consecutive assignments may touch (first group included).
constexpr int kCompactMaxSpan = 8;

// token_slot = e*G*C + r(g, c)  ->  token_row = e*G*C + rows of expert e before group g + c,
// for the 256 assignments block * 256 .. block * 256 + 255.  For E <= 256 and groups of at
// least 37 assignments (a workgroup then touches at most kCompactMaxSpan groups): the
// workgroup adds up the fill counts of the groups before its first group itself -- 256 / E
// threads per expert, each a strided share of the groups, joined in LDS -- and then, per
// expert, the counts of the groups it touches.  Workgroup 0 also writes the experts' row
// counts.

__device__ __forceinline__ void compact_rows_fused_block(
    const int32_t* __restrict__ fill, const int32_t* __restrict__ token_slot,
    int32_t* __restrict__ token_row, int32_t* __restrict__ row_token,
    int32_t* __restrict__ rows_per_expert, int G, int E, int C, int per_group, int K, size_t n,
    unsigned block) {
  __shared__ int32_t part[256];
  __shared__ int32_t before[kCompactMaxSpan][256];   // rows of expert e before group g_lo + j
  const int tid = threadIdx.x;
  const size_t i0 = (size_t)block * 256;
  const int g_lo = (int)(i0 / per_group);
  const int parts = 256 / E;
  const int e_t = tid % E, q = tid / E;
  auto column_sum = [&](int g_end) {   // sum of fill[0 .. g_end) [e], valid in threads tid < E
    int acc = 0;
    if (q < parts)
      for (int g = q; g < g_end; g += parts) acc += fill[(size_t)g * E + e_t];
    part[tid] = acc;
    __syncthreads();
    int total = 0;
    if (tid < E)
      for (int j = 0; j < parts; ++j) total += part[j * E + tid];
    __syncthreads();
    return total;
  };
  const int lo = column_sum(g_lo);
  if (tid < E) {
    int acc = lo;
#pragma unroll
    for (int j = 0; j < kCompactMaxSpan; ++j) {      // the groups that the block's 256 assignments touch
      before[j][tid] = acc;
      if (g_lo + j < G) acc += fill[(size_t)(g_lo + j) * E + tid];
    }
  }
  if (block == 0) {
    const int total = column_sum(G);
    if (tid < E) rows_per_expert[tid] = total;
  }
  __syncthreads();
  const size_t i = i0 + tid;
  if (i >= n) return;
  const int slot = token_slot[i];
  int row = -1;
  if (slot >= 0) {
    const int g = (int)(i / per_group);
    row = packed_row(slot, before[g - g_lo][slot_expert(slot, G, C)], G, C);
    if (row_token != nullptr) row_token[row] = (int)(i / K);
  }
  token_row[i] = row;
}

// Whether the one-launch form applies (else a prefix launch goes first): a block's 256
// consecutive assignments lie in at most kCompactMaxSpan groups.
inline bool compact_rows_fused_ok(int G, int S, int E, int K) {
  const int parts = E <= 256 ? 256 / E : 1;
  const int64_t per_group = (int64_t)S * K;
  return E <= 256 && (255 + per_group - 1) / per_group + 1 <= kCompactMaxSpan &&
         (G + parts - 1) / parts <= 16;
}

}  // namespace vmoe
#endif  // VMOE_COMPACT_ROWS_H_
