// Argument block shared by the FP8 GEMM kernels.
#pragma once
#include "common.h"

namespace pt {

enum { GEMM_DENSE = 0, GEMM_M_GROUPED = 1, GEMM_K_GROUPED = 2 };

struct GemmArgs {
  const uint8_t* a; int64_t lda;          // [rows_a, red] bytes
  const uint8_t* b; int64_t ldb;          // [rows_b, red] bytes
  const float* sa; int64_t sa_rs, sa_ks; int sa_shift;  // scale(row,kb) = sa[(row>>shift)*rs + kb*ks]
  const float* sb; int64_t sb_rs, sb_ks; int sb_shift;
  void* out; int64_t ldo;                 // elements
  int out_dtype; int accumulate;
  int64_t rows_a, rows_b, red;            // output is rows_a x rows_b; red = reduction length (dense / m-grouped)
  const int32_t* offs; int G;
  int mode;
  int64_t b_stride_g, sb_stride_g, out_stride_g;
  int tiles_a, tiles_b;                   // tile counts along rows_a / rows_b
  int64_t a_bytes, b_bytes, sa_bytes, sb_bytes;  // extents of a, one group of b, and their scale arrays
  int64_t total_tiles;
  const int32_t* out_row_index;           // m-grouped only: output row of result row r (negative: dropped); null = identity
  int64_t out_rows;                       // rows of the output when out_row_index is given
  const void* bias;                       // m-grouped only: [G, rows_b] in the output's type, row g added to the rows of group g
  int64_t split_len;                      // k-grouped with offs == null: group g reduces over [g, g + 1) * split_len (split-K)
  int b_kmajor;                           // m-grouped, row-split kernel: b is [red, rows_b] per group (row pitch ldb) instead of [rows_b, red]
};

// End of group g's reduction range in the k-grouped mode (its start is the end of group g - 1).
__device__ __forceinline__ int k_group_end(const GemmArgs& p, int g) {
  if (p.offs) return p.offs[g];
  const int64_t e = (int64_t)(g + 1) * p.split_len;
  return (int)(e < p.red ? e : p.red);
}


// persistent kernel with the two-phase main loop (gemm_persistent.hip); variant selects the wave layout
int launch_gemm_persistent(const GemmArgs& a, int variant, hipStream_t stream);
// persistent kernel with the software-pipelined main loop (gemm_pipelined.hip)
int launch_gemm_pipelined(const GemmArgs& a, int variant, hipStream_t stream);
// persistent kernel whose two steps per 128-block split the tile by rows (gemm_rowsplit.hip)
int launch_gemm_rowsplit(const GemmArgs& a, int variant, hipStream_t stream);

}  // namespace pt
