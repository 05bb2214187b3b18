// What the bfloat16 products for few rows (gemm.hip: at most 16 rows; gemm_wide.hip: 17 to 192) do with a
// finished output element, and the arguments of those epilogues.
#pragma once

#include "common.h"
#include "fmsamd.h"

__device__ __forceinline__ float sk_activate(float x, int kind) {
  if (kind == FMS_ACT_SILU) return x / (1.f + __expf(-x));  // the one every served model has: the fast exponential
  return fms_activate(x, kind);
}

// What the skinny kernel does with a finished output element.
#define EPI_PLAIN 0  // store (+ bias)
#define EPI_GATED 1  // the block's second tile is the "up" half: out = act(first) * second, N is the hidden size
#define EPI_ROPE 2   // the output row is [queries | keys | values] of attention: rotate q and k, store q, and
                     // write k and v into their cache pages (layout: see rope.hip)
#define EPI_RESID 3  // add the product to the float32 residual stream in place, store the new stream times the
                     // next norm's weight in the activation type, and leave the rows' sums of squares by tile

// The rows of x are not yet divided by their root mean square: the kernel that made them left, for each
// row, `count` partial sums of squares (partials[m * count + i]).  The product is multiplied by
// rsqrt(sum / width + eps) of its row before the bias.  partials == null: the rows are taken as they are.
struct RowScale {
  const float* partials;
  int count;
  float inv_width, eps;
};

struct ResidEpilogue {
  float* resid;  // [M, N] float32, read and written
  long ldr;
  const void* norm_w;  // [N] or null
  int norm_w_f32;
  float* partials;  // [M, tiles]: sum over the tile's 16 columns of the new stream squared
  int tiles;
};

struct RopeEpilogue {
  const int* positions;     // [M]
  const int* seq_of_token;  // [M], -1: padding row
  const int* block_table;
  int table_stride;
  const float* cos_t;  // [max_pos, rot_dim/2] or null
  const float* sin_t;
  int rot_dim, max_pos;
  bf16* k_cache;  // null: queries only
  bf16* v_cache;
  int nheads, kvheads, head_dim;
};


#define FMS_SKINNY_MAX_ROWS 192

// ---- 17 to 192 rows (gemm_wide.hip) ------------------------------------------
// The product runs as two kernels: blocks of 128 weight rows times a slice of K leave float32 partial sums
// in a workspace [slices][M][rows]; a second kernel adds the slices in a fixed order and applies the epilogue.
// `rows` counts all rows of W (for the gated product both halves).
long wide_workspace_bytes(int M, int rows, int K);
int wide_product(int epi, const void* x, long ldx, const void* w, const void* bias, int bias_dtype, void* out,
                 int out_dtype, long ldo, int M, int N, int K, int tile2_offset, int act, RowScale scale,
                 RopeEpilogue rope, ResidEpilogue res, void* workspace, long workspace_bytes, hipStream_t stream);
