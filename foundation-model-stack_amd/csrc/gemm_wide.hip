// bfloat16 products y = x W^T for 17 to 64 rows of x, weights [rows, K] with K contiguous.
//
// With this many rows of x the activations are no longer small beside the weights: a block that owns 16
// weight rows and all of K (gemm.hip) reads four times as many bytes of x as of W.  Here a block owns 128
// weight rows (a 16-row tile per wave) and a slice of K, and its waves share the x rows of the slice through
// LDS, so x is read once per 128 weight rows.  The price is that the slices of K meet in memory: the
// product kernel leaves float32 partial sums in a workspace, and a second kernel adds them in a fixed order
// (the same bits whatever the launch looks like) and applies the epilogue.
#include "gemm_epilogue.h"

#define WD_ROWS 128   // weight rows per block
#define WD_GROUP 128  // k-values per step of the stream
#define WD_COMPUTE_UNITS 256
#define WD_DEPTH 4  // steps whose loads are in flight (even)

// Loads are 16 rows' 256 contiguous bytes as 4 instructions of 4 rows (what the memory system streams at
// full rate); LDS holds them as loaded, with the 16-byte pieces of a row XOR-swizzled by the row, and gives
// them back in the MFMA operand layout (lane (r, g) takes row r, k-step s at piece 4 s + g).
template <int MT>
__global__ void __launch_bounds__(512)
    wide_partial_kernel(const bf16* __restrict__ x, long ldx, const bf16* __restrict__ w, float* __restrict__ part,
                        int M, int rows, int K, int groups_per_slice) {
  __shared__ __attribute__((aligned(16))) bf16 xs[2][MT * 16 * WD_GROUP];  // two steps of x: one read, one written
  __shared__ __attribute__((aligned(16))) bf16 ws[8][16 * WD_GROUP];       // a wave's own weight tile
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x & (WAVE - 1);
  const int r = lane & 15, g = lane >> 4;
  const int lrow = lane >> 4, seg = lane & 15;
  const int n0 = blockIdx.x * WD_ROWS + wave * 16;
  const int ngroups = (K + WD_GROUP - 1) / WD_GROUP;
  const int g_begin = blockIdx.y * groups_per_slice;
  const int g_end = g_begin + groups_per_slice < ngroups ? g_begin + groups_per_slice : ngroups;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  // x pieces of a step: MT * 16 rows x 16 pieces, dealt over the 512 threads (row = id / 16, piece = id % 16).
  // Loads never sit behind a branch and their data is not touched before the step that uses it (either makes
  // the compiler wait for every load in flight): a piece out of range is read from a valid address, and is
  // replaced by zeros only when it goes to LDS.
  constexpr int XP = (MT * 256 + 511) / 512;
  auto x_ok = [&](int grp, int i) {
    const int id = threadIdx.x + i * 512;
    return id < MT * 256 && (id >> 4) < M && grp * WD_GROUP + (id & 15) * 8 < K;
  };
  auto w_ok = [&](int grp, int q) { return n0 + 4 * q + lrow < rows && grp * WD_GROUP + seg * 8 < K; };
  auto load_x = [&](int grp, bf16x8 (&xr)[XP]) {
#pragma unroll
    for (int i = 0; i < XP; ++i) {
      const int id = threadIdx.x + i * 512;
      const size_t at = x_ok(grp, i) ? (size_t)(id >> 4) * ldx + grp * WD_GROUP + (id & 15) * 8 : 0;
      xr[i] = *reinterpret_cast<const bf16x8*>(x + at);
    }
  };
  auto store_x = [&](int grp, int buf, const bf16x8 (&xr)[XP]) {
#pragma unroll
    for (int i = 0; i < XP; ++i) {
      const int id = threadIdx.x + i * 512;
      const int m = id >> 4, piece = id & 15;
      if (id < MT * 256)
        *reinterpret_cast<bf16x8*>(xs[buf] + m * WD_GROUP + ((piece ^ m) & 15) * 8) = x_ok(grp, i) ? xr[i] : zero;
    }
  };
  auto load_w = [&](int grp, bf16x8 (&wr)[4]) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const size_t at = w_ok(grp, q) ? (size_t)(n0 + 4 * q + lrow) * K + grp * WD_GROUP + seg * 8 : 0;
      wr[q] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(w + at));
    }
  };

  f32x4 acc[MT];
#pragma unroll
  for (int j = 0; j < MT; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // WD_DEPTH steps in flight: while step t multiplies, the loads of steps t + 1 .. t + WD_DEPTH - 1 are under
  // way (a load takes several steps' time to arrive)
  // Every step issues the loads of the step WD_DEPTH - 1 ahead, in range or not (past the slice's end the last
  // step is loaded again and never used): with the same number of loads under way wherever the loop is, the
  // compiler can wait for exactly the oldest ones instead of for all.
  bf16x8 xr[WD_DEPTH][XP], wr[WD_DEPTH][4];
  const int g_last = g_end - 1;
#pragma unroll
  for (int d = 0; d < WD_DEPTH - 1; ++d) {
    const int at = g_begin + d < g_end ? g_begin + d : g_last;
    load_x(at, xr[d]);
    load_w(at, wr[d]);
  }
  for (int grp = g_begin; grp < g_end; grp += WD_DEPTH) {
#pragma unroll
    for (int d = 0; d < WD_DEPTH; ++d) {
      const int cur = grp + d;
      constexpr int ahead = WD_DEPTH - 1;
      {
        const int at = cur + ahead < g_end ? cur + ahead : g_last;
        load_x(at, xr[(d + ahead) % WD_DEPTH]);
        load_w(at, wr[(d + ahead) % WD_DEPTH]);
      }
      const int buf = d & 1;  // WD_DEPTH is even: steps alternate between the two x buffers
      store_x(cur, buf, xr[d]);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int row = 4 * q + lrow;
        *reinterpret_cast<bf16x8*>(ws[wave] + row * WD_GROUP + ((seg ^ row) & 15) * 8) = w_ok(cur, q) ? wr[d][q] : zero;
      }
      block_sync_lds();  // the step's x is whole; the buffer written now was last read two steps ago
      if (cur < g_end) {  // uniform; a step past the end multiplies nothing
        bf16x8 a[4];
#pragma unroll
        for (int st = 0; st < 4; ++st)
          a[st] = *reinterpret_cast<const bf16x8*>(ws[wave] + r * WD_GROUP + (((st * 4 + g) ^ r) & 15) * 8);
        // all operands of the step first, then the products: a read that waits in front of every product
        // would pay the LDS latency sixteen times a step
        bf16x8 b[MT][4];
#pragma unroll
        for (int j = 0; j < MT; ++j)
#pragma unroll
          for (int st = 0; st < 4; ++st) {
            const int m = j * 16 + r;
            b[j][st] = *reinterpret_cast<const bf16x8*>(xs[buf] + m * WD_GROUP + (((st * 4 + g) ^ m) & 15) * 8);
          }
#pragma unroll
        for (int j = 0; j < MT; ++j)
#pragma unroll
          for (int st = 0; st < 4; ++st) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[st], b[j][st], acc[j], 0, 0, 0);
      }
    }
  }
  // acc[j][e]: weight row n0 + 4 g + e, x row 16 j + r
  float* dst = part + (size_t)blockIdx.y * M * rows;
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    const int m = j * 16 + r;
    if (m >= M) continue;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int n = n0 + 4 * g + e;
      if (n < rows) dst[(size_t)m * rows + n] = acc[j][e];
    }
  }
}

// One wave per row m and 64 columns: adds the slices and finishes the element as the epilogue says.
template <int EPI, typename OutT, typename BiasT>
__global__ void __launch_bounds__(256)
    wide_finish_kernel(const float* __restrict__ part, int slices, int rows, const BiasT* __restrict__ bias,
                       OutT* __restrict__ out, long ldo, int M, int N, int tile2_offset, int act, RowScale scale,
                       RopeEpilogue rope, ResidEpilogue res) {
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x & (WAVE - 1);
  const int m = blockIdx.y * 4 + wave;
  const int n = blockIdx.x * WAVE + lane;
  if (m >= M) return;  // whole waves
  const bool live = n < N;

  float row_scale = 1.f;
  if (scale.partials != nullptr) {
    float sum = 0.f;
    for (int i = lane; i < scale.count; i += WAVE) sum += scale.partials[(size_t)m * scale.count + i];
    row_scale = rsqrtf(wave_sum(sum) * scale.inv_width + scale.eps);
  }
  float v = 0.f, u = 0.f;
  if (live) {
    for (int s = 0; s < slices; ++s) v += part[((size_t)s * M + m) * rows + n];
    if (EPI == EPI_GATED)
      for (int s = 0; s < slices; ++s) u += part[((size_t)s * M + m) * rows + tile2_offset + n];
  }
  v *= row_scale;
  u *= row_scale;

  if (EPI == EPI_GATED) {
    if (!live) return;
    if (bias) {
      v += to_f32(bias[n]);
      u += to_f32(bias[tile2_offset + n]);
    }
    out[(size_t)m * ldo + n] = from_f32<OutT>(sk_activate(v, act) * u);
  } else if (EPI == EPI_ROPE) {
    if (bias && live) v += to_f32(bias[n]);
    const float partner = __shfl_xor(v, 1, WAVE);  // the other element of the rotary pair (N is even)
    if (!live) return;
    const int D = rope.head_dim;
    const int hh = n / D, d = n - hh * D;
    const int pos = rope.positions[m], seq = rope.seq_of_token[m];
    if (hh < rope.nheads + rope.kvheads && rope.cos_t != nullptr && d < rope.rot_dim) {
      const int tpos = pos < rope.max_pos ? pos : rope.max_pos - 1;  // the host has checked the range
      const float c = rope.cos_t[(size_t)tpos * (rope.rot_dim / 2) + d / 2];
      const float sn = rope.sin_t[(size_t)tpos * (rope.rot_dim / 2) + d / 2];
      v = (d & 1) ? sn * partner + c * v : c * v - sn * partner;
    }
    if (hh < rope.nheads) {
      out[(size_t)m * ldo + n] = from_f32<OutT>(v);
    } else if (seq >= 0 && rope.k_cache != nullptr) {
      const size_t page = (size_t)rope.block_table[(size_t)seq * rope.table_stride + pos / PAGE_TOKENS];
      const size_t page_elems = (size_t)rope.kvheads * PAGE_TOKENS * D;
      const int in_page = pos % PAGE_TOKENS;
      if (hh < rope.nheads + rope.kvheads) {
        const int kh = hh - rope.nheads;
        rope.k_cache[page * page_elems + ((size_t)kh * PAGE_TOKENS + in_page) * D + d] = (bf16)v;
      } else {
        const int kh = hh - rope.nheads - rope.kvheads;
        rope.v_cache[page * page_elems + ((size_t)kh * D + d) * PAGE_TOKENS + in_page] = (bf16)v;
      }
    }
  } else if (EPI == EPI_RESID) {
    float stream = 0.f;
    if (live) {
      if (bias) v += to_f32(bias[n]);
      stream = res.resid[(size_t)m * res.ldr + n] + v;
      res.resid[(size_t)m * res.ldr + n] = stream;
      float nw = 1.f;
      if (res.norm_w != nullptr)
        nw = res.norm_w_f32 ? ((const float*)res.norm_w)[n] : to_f32(((const bf16*)res.norm_w)[n]);
      out[(size_t)m * ldo + n] = from_f32<OutT>(stream * nw);
    }
    float sq = stream * stream;  // sums over the groups of 16 neighbouring columns
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) sq += __shfl_xor(sq, off, WAVE);
    if ((lane & 15) == 0 && n / 16 < res.tiles) res.partials[(size_t)m * res.tiles + n / 16] = sq;
  } else {
    if (!live) return;
    if (bias) v += to_f32(bias[n]);
    out[(size_t)m * ldo + n] = from_f32<OutT>(v);
  }
}

// Slices of K.  A block's time goes with its steps; the blocks run in rounds over the compute units; and the
// partial sums are written and read once per slice.  The number of slices with the least of
//   rounds x steps per slice + (partial bytes a compute unit moves) / (bytes of a step)
// wins: 48 blocks of rows in 5 slices are one round of 7 steps, in 6 slices two rounds of 6.
static int wide_slices(int M, int rows, int K) {
  const int row_blocks = ceil_div(rows, WD_ROWS);
  const int ngroups = ceil_div(K, WD_GROUP);
  int best = 1;
  double best_cost = 0;
  for (int slices = 1; slices <= ngroups && slices <= 64; ++slices) {
    const double rounds = ceil_div((long)row_blocks * slices, WD_COMPUTE_UNITS);
    const double steps = ceil_div(ngroups, slices);
    const double partial = (double)slices * M * rows * 8 / WD_COMPUTE_UNITS / (WD_ROWS * WD_GROUP * 2);
    const double cost = rounds * steps + partial + 1.0;  // + a step's worth of start and end per slice's block
    if (slices == 1 || cost < best_cost) best = slices, best_cost = cost;
  }
  return best;
}

long wide_workspace_bytes(int M, int rows, int K) {
  return (long)wide_slices(M, rows, K) * M * rows * (long)sizeof(float);
}

template <int EPI>
static void launch_finish(const float* part, int slices, int rows, const void* bias, int bias_dtype, void* out,
                          int out_dtype, long ldo, int M, int N, int tile2_offset, int act, RowScale scale,
                          RopeEpilogue rope, ResidEpilogue res, hipStream_t stream) {
  dim3 grid(ceil_div(N, WAVE), ceil_div(M, 4));
  const bool fb = bias != nullptr && bias_dtype == FMS_F32;
#define FMS_WF(O, B)                                                                                             \
  wide_finish_kernel<EPI, O, B><<<grid, 256, 0, stream>>>(part, slices, rows, (const B*)bias, (O*)out, ldo, M, N, \
                                                          tile2_offset, act, scale, rope, res)
  if (out_dtype == FMS_BF16) {
    if (fb)
      FMS_WF(bf16, float);
    else
      FMS_WF(bf16, bf16);
  } else if (EPI != EPI_ROPE && EPI != EPI_RESID) {
    if (fb)
      FMS_WF(float, float);
    else
      FMS_WF(float, bf16);
  }
#undef FMS_WF
}

// N: columns of the output (for the gated product the hidden size; W then has tile2_offset + N rows).
int wide_product(int epi, const void* x, long ldx, const void* w, const void* bias, int bias_dtype, void* out,
                 int out_dtype, long ldo, int M, int N, int K, int tile2_offset, int act, RowScale scale,
                 RopeEpilogue rope, ResidEpilogue res, void* workspace, long workspace_bytes, hipStream_t stream) {
  const int rows = epi == EPI_GATED ? tile2_offset + N : N;
  FMS_REQUIRE(M > 16 && M <= 64, "wide product: %d rows (17..64)", M);
  FMS_REQUIRE(workspace != nullptr && workspace_bytes >= wide_workspace_bytes(M, rows, K),
              "wide product: workspace of %ld bytes, %ld needed", workspace_bytes, wide_workspace_bytes(M, rows, K));
  const int slices = wide_slices(M, rows, K);
  const int ngroups = ceil_div(K, WD_GROUP);
  const int per_slice = ceil_div(ngroups, slices);
  dim3 grid(ceil_div(rows, WD_ROWS), slices);
  FMS_REQUIRE(grid.y <= 65535, "wide product: %d slices", slices);
  float* part = (float*)workspace;
  const int mt = ceil_div(M, 16);
  if (mt == 2)
    wide_partial_kernel<2><<<grid, 512, 0, stream>>>((const bf16*)x, ldx, (const bf16*)w, part, M, rows, K, per_slice);
  else if (mt == 3)
    wide_partial_kernel<3><<<grid, 512, 0, stream>>>((const bf16*)x, ldx, (const bf16*)w, part, M, rows, K, per_slice);
  else
    wide_partial_kernel<4><<<grid, 512, 0, stream>>>((const bf16*)x, ldx, (const bf16*)w, part, M, rows, K, per_slice);
  FMS_LAUNCH_CHECK("wide product");
  switch (epi) {
    case EPI_PLAIN:
      launch_finish<EPI_PLAIN>(part, slices, rows, bias, bias_dtype, out, out_dtype, ldo, M, N, 0, 0, scale, rope, res, stream);
      break;
    case EPI_GATED:
      launch_finish<EPI_GATED>(part, slices, rows, bias, bias_dtype, out, out_dtype, ldo, M, N, tile2_offset, act, scale,
                               rope, res, stream);
      break;
    case EPI_ROPE:
      launch_finish<EPI_ROPE>(part, slices, rows, bias, bias_dtype, out, out_dtype, ldo, M, N, 0, 0, scale, rope, res, stream);
      break;
    default:
      launch_finish<EPI_RESID>(part, slices, rows, bias, bias_dtype, out, out_dtype, ldo, M, N, 0, 0, scale, rope, res, stream);
  }
  FMS_LAUNCH_CHECK("wide product finish");
  return 0;
}
