// bfloat16 products y = x W^T for 17 to 192 rows of x, weights [rows, K] with K contiguous.
//
// With this many rows of x the activations are no longer small beside the weights: a block that owns 16
// weight rows and all of K (gemm.hip) reads four times as many bytes of x as of W.  Here a block owns 128
// weight rows (a 16-row tile per wave) and a slice of K, and its waves share the x rows of the slice through
// LDS, so x is read once per 128 weight rows.  When K has to be cut into slices to fill the compute units,
// the slices meet in memory: the product kernel leaves float32 partial sums in a workspace, and a second
// kernel adds them in a fixed order (the same bits whatever the launch looks like) and applies the epilogue.
// A product with enough weight rows for one slice (the gated feed-forward product, the output head) is
// finished by the product kernel itself.
// From 33 rows on the products are 32x32x16 matrix instructions on tiles of 32 weight rows and 32 rows of x, two
// waves to a tile row (a kernel of nothing but those instructions runs at twice the rate of one of 16x16x32 on this
// GPU, and a wave then reads half the rows of x from LDS): 9.5 against 9.97 ms a decode step of 128 sequences of the
// Llama-3-8B shape, 8.14 against 8.36 of 96, 13.1 against 13.9 of 192.
// Above 128 rows the registers no longer hold four steps of x: the rows of x (which come from L2, not from memory)
// are asked for one step ahead.  (Also built for these row counts and measured slower: one buffer of x with a barrier
// on either side of its filling, and blocks of four waves with 32 weight rows each, which leave a SIMD with a single
// wave to hide its waits.)
#include "gemm_epilogue.h"

#define WD_ROWS 128   // weight rows per block
#define WD_GROUP 128  // k-values per step of the stream
#define WD_COMPUTE_UNITS 256
#define WD_MAX_ROWS FMS_SKINNY_MAX_ROWS  // rows of x: twelve tiles of 16
#define WD_DEPTH 4       // steps whose loads are in flight (even)
#define WD_TILE_LD 132   // floats per row of the block's result tile in LDS: 128 and a shift of the banks

// What the product kernel does with its block's result tile.
#define WD_PARTIAL 0  // a slice of K: float32 partial sums into the workspace
#define WD_PLAIN 1    // all of K: row scale, bias, store
#define WD_GATED 2    // all of K; the block owns 64 gate rows and their 64 up rows: act(gate) * up

struct WideOut {
  void* out;
  long ldo;
  const void* bias;
  int bias_f32;
  int N, tile2_offset, act;
  int gate_rows;  // WD_GATED: gate rows (and up rows) a block owns, a multiple of 4, at most 64
  int vec;  // rows of the destination start 16-byte aligned: four elements at a time
  RowScale scale;
};

__device__ __forceinline__ float wide_bias(const WideOut& o, int n) {
  return o.bias_f32 ? ((const float*)o.bias)[n] : to_f32(((const bf16*)o.bias)[n]);
}
__device__ __forceinline__ void store4(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
__device__ __forceinline__ void store4(bf16* p, f32x4 v) {
  const bf16x4 b = {(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
  *reinterpret_cast<bf16x4*>(p) = b;
}

// Loads are 16 rows' 256 contiguous bytes as 4 instructions of 4 rows (what the memory system streams at
// full rate); LDS holds them as loaded, with the 16-byte pieces of a row XOR-swizzled by the row, and gives
// them back in the MFMA operand layout (lane (r, g) takes row r, k-step s at piece 4 s + g).
template <int MT, int MODE, typename OutT, bool SQ>
__global__ void __launch_bounds__(512)
    wide_kernel(const bf16* __restrict__ x, long ldx, const bf16* __restrict__ w, float* __restrict__ part, int M,
                int rows, int K, int groups_per_slice, WideOut o) {
  constexpr bool TALL = MT > 8;                          // more than 128 rows of x
  constexpr int XDEPTH = TALL ? 2 : WD_DEPTH;            // steps whose loads of x are in flight: the registers hold no more
  // SQ: products of 32 weight rows against 32 rows of x (32x32x16; a kernel of nothing but those runs at twice the rate
  // of one of 16x16x32 products on this GPU).  The waves form four rows of two: a pair shares 32 weight rows (each
  // wave loads 16 of them) and deals the tiles of 32 rows of x between its two waves, so that a wave reads half the
  // rows of x from LDS.  The weight tiles are then read by a neighbour too, and have two buffers like x.
  constexpr int MT32 = (MT + 1) / 2;                     // SQ: tiles of 32 rows of x
  constexpr int XROWS = SQ ? MT32 * 32 : MT * 16;        // rows of x in LDS
  constexpr int WBUFS = SQ ? 2 : 1;
  constexpr int XS_BYTES = 2 * XROWS * WD_GROUP * 2;     // two steps of x: one read, one written
  constexpr int WS_BYTES = 8 * 16 * WD_GROUP * 2;        // a weight tile per wave
  constexpr int TILE_BYTES = XROWS * WD_TILE_LD * 4;     // the block's results, once the stream has ended
  // The rows' scales (1 / rms, if the norm of x was left to this product) are worked out while the first loads are
  // under way, kept one a lane, and put into LDS behind the result tile when the stream has ended: at 192 rows the
  // stream's buffers take all of LDS.
  constexpr int STREAM_BYTES = XS_BYTES + WBUFS * WS_BYTES;
  constexpr int SMEM = STREAM_BYTES > TILE_BYTES + MT * 16 * 4 ? STREAM_BYTES : TILE_BYTES + MT * 16 * 4;
  static_assert(SMEM <= 160 * 1024, "the stream's buffers must fit the LDS of a compute unit");
  __shared__ __attribute__((aligned(16))) char smem[SMEM];
  float* const row_scale = reinterpret_cast<float*>(smem + TILE_BYTES);
  float my_scale = 1.f;  // of row wave * RPW + lane, for lane < RPW
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x & (WAVE - 1);
  bf16* const xs = reinterpret_cast<bf16*>(smem);
  bf16* const ws = reinterpret_cast<bf16*>(smem + XS_BYTES) + wave * 16 * WD_GROUP;
  float* const tile = reinterpret_cast<float*>(smem);
  const int r = lane & 15, g = lane >> 4;
  const int lrow = lane >> 4, seg = lane & 15;
  const int li = lane & 31, kb = lane >> 5;     // SQ: the lane's row of a 32-row tile and its half of a k-step's 16 values
  const int pair = wave >> 1, side = wave & 1;  // SQ: the wave's row of waves, and which of its two waves it is
  // the wave's 16 weight rows start at n0; rows from n_end on are not the wave's to read
  int n0 = blockIdx.x * WD_ROWS + wave * 16, n_end = rows;
  if (MODE == WD_GATED) {
    const int first = blockIdx.x * o.gate_rows + (wave & 3) * 16;
    const int last = ((int)blockIdx.x + 1) * o.gate_rows < o.N ? ((int)blockIdx.x + 1) * o.gate_rows : o.N;  // the block's end
    n0 = wave < 4 ? first : o.tile2_offset + first;
    n_end = wave < 4 ? last : o.tile2_offset + last;
  }
  const int ngroups = (K + WD_GROUP - 1) / WD_GROUP;
  const int g_begin = blockIdx.y * groups_per_slice;
  const int g_end = g_begin + groups_per_slice < ngroups ? g_begin + groups_per_slice : ngroups;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  // x pieces of a step: MT * 16 rows x 16 pieces, dealt over the 512 threads (row = id / 16, piece = id % 16).
  // Loads never sit behind a branch and their data is not touched before the step that uses it (either makes
  // the compiler wait for every load in flight): a piece out of range is read from a valid address, and is
  // replaced by zeros only when it goes to LDS.
  constexpr int XP = (XROWS * 16 + 511) / 512;
  auto x_ok = [&](int grp, int i) {
    const int id = threadIdx.x + i * 512;
    return id < XROWS * 16 && (id >> 4) < M && grp * WD_GROUP + (id & 15) * 8 < K;
  };
  auto w_ok = [&](int grp, int q) { return n0 + 4 * q + lrow < n_end && grp * WD_GROUP + seg * 8 < K; };
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
      if (id < XROWS * 16)
        *reinterpret_cast<bf16x8*>(xs + buf * (XROWS * WD_GROUP) + m * WD_GROUP + ((piece ^ m) & 15) * 8) =
            x_ok(grp, i) ? xr[i] : zero;
    }
  };
  auto load_w = [&](int grp, bf16x8 (&wr)[4]) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const size_t at = w_ok(grp, q) ? (size_t)(n0 + 4 * q + lrow) * K + grp * WD_GROUP + seg * 8 : 0;
      wr[q] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(w + at));
    }
  };

  f32x4 acc[SQ ? 1 : MT];
#pragma unroll
  for (int j = 0; j < (SQ ? 1 : MT); ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  constexpr int NT32 = (MT32 + 1) / 2;  // SQ: tiles of x a wave takes at most (tiles side, side + 2, ...)
  f32x16 acc32[SQ ? NT32 : 1];
#pragma unroll
  for (int j = 0; j < (SQ ? NT32 : 1); ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc32[j][v] = 0.f;

  // WD_DEPTH steps in flight: while step t multiplies, the loads of steps t + 1 .. t + WD_DEPTH - 1 are under
  // way (a load takes several steps' time to arrive).  Every step issues the loads of the step WD_DEPTH - 1
  // ahead, in range or not (past the slice's end the last step is loaded again and never used): with the same
  // number of loads under way wherever the loop is, the compiler can wait for exactly the oldest ones instead
  // of for all.
  // The blocks walk their slice from different starting steps and wrap around: blocks that all read the same
  // 256 bytes of their rows at the same time (rows lie a multiple of kilobytes apart) crowd into few memory
  // channels.  The start depends on the block's place only, so the order of the sum does too.
  bf16x8 xr[XDEPTH][XP], wr[WD_DEPTH][4];
  const int n_steps = g_end - g_begin;
  const int rot = (blockIdx.x * 5) % n_steps;
  auto group_of = [&](int t) {  // the k-group of the slice's step t (steps past the end repeat the last one)
    const int u = (t < n_steps ? t : n_steps - 1) + rot;
    return g_begin + (u >= n_steps ? u - n_steps : u);
  };
  // (a step asks for its rows of x before its rows of W: loads come back in the order they were asked for, and with
  // many rows of x those are asked for one step ahead only; they come from L2, not from memory)
#pragma unroll
  for (int d = 0; d < WD_DEPTH - 1; ++d) {
    if (d < XDEPTH - 1) load_x(group_of(d), xr[d]);
    load_w(group_of(d), wr[d]);
  }
  if (MODE != WD_PARTIAL) {
    // 1 / rms of the rows of x, if their norm was left to this product.  The partial sums are asked for behind the
    // stream's first loads and all at once: in front of them, one round trip after the other, they kept the
    // stream from starting for as long as four of its steps take.
    constexpr int RPW = MT * 2, PRE = TALL ? 2 : 4;  // rows a wave, loads a row that are under way together
    if (o.scale.partials != nullptr) {
      float pre[RPW][PRE];
#pragma unroll
      for (int k = 0; k < RPW; ++k)
#pragma unroll
        for (int j = 0; j < PRE; ++j) {
          const int m = wave * RPW + k < M ? wave * RPW + k : M - 1, i = lane + j * WAVE;
          pre[k][j] = o.scale.partials[(size_t)m * o.scale.count + (i < o.scale.count ? i : 0)];
        }
#pragma unroll
      for (int k = 0; k < RPW; ++k) {
        const int m = wave * RPW + k < M ? wave * RPW + k : M - 1;
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < PRE; ++j) sum += lane + j * WAVE < o.scale.count ? pre[k][j] : 0.f;
        for (int i = lane + PRE * WAVE; i < o.scale.count; i += WAVE) sum += o.scale.partials[(size_t)m * o.scale.count + i];
        const float total = wave_sum(sum);
        if (lane == k) my_scale = rsqrtf(total * o.scale.inv_width + o.scale.eps);
      }
    }
  }
  for (int t = 0; t < n_steps; t += WD_DEPTH) {
#pragma unroll
    for (int d = 0; d < WD_DEPTH; ++d) {
      const int cur = t + d;
      constexpr int ahead = WD_DEPTH - 1, x_ahead = XDEPTH - 1;
      load_x(group_of(cur + x_ahead), xr[(d + x_ahead) % XDEPTH]);
      load_w(group_of(cur + ahead), wr[(d + ahead) % WD_DEPTH]);
      const int buf = d & 1;  // WD_DEPTH is even: steps alternate between the two x buffers
      const int cur_g = group_of(cur);
      store_x(cur_g, buf, xr[d % XDEPTH]);
      bf16* const wsb = ws + (SQ ? buf * (WS_BYTES / 2) : 0);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int row = 4 * q + lrow;
        *reinterpret_cast<bf16x8*>(wsb + row * WD_GROUP + ((seg ^ row) & 15) * 8) = w_ok(cur_g, q) ? wr[d][q] : zero;
      }
      block_sync_lds();  // the step's x is whole; the buffer written now was last read two steps ago
      if (SQ) {
        if (cur < n_steps) {  // uniform; a step past the end multiplies nothing
          // the pair's 32 weight rows: this wave's 16 and its neighbour's, side by side in LDS
          const bf16* const wpair = reinterpret_cast<const bf16*>(smem + XS_BYTES) + buf * (WS_BYTES / 2) + pair * 32 * WD_GROUP;
          bf16x8 a[8];
#pragma unroll
          for (int st = 0; st < 8; ++st)
            a[st] = *reinterpret_cast<const bf16x8*>(wpair + li * WD_GROUP + (((st * 2 + kb) ^ li) & 15) * 8);
#pragma unroll
          for (int t32 = 0; t32 < NT32; ++t32) {
            const int jt = side + 2 * t32;  // uniform over the wave
            if (jt < MT32) {
              bf16x8 b[8];
              const int m = jt * 32 + li;
#pragma unroll
              for (int st = 0; st < 8; ++st)
                b[st] = *reinterpret_cast<const bf16x8*>(xs + buf * (XROWS * WD_GROUP) + m * WD_GROUP + (((st * 2 + kb) ^ m) & 15) * 8);
#pragma unroll
              for (int st = 0; st < 8; ++st)
                acc32[t32] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[st], b[st], acc32[t32], 0, 0, 0);
            }
          }
        }
      } else if (cur < n_steps) {  // uniform; a step past the end multiplies nothing
        bf16x8 a[4];
#pragma unroll
        for (int st = 0; st < 4; ++st)
          a[st] = *reinterpret_cast<const bf16x8*>(ws + r * WD_GROUP + (((st * 4 + g) ^ r) & 15) * 8);
        // all operands of four tiles of x first, then their products: a read that waits in front of every
        // product would pay the LDS latency sixteen times a step
        constexpr int JT = TALL ? 2 : (MT < 4 ? MT : 4);  // many rows: the registers hold the operands of two tiles
#pragma unroll
        for (int j0 = 0; j0 < MT; j0 += JT) {
          bf16x8 b[JT][4];
#pragma unroll
          for (int jj = 0; jj < JT; ++jj)
#pragma unroll
            for (int st = 0; st < 4; ++st) {
              const int m = (j0 + jj < MT ? j0 + jj : MT - 1) * 16 + r;
              b[jj][st] = *reinterpret_cast<const bf16x8*>(xs + buf * (MT * 16 * WD_GROUP) + m * WD_GROUP +
                                                           (((st * 4 + g) ^ m) & 15) * 8);
            }
#pragma unroll
          for (int jj = 0; jj < JT; ++jj)
            if (j0 + jj < MT)
#pragma unroll
              for (int st = 0; st < 4; ++st)
                acc[j0 + jj] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[st], b[jj][st], acc[j0 + jj], 0, 0, 0);
        }
      }
    }
  }

  // The block's results meet in LDS (where the stream's buffers were): row m of x, then the block's 128
  // weight rows in the order of the waves; from there they leave in whole rows of 256 or 512 bytes.
  // acc[j][e]: the wave's weight row 4 g + e, x row 16 j + r.
  __syncthreads();
  if (SQ) {
    // acc32[t][v]: x row 32 (side + 2 t) + li, the pair's weight row 8 (v / 4) + 4 kb + v % 4
#pragma unroll
    for (int t32 = 0; t32 < NT32; ++t32) {
      const int jt = side + 2 * t32;
      if (jt < MT32)
#pragma unroll
        for (int u = 0; u < 4; ++u)
          *reinterpret_cast<f32x4*>(tile + (jt * 32 + li) * WD_TILE_LD + pair * 32 + 8 * u + 4 * kb) =
              f32x4{acc32[t32][4 * u], acc32[t32][4 * u + 1], acc32[t32][4 * u + 2], acc32[t32][4 * u + 3]};
    }
  } else {
#pragma unroll
    for (int j = 0; j < MT; ++j) *reinterpret_cast<f32x4*>(tile + (j * 16 + r) * WD_TILE_LD + wave * 16 + 4 * g) = acc[j];
  }
  if (MODE != WD_PARTIAL && lane < MT * 2) row_scale[wave * (MT * 2) + lane] = my_scale;
  __syncthreads();

  if (MODE == WD_GATED) {
    // 16 threads a row: four gate columns and their four up columns each
    const int c = 4 * (threadIdx.x & 15);
    const int n = blockIdx.x * o.gate_rows + c;
    const int n_hi = ((int)blockIdx.x + 1) * o.gate_rows < o.N ? ((int)blockIdx.x + 1) * o.gate_rows : o.N;
    OutT* const out = (OutT*)o.out;
#pragma unroll
    for (int p = 0; p < (MT + 1) / 2; ++p) {
      const int m = p * 32 + (threadIdx.x >> 4);
      if (m >= M || m >= MT * 16 || n >= n_hi) continue;
      const f32x4 gate = *reinterpret_cast<const f32x4*>(tile + m * WD_TILE_LD + c);
      const f32x4 up = *reinterpret_cast<const f32x4*>(tile + m * WD_TILE_LD + WD_ROWS / 2 + c);
      const float rs = row_scale[m];
      f32x4 res;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v = gate[e] * rs, u = up[e] * rs;
        if (o.bias != nullptr && n + e < n_hi) {
          v += wide_bias(o, n + e);
          u += wide_bias(o, o.tile2_offset + n + e);
        }
        res[e] = sk_activate(v, o.act) * u;
      }
      if (o.vec && n + 3 < n_hi) {
        store4(out + (size_t)m * o.ldo + n, res);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < n_hi) out[(size_t)m * o.ldo + n + e] = from_f32<OutT>(res[e]);
      }
    }
  } else {
    // 32 threads a row: four columns each
    const int c = 4 * (threadIdx.x & 31);
    const int n = blockIdx.x * WD_ROWS + c;
    const int n_lim = MODE == WD_PLAIN ? o.N : rows;
#pragma unroll
    for (int p = 0; p < MT; ++p) {
      const int m = p * 16 + (threadIdx.x >> 5);
      if (m >= M || n >= n_lim) continue;
      f32x4 v = *reinterpret_cast<const f32x4*>(tile + m * WD_TILE_LD + c);
      if (MODE == WD_PLAIN) {
        const float rs = row_scale[m];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] *= rs;
          if (o.bias != nullptr && n + e < n_lim) v[e] += wide_bias(o, n + e);
        }
        OutT* const out = (OutT*)o.out;
        if (o.vec && n + 3 < n_lim) {
          store4(out + (size_t)m * o.ldo + n, v);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < n_lim) out[(size_t)m * o.ldo + n + e] = from_f32<OutT>(v[e]);
        }
      } else {
        float* const dst = part + ((size_t)blockIdx.y * M + m) * rows + n;
        if (o.vec && n + 3 < n_lim) {
          store4(dst, v);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < n_lim) dst[e] = v[e];
        }
      }
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
  const int nn = live ? n : 0;  // a lane past the end reads column 0 and stores nothing

  // Every load that does not wait for another one's result is asked for here, at once and not behind a branch:
  // the first slices, the partial sums of the rows' norm, the row's position and sequence, the stream and the next
  // norm's weight.  One after the other they were six to eight round trips to memory for a kernel that moves a
  // few megabytes.  What is out of range is read from a valid address and set aside where it is used.
  constexpr int FIRST = 8, PRE = 4;
  const size_t stride = (size_t)M * rows;
  const float* const pv = part + (size_t)m * rows + nn;
  const float* const pu = pv + tile2_offset;
  float av[FIRST], au[FIRST], pre[PRE];  // au: the up half of a gated product, unused otherwise
#pragma unroll
  for (int s = 0; s < FIRST; ++s) {
    const size_t at = (size_t)(s < slices ? s : 0) * stride;
    av[s] = pv[at];
    if (EPI == EPI_GATED) au[s] = pu[at];
  }
  if (scale.partials != nullptr) {  // uniform
#pragma unroll
    for (int j = 0; j < PRE; ++j) {
      const int i = lane + j * WAVE;
      pre[j] = scale.partials[(size_t)m * scale.count + (i < scale.count ? i : 0)];
    }
  }
  int pos = 0, seq = -1;
  if (EPI == EPI_ROPE) pos = rope.positions[m], seq = rope.seq_of_token[m];
  float stream_in = 0.f, nw = 1.f, bias_v = 0.f, bias_u = 0.f;
  if (EPI == EPI_RESID) {
    stream_in = res.resid[(size_t)m * res.ldr + nn];
    if (res.norm_w != nullptr) nw = res.norm_w_f32 ? ((const float*)res.norm_w)[nn] : to_f32(((const bf16*)res.norm_w)[nn]);
  }
  if (bias) {
    bias_v = to_f32(bias[nn]);
    if (EPI == EPI_GATED) bias_u = to_f32(bias[tile2_offset + nn]);
  }

  // The slices are added in their order, whatever the launch looks like.
  auto add_slices = [&](const float* p, const float (&first)[FIRST]) {
    float sum = 0.f;
#pragma unroll
    for (int s = 0; s < FIRST; ++s)
      if (s < slices) sum += first[s];
    int s = FIRST;
    for (; s + 4 <= slices; s += 4) {
      const float a0 = p[(size_t)s * stride], a1 = p[(size_t)(s + 1) * stride], a2 = p[(size_t)(s + 2) * stride],
                  a3 = p[(size_t)(s + 3) * stride];
      sum = (((sum + a0) + a1) + a2) + a3;
    }
    for (; s < slices; ++s) sum += p[(size_t)s * stride];
    return sum;
  };
  float v = add_slices(pv, av), u = 0.f;
  if (EPI == EPI_GATED) u = add_slices(pu, au);
  float row_scale = 1.f;
  if (scale.partials != nullptr) {
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < PRE; ++j) sum += lane + j * WAVE < scale.count ? pre[j] : 0.f;
    for (int i = lane + PRE * WAVE; i < scale.count; i += WAVE) sum += scale.partials[(size_t)m * scale.count + i];
    row_scale = rsqrtf(wave_sum(sum) * scale.inv_width + scale.eps);
  }
  v *= row_scale;
  u *= row_scale;

  if (EPI == EPI_GATED) {
    if (!live) return;
    out[(size_t)m * ldo + n] = from_f32<OutT>(sk_activate(v + bias_v, act) * (u + bias_u));
  } else if (EPI == EPI_ROPE) {
    v += bias_v;
    const float partner = __shfl_xor(v, 1, WAVE);  // the other element of the rotary pair (N is even)
    if (!live) return;
    const int D = rope.head_dim;
    const int hh = n / D, d = n - hh * D;
    if (hh < rope.nheads + rope.kvheads && rope.cos_t != nullptr && d < rope.rot_dim) {
      const int tpos = pos < 0 ? 0 : (pos < rope.max_pos ? pos : rope.max_pos - 1);  // the host has checked the range
      const float c = rope.cos_t[(size_t)tpos * (rope.rot_dim / 2) + d / 2];
      const float sn = rope.sin_t[(size_t)tpos * (rope.rot_dim / 2) + d / 2];
      v = (d & 1) ? sn * partner + c * v : c * v - sn * partner;
    }
    if (hh < rope.nheads) {
      out[(size_t)m * ldo + n] = from_f32<OutT>(v);
    } else if (seq >= 0 && rope.k_cache != nullptr) {
      const int entry = rope.block_table[(size_t)seq * rope.table_stride + pos / PAGE_TOKENS];
      const size_t page = readable_page(entry);
      const size_t page_elems = (size_t)rope.kvheads * PAGE_TOKENS * D;
      const int in_page = pos % PAGE_TOKENS;
      if (entry < 0) {
        // no page for this token: nothing is written
      } else if (hh < rope.nheads + rope.kvheads) {
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
      stream = stream_in + (v + bias_v);
      res.resid[(size_t)m * res.ldr + n] = stream;
      out[(size_t)m * ldo + n] = from_f32<OutT>(stream * nw);
    }
    float sq = stream * stream;  // sums over the groups of 16 neighbouring columns
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) sq += __shfl_xor(sq, off, WAVE);
    if ((lane & 15) == 0 && n / 16 < res.tiles) res.partials[(size_t)m * res.tiles + n / 16] = sq;
  } else {
    if (!live) return;
    out[(size_t)m * ldo + n] = from_f32<OutT>(v + bias_v);
  }
}

// Slices of K.  A block's time goes with its steps; the blocks run in rounds over the compute units; and the
// partial sums are written and read once per slice (not at all when the product kernel finishes its one
// slice itself).  The number of slices with the least of
//   rounds x steps per slice + (partial bytes a compute unit moves) / (bytes of a step)
// wins: 48 blocks of rows in 5 slices are one round of 7 steps, in 6 slices two rounds of 6.
static bool wide_finishes_itself(int epi) { return epi == EPI_PLAIN || epi == EPI_GATED; }

static int wide_slices(int epi, int M, int rows, int K) {
  const int row_blocks = ceil_div(rows, WD_ROWS);
  const int ngroups = ceil_div(K, WD_GROUP);
  int best = 1;
  double best_cost = 0;
  for (int slices = 1; slices <= ngroups && slices <= 64; ++slices) {
    const double rounds = ceil_div((long)row_blocks * slices, WD_COMPUTE_UNITS);
    const double steps = ceil_div(ngroups, slices);
    double partial = (double)slices * M * rows * 8 / WD_COMPUTE_UNITS / (WD_ROWS * WD_GROUP * 2);
    if (slices == 1 && wide_finishes_itself(epi)) partial = 0;
    const double cost = rounds * steps + partial + 1.0;  // + a step's worth of start and end per slice's block
    if (slices == 1 || cost < best_cost) best = slices, best_cost = cost;
  }
  return best;
}

// Enough for any epilogue of this shape.
long wide_workspace_bytes(int M, int rows, int K) {
  return (long)wide_slices(EPI_RESID, M, rows, K) * M * rows * (long)sizeof(float);
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

template <int MODE, typename OutT>
static void launch_wide(dim3 grid, const void* x, long ldx, const void* w, float* part, int M, int rows, int K,
                        int per_slice, const WideOut& o, hipStream_t stream) {
  const int mt = ceil_div(M, 16);
  // from 33 rows on: products of 32 x 32 tiles; fewer rows are one tile of 16 or two
#define FMS_WK(MT) \
  wide_kernel<MT, MODE, OutT, (MT >= 3)><<<grid, 512, 0, stream>>>((const bf16*)x, ldx, (const bf16*)w, part, M, rows, K, per_slice, o)
  if (mt == 2)
    FMS_WK(2);
  else if (mt == 3)
    FMS_WK(3);
  else if (mt == 4)
    FMS_WK(4);
  else if (mt == 5)
    FMS_WK(5);
  else if (mt == 6)
    FMS_WK(6);
  else if (mt == 7)
    FMS_WK(7);
  else if (mt == 8)
    FMS_WK(8);
  else if (mt <= 10)  // many rows: tiles in pairs (their operands are taken two at a time); an empty tile is zeros
    FMS_WK(10);
  else
    FMS_WK(12);
#undef FMS_WK
}

// Gate rows per block of a gated product that finishes in one kernel: what a compute unit has to pull is its
// blocks (a whole number) times a block's rows of W and of x; 14336 columns in blocks of 64 are 224 blocks for 256
// units, in blocks of 56 one block for each.
static int wide_gate_rows(int M, int N) {
  int best = 0;
  long best_cost = 0;
  for (int rows = 32; rows <= WD_ROWS / 2; rows += 4) {
    const long cost = (long)ceil_div(ceil_div(N, rows), WD_COMPUTE_UNITS) * (2 * rows + M);
    if (best == 0 || cost <= best_cost) best = rows, best_cost = cost;
  }
  return best;
}

static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// N: columns of the output (for the gated product the hidden size; W then has tile2_offset + N rows).
int wide_product(int epi, const void* x, long ldx, const void* w, const void* bias, int bias_dtype, void* out,
                 int out_dtype, long ldo, int M, int N, int K, int tile2_offset, int act, RowScale scale,
                 RopeEpilogue rope, ResidEpilogue res, void* workspace, long workspace_bytes, hipStream_t stream) {
  const int rows = epi == EPI_GATED ? tile2_offset + N : N;
  FMS_REQUIRE(M > 16 && M <= WD_MAX_ROWS, "wide product: %d rows (17..%d)", M, WD_MAX_ROWS);
  const int ngroups = ceil_div(K, WD_GROUP);
  const int per_slice = ceil_div(ngroups, wide_slices(epi, M, rows, K));
  const int slices = ceil_div(ngroups, per_slice);  // no slice without a step (the kernel divides by its steps)
  const bool itself = slices == 1 && wide_finishes_itself(epi);
  WideOut o{out, ldo, bias, bias != nullptr && bias_dtype == FMS_F32, N, tile2_offset, act, WD_ROWS / 2, 0, scale};

  if (itself) {
    const long elem = out_dtype == FMS_BF16 ? 2 : 4;
    o.vec = ((uintptr_t)out % (4 * elem)) == 0 && ldo % 4 == 0;
    if (epi == EPI_GATED) {
      o.gate_rows = wide_gate_rows(M, N);
      dim3 grid(ceil_div(N, o.gate_rows), 1);
      if (out_dtype == FMS_BF16)
        launch_wide<WD_GATED, bf16>(grid, x, ldx, w, nullptr, M, rows, K, per_slice, o, stream);
      else
        launch_wide<WD_GATED, float>(grid, x, ldx, w, nullptr, M, rows, K, per_slice, o, stream);
    } else {
      dim3 grid(ceil_div(N, WD_ROWS), 1);
      if (out_dtype == FMS_BF16)
        launch_wide<WD_PLAIN, bf16>(grid, x, ldx, w, nullptr, M, rows, K, per_slice, o, stream);
      else
        launch_wide<WD_PLAIN, float>(grid, x, ldx, w, nullptr, M, rows, K, per_slice, o, stream);
    }
    FMS_LAUNCH_CHECK("wide product");
    return 0;
  }

  const long needed = (long)slices * M * rows * (long)sizeof(float);
  FMS_REQUIRE(workspace != nullptr && workspace_bytes >= needed, "wide product: workspace of %ld bytes, %ld needed",
              workspace_bytes, needed);
  dim3 grid(ceil_div(rows, WD_ROWS), slices);
  FMS_REQUIRE(grid.y <= 65535, "wide product: %d slices", slices);
  float* part = (float*)workspace;
  o.vec = aligned16(workspace) && rows % 4 == 0;
  launch_wide<WD_PARTIAL, float>(grid, x, ldx, w, part, M, rows, K, per_slice, o, stream);
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
