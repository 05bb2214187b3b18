// Matrix products y = x W^T (+ bias) for weights stored [N, K] with K contiguous,
// which is how every linear layer of a checkpoint is stored.
//
//   * sgemm_nt_kernel: float32 in, float32 FMA accumulation, float32 out.  The
//     true 32-bit path: no matrix-core shortcut, no reduced-precision inputs.
//   * gemm_bf16_kernel: bfloat16 in, MFMA 16x16x32 with float32 accumulation,
//     bfloat16 or float32 out; LDS-tiled 128x128x32.  Any M and N; K % 8 == 0.
//   * skinny_bf16_kernel: M <= 16 rows of x (decode).  Weight-streaming: a
//     block owns one or two 16-row tiles of W, its waves split K, loads take
//     long contiguous runs and change to the MFMA layout in LDS, partial
//     sums meet in LDS.  Epilogues: plain, act(x Wg^T) * (x Wu^T), rotation
//     and cache write, addition into the residual stream.  The entry points
//     hand 17 to 192 rows to the kernels of gemm_wide.hip.
#include "common.h"
#include "fmsamd.h"
#include "gemm_epilogue.h"

// ==========================================================================
// float32
// ==========================================================================
#define SG_BM 64
#define SG_BN 64
#define SG_BK 16

// InT float: the true 32-bit product.  InT bf16: the product for sizes the MFMA kernels refuse (K or a row
// stride that is no multiple of 8, so that rows are not 16-byte aligned): element loads, float32 FMA.
template <typename InT, typename BiasT, typename OutT>
__global__ void __launch_bounds__(256)
    sgemm_nt_kernel(const InT* __restrict__ a, long lda, const InT* __restrict__ w, const BiasT* __restrict__ bias,
                    OutT* __restrict__ c, long ldc, int M, int N, int K) {
  __shared__ float as[SG_BK][SG_BM + 1];
  __shared__ float ws[SG_BK][SG_BN + 1];
  const int tx = threadIdx.x % 16;  // n direction
  const int ty = threadIdx.x / 16;  // m direction
  const int m0 = blockIdx.y * SG_BM;
  const int n0 = blockIdx.x * SG_BN;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += SG_BK) {
    for (int i = threadIdx.x; i < SG_BM * SG_BK; i += 256) {
      const int row = i / SG_BK, kk = i % SG_BK;
      const int m = m0 + row, k = k0 + kk;
      as[kk][row] = (m < M && k < K) ? to_f32(a[(size_t)m * lda + k]) : 0.f;
      const int n = n0 + row;
      ws[kk][row] = (n < N && k < K) ? to_f32(w[(size_t)n * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < SG_BK; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        av[i] = as[kk][ty * 4 + i];
        wv[i] = ws[kk][tx * 4 + i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) c[(size_t)m * ldc + n] = from_f32<OutT>(acc[i][j] + (bias ? to_f32(bias[n]) : 0.f));
    }
  }
}

extern "C" int fmsamd_gemm_f32(const float* a, long lda, const float* w, const float* bias, float* c, long ldc, int M,
                               int N, int K, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  FMS_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_f32: bad sizes M=%d N=%d K=%d", M, N, K);
  FMS_REQUIRE(lda >= K && ldc >= N, "gemm_f32: leading dimensions too small");
  dim3 grid(ceil_div(N, SG_BN), ceil_div(M, SG_BM));
  FMS_REQUIRE(grid.y <= 65535, "gemm_f32: M=%d exceeds one launch", M);
  sgemm_nt_kernel<float, float, float><<<grid, 256, 0, stream>>>(a, lda, w, bias, c, ldc, M, N, K);
  FMS_LAUNCH_CHECK("gemm_f32");
  return 0;
}

extern "C" int fmsamd_gemm_bf16_any(const void* a, long lda, const void* w, const void* bias, int bias_dtype, void* c,
                                    int out_dtype, long ldc, int M, int N, int K, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  FMS_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_bf16_any: bad sizes M=%d N=%d K=%d", M, N, K);
  FMS_REQUIRE(lda >= K && ldc >= N, "gemm_bf16_any: leading dimensions too small");
  dim3 grid(ceil_div(N, SG_BN), ceil_div(M, SG_BM));
  FMS_REQUIRE(grid.y <= 65535, "gemm_bf16_any: M=%d exceeds one launch", M);
  const bool fb = bias != nullptr && bias_dtype == FMS_F32;
#define FMS_SG(B, O)                                                                                                 \
  sgemm_nt_kernel<bf16, B, O><<<grid, 256, 0, stream>>>((const bf16*)a, lda, (const bf16*)w, (const B*)bias, (O*)c, \
                                                        ldc, M, N, K)
  if (out_dtype == FMS_BF16 && !fb)
    FMS_SG(bf16, bf16);
  else if (out_dtype == FMS_BF16 && fb)
    FMS_SG(float, bf16);
  else if (out_dtype == FMS_F32 && !fb)
    FMS_SG(bf16, float);
  else if (out_dtype == FMS_F32 && fb)
    FMS_SG(float, float);
  else
    FMS_REQUIRE(false, "gemm_bf16_any: unknown output dtype %d", out_dtype);
#undef FMS_SG
  FMS_LAUNCH_CHECK("gemm_bf16_any");
  return 0;
}

// ==========================================================================
// bfloat16, any M
// ==========================================================================
#define GB_BM 128
#define GB_BN 128
#define GB_BK 32
#define GB_LD 40  // padded LDS row (elements): 80 bytes keeps 16-byte reads conflict-poor

template <typename OutT, typename BiasT>
__global__ void __launch_bounds__(256)
    gemm_bf16_kernel(const bf16* __restrict__ a, long lda, const bf16* __restrict__ w, const BiasT* __restrict__ bias,
                     OutT* __restrict__ c, long ldc, int M, int N, int K) {
  __shared__ __attribute__((aligned(16))) bf16 as[GB_BM * GB_LD];
  __shared__ __attribute__((aligned(16))) bf16 ws[GB_BN * GB_LD];
  const int wave = threadIdx.x / WAVE;
  const int lane = threadIdx.x & (WAVE - 1);
  const int r = lane & 15, g = lane >> 4;
  const int wm = (wave >> 1) * 64;  // this wave's 64x64 corner inside the block tile
  const int wn = (wave & 1) * 64;
  const int m0 = blockIdx.y * GB_BM;
  const int n0 = blockIdx.x * GB_BN;

  f32x4 acc[4][4];  // [n tile][m tile]: rows n = nt*16 + g*4 + i, column m = mt*16 + r
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int k0 = 0; k0 < K; k0 += GB_BK) {
    // 128 rows x 4 chunks of 8 elements for each operand; 256 threads take two chunks each
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int idx = threadIdx.x + it * 256;
      const int row = idx >> 2, ch = idx & 3;
      const int k = k0 + ch * 8;
      bf16x8 va = {0, 0, 0, 0, 0, 0, 0, 0}, vw = {0, 0, 0, 0, 0, 0, 0, 0};
      if (k < K) {
        if (m0 + row < M) va = *reinterpret_cast<const bf16x8*>(a + (size_t)(m0 + row) * lda + k);
        if (n0 + row < N) vw = *reinterpret_cast<const bf16x8*>(w + (size_t)(n0 + row) * K + k);
      }
      *reinterpret_cast<bf16x8*>(as + row * GB_LD + ch * 8) = va;
      *reinterpret_cast<bf16x8*>(ws + row * GB_LD + ch * 8) = vw;
    }
    __syncthreads();
    bf16x8 av[4], wv[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      av[t] = *reinterpret_cast<const bf16x8*>(as + (wm + t * 16 + r) * GB_LD + g * 8);
      wv[t] = *reinterpret_cast<const bf16x8*>(ws + (wn + t * 16 + r) * GB_LD + g * 8);
    }
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int mt = 0; mt < 4; ++mt)
        acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[nt], av[mt], acc[nt][mt], 0, 0, 0);
    __syncthreads();
  }

#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
    const int m = m0 + wm + mt * 16 + r;
    if (m >= M) continue;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + wn + nt * 16 + g * 4 + i;
        if (n < N) {
          float v = acc[nt][mt][i];
          if (bias) v += to_f32(bias[n]);
          c[(size_t)m * ldc + n] = from_f32<OutT>(v);
        }
      }
    }
  }
}

extern "C" int fmsamd_gemm_bf16(const void* a, long lda, const void* w, const void* bias, int bias_dtype, void* c,
                                int out_dtype, long ldc, int M, int N, int K, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  FMS_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_bf16: bad sizes M=%d N=%d K=%d", M, N, K);
  FMS_REQUIRE(K % 8 == 0 && lda % 8 == 0, "gemm_bf16: K=%d and the row stride %ld must be multiples of 8", K, lda);
  FMS_REQUIRE(lda >= K && ldc >= N, "gemm_bf16: leading dimensions too small");
  dim3 grid(ceil_div(N, GB_BN), ceil_div(M, GB_BM));
  FMS_REQUIRE(grid.y <= 65535, "gemm_bf16: M=%d exceeds one launch", M);
  const bool fb = bias != nullptr && bias_dtype == FMS_F32;
#define FMS_GB(O, B)                                                                                          \
  gemm_bf16_kernel<O, B><<<grid, 256, 0, stream>>>((const bf16*)a, lda, (const bf16*)w, (const B*)bias, (O*)c, \
                                                   ldc, M, N, K)
  if (out_dtype == FMS_BF16 && !fb)
    FMS_GB(bf16, bf16);
  else if (out_dtype == FMS_BF16 && fb)
    FMS_GB(bf16, float);
  else if (out_dtype == FMS_F32 && !fb)
    FMS_GB(float, bf16);
  else if (out_dtype == FMS_F32 && fb)
    FMS_GB(float, float);
  else
    FMS_REQUIRE(false, "gemm_bf16: unknown output dtype %d", out_dtype);
#undef FMS_GB
  FMS_LAUNCH_CHECK("gemm_bf16");
  return 0;
}

// ==========================================================================
// bfloat16, M <= 16 (and the entry points for M <= 192)
// ==========================================================================

// NTB: 16-row tiles of W per block (the second tile starts `tile2_offset` rows after the first).
// MT : 16-row tiles of x.
// SK_WAVES: waves of a block.
// UNR: groups of 128 k-values whose loads a wave issues before it multiplies: what keeps enough
// bytes in flight to stream from HBM (a wave has UNR * (NTB + MT) * 4 loads of 16 bytes outstanding).
template <int SK_WAVES, int UNR, int NTB, int MT, int EPI, typename OutT, typename BiasT>
__global__ void __launch_bounds__(SK_WAVES* WAVE)
    __attribute__((amdgpu_waves_per_eu(MT > 1 ? 2 : 4)))  // two blocks a compute unit; one with several tiles of x
    skinny_bf16_kernel(const bf16* __restrict__ x, long ldx, const bf16* __restrict__ w, const BiasT* __restrict__ bias,
                       OutT* __restrict__ out, long ldo, int M, int N, int K, int tile2_offset, int act,
                       int rows_per_block, RowScale scale, RopeEpilogue rope, ResidEpilogue res) {
  constexpr bool GATED = EPI == EPI_GATED;
  // per wave: one tile of 16 rows x 128 k (4 KB) of W and one of x between load and MFMA layout; after
  // the stream the region holds the wave's partial output tiles
  constexpr int STAGE_BYTES = NTB * MT * 16 * 17 * 4 > 8192 ? NTB * MT * 16 * 17 * 4 : 8192;
  __shared__ __attribute__((aligned(16))) unsigned char stage[SK_WAVES * STAGE_BYTES];
  __shared__ int s_pos[MT * 16], s_seq[MT * 16], s_page[MT * 16];
  __shared__ float s_scale[MT * 16];
  const int wave = threadIdx.x / WAVE;
  const int lane = threadIdx.x & (WAVE - 1);
  const int r = lane & 15, g = lane >> 4;
  // A block owns rows_per_block rows of W (at most 16 * NTB; its last tile may be partly
  // empty): 24 rows make 256 equal blocks of 6144 rows where 16 would make 384.  Gated: that many gate rows in the
  // first tile and their up rows in the second.
  const int n0 = blockIdx.x * rows_per_block;
  const int n_end = n0 + rows_per_block < N ? n0 + rows_per_block : N;

  if (EPI == EPI_ROPE && threadIdx.x < MT * 16) {
    // index data of the rows, fetched while the weights stream
    const int m = threadIdx.x;
    int pos = 0, seq = -1, page = -1;
    if (m < M) {
      seq = rope.seq_of_token[m];
      pos = rope.positions[m];
      if (seq >= 0 && rope.k_cache) page = rope.block_table[(size_t)seq * rope.table_stride + pos / PAGE_TOKENS];
    }
    s_pos[m] = pos, s_seq[m] = seq, s_page[m] = page;
  }

  // Loads whose data the epilogue needs are issued here, ahead of the weight stream, so that their latency
  // is not paid at the end: the first partial sums of a deferred row norm (a wave per row, 256 sums deep) and the residual stream with the next norm's weight.
  // None of these loads sits behind a branch, and none of their data is touched before the epilogue: either
  // would make the compiler wait for the load on the spot.  What is out of range is read from a valid address
  // and set aside when it is used.
  constexpr int PRE_ROWS = (MT * 16 + SK_WAVES - 1) / SK_WAVES, PRE_DEPTH = 4;  // every row of x, 256 sums deep
  float pre[PRE_ROWS][PRE_DEPTH];
  if (scale.partials != nullptr) {
#pragma unroll
    for (int i = 0; i < PRE_ROWS; ++i)
#pragma unroll
      for (int j = 0; j < PRE_DEPTH; ++j) {
        const int m = wave + i * SK_WAVES, b = lane + j * WAVE;
        pre[i][j] = scale.partials[(size_t)(m < M ? m : 0) * scale.count + (b < scale.count ? b : 0)];
      }
  }
  constexpr int OUT_TILES = GATED ? 1 : NTB;
  constexpr int ROUNDS = (OUT_TILES * MT * 256 + SK_WAVES * WAVE - 1) / (SK_WAVES * WAVE);
  float pre_resid[ROUNDS], pre_nw[ROUNDS];  // EPI_ROPE: cosine and sine of the element's angle
  bf16 pre_nw16[ROUNDS];
  if (EPI == EPI_ROPE) {
#pragma unroll
    for (int rd = 0; rd < ROUNDS; ++rd) {
      const int idx = threadIdx.x + rd * SK_WAVES * WAVE;
      const int m = ((idx >> 8) % MT) * 16 + ((idx >> 4) & 15);
      const int n = n0 + ((idx >> 8) / MT) * 16 + (idx & 15);
      const int hh = n / rope.head_dim, d = n - hh * rope.head_dim;
      pre_resid[rd] = 1.f, pre_nw[rd] = 0.f;
      if (rope.cos_t != nullptr) {  // uniform
        const bool rotates = m < M && n < n_end && hh < rope.nheads + rope.kvheads && d < rope.rot_dim;
        const int pos = rope.positions[m < M ? m : 0];
        const int tpos = pos < 0 ? 0 : (pos < rope.max_pos ? pos : rope.max_pos - 1);  // the host has checked the range
        const size_t at = rotates ? (size_t)tpos * (rope.rot_dim / 2) + d / 2 : 0;
        pre_resid[rd] = rope.cos_t[at];
        pre_nw[rd] = rope.sin_t[at];
      }
    }
  }
  if (EPI == EPI_RESID) {
#pragma unroll
    for (int rd = 0; rd < ROUNDS; ++rd) {
      const int idx = threadIdx.x + rd * SK_WAVES * WAVE;
      const int m = ((idx >> 8) % MT) * 16 + ((idx >> 4) & 15);
      const int n = n0 + ((idx >> 8) / MT) * 16 + (idx & 15);
      const bool live = idx < OUT_TILES * MT * 256 && m < M && n < n_end;
      pre_resid[rd] = res.resid[live ? (size_t)m * res.ldr + n : 0];
      pre_nw[rd] = 1.f;
      pre_nw16[rd] = (bf16)1.f;
      if (res.norm_w != nullptr) {  // uniform
        if (res.norm_w_f32)
          pre_nw[rd] = ((const float*)res.norm_w)[live ? n : 0];
        else
          pre_nw16[rd] = ((const bf16*)res.norm_w)[live ? n : 0];
      }
    }
  }

  // ---- the weight stream --------------------------------------------------
  // K in groups of 128.  A load instruction takes 4 rows x 256 contiguous bytes (16 lanes of 16 bytes a
  // row): runs that long are what the memory system streams at full rate, where the MFMA operand layout
  // (16 rows x 64 bytes) reaches two thirds of it.  The group goes through the wave's own LDS region to
  // change layout: written as loaded, read back as MFMA operands (lane (r, g) takes row r, k-step s at
  // 16-byte piece 4 s + g).  Pieces are XOR-swizzled with the row so that both directions spread over
  // the banks.  Weights are loaded non-temporally: they are read once.
  const int lrow = lane >> 4, seg = lane & 15;
  bf16* const stage_w = reinterpret_cast<bf16*>(stage + (size_t)wave * STAGE_BYTES);
  bf16* const stage_x = stage_w + 2048;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int i = lane; i < 256; i += WAVE) *reinterpret_cast<bf16x8*>(stage_x + i * 8) = zero;

  f32x4 acc[NTB][MT];
#pragma unroll
  for (int i = 0; i < NTB; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int ngroups = (K + 127) / 128;
  for (int c0 = wave * UNR; c0 < ngroups; c0 += SK_WAVES * UNR) {
    bf16x8 wreg[UNR][NTB][4], xreg[UNR][MT][4];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int k = (c0 + u) * 128 + seg * 8;
      const bool kok = k < K;
#pragma unroll
      for (int t = 0; t < NTB; ++t) {
        const int nbase = n0 + (t == 0 ? 0 : (GATED ? tile2_offset : 16 * t));
        const int limit = GATED && t == 1 ? tile2_offset + n_end : n_end;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          // a row past the block's last is read from the first row of the block's half, which is always there
          // (the tile's own first row may lie past the end of W when the last block is short; its sums are never
          // stored), a piece past K from the row's start (it meets zeros of x)
          const int n = nbase + 4 * q + lrow;
          const int first = GATED && t == 1 ? tile2_offset + n0 : n0;
          const size_t at = (size_t)(n < limit ? n : first) * K + (kok ? k : 0);
          wreg[u][t][q] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(w + at));
        }
      }
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int m = t * 16 + 4 * q + lrow;
          if (t * 16 + 4 * q < M)  // uniform: whole instructions fall away for few rows
            xreg[u][t][q] = *reinterpret_cast<const bf16x8*>(x + (size_t)(m < M ? m : 0) * ldx + (kok ? k : 0));
        }
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      if (c0 + u >= ngroups) break;  // uniform
      // the wave's two 4 KB regions are its own: LDS operations of one wave keep their order, so a tile
      // may overwrite the one before it as soon as that one's reads are issued
      bf16x8 a[NTB][4];
#pragma unroll
      for (int t = 0; t < NTB; ++t) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int row = 4 * q + lrow;
          *reinterpret_cast<bf16x8*>(stage_w + row * 128 + ((seg ^ row) & 15) * 8) = wreg[u][t][q];
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int st = 0; st < 4; ++st)
          a[t][st] = *reinterpret_cast<const bf16x8*>(stage_w + r * 128 + (((st * 4 + g) ^ r) & 15) * 8);
        __builtin_amdgcn_wave_barrier();
      }
#pragma unroll
      for (int j = 0; j < MT; ++j) {
        if (j * 16 >= M) break;  // uniform: the tile has no rows, its sums stay zero
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int row = 4 * q + lrow;
          const bool loaded = j * 16 + 4 * q < M;  // uniform
          if (MT == 1 && !loaded) continue;        // one tile only: its empty rows were zeroed at the start
          const bool inside = loaded && j * 16 + row < M && (c0 + u) * 128 + seg * 8 < K;
          *reinterpret_cast<bf16x8*>(stage_x + row * 128 + ((seg ^ row) & 15) * 8) = inside ? xreg[u][j][q] : zero;
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int st = 0; st < 4; ++st) {
          const bf16x8 bx = *reinterpret_cast<const bf16x8*>(stage_x + r * 128 + (((st * 4 + g) ^ r) & 15) * 8);
#pragma unroll
          for (int i = 0; i < NTB; ++i) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i][st], bx, acc[i][j], 0, 0, 0);
        }
        __builtin_amdgcn_wave_barrier();
      }
    }
  }

  // partial tiles meet in LDS, each wave's in its own region: [tile n][tile m][n row][m column (17)]
  {
    float* red_w = reinterpret_cast<float*>(stage + (size_t)wave * STAGE_BYTES);
#pragma unroll
    for (int i = 0; i < NTB; ++i)
#pragma unroll
      for (int j = 0; j < MT; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) red_w[((i * MT + j) * 16 + g * 4 + e) * 17 + r] = acc[i][j][e];
  }

  if (scale.partials != nullptr) {
    // the rows' scales: partial sums in a fixed order, the same bits whatever the launch looks like
#pragma unroll
    for (int i = 0; i < PRE_ROWS; ++i) {
      const int m = wave + i * SK_WAVES;
      if (m < M) {
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < PRE_DEPTH; ++j) sum += lane + j * WAVE < scale.count ? pre[i][j] : 0.f;
        for (int b = lane + PRE_DEPTH * WAVE; b < scale.count; b += WAVE) sum += scale.partials[(size_t)m * scale.count + b];
        sum = wave_sum(sum);
        if (lane == 0) s_scale[m] = rsqrtf(sum * scale.inv_width + scale.eps);
      }
    }
    for (int m = wave + PRE_ROWS * SK_WAVES; m < M; m += SK_WAVES) {
      float sum = 0.f;
      for (int b = lane; b < scale.count; b += WAVE) sum += scale.partials[(size_t)m * scale.count + b];
      sum = wave_sum(sum);
      if (lane == 0) s_scale[m] = rsqrtf(sum * scale.inv_width + scale.eps);
    }
  }
  __syncthreads();

  // every thread of a wave runs the same number of rounds (the rotation reads its neighbour's value)
#pragma unroll
  for (int rd = 0; rd < ROUNDS; ++rd) {
    const int idx = threadIdx.x + rd * SK_WAVES * WAVE;
    if (idx >= OUT_TILES * MT * 256) break;  // whole waves leave together: the tile count is a multiple of 64
    const int nn = idx & 15;           // n within tile: fastest, so that stores of a row are contiguous
    const int mm = (idx >> 4) & 15;    // m within tile
    const int tj = (idx >> 8) % MT;    // m tile
    const int ti = (idx >> 8) / MT;    // n tile
    const int m = tj * 16 + mm;
    const int n = n0 + ti * 16 + nn;
    const bool live = m < M && n < n_end;
    float v = 0.f;
#pragma unroll
    for (int wv = 0; wv < SK_WAVES; ++wv)
      v += reinterpret_cast<const float*>(stage + (size_t)wv * STAGE_BYTES)[((ti * MT + tj) * 16 + nn) * 17 + mm];
    const float row_scale = (scale.partials != nullptr && m < M) ? s_scale[m] : 1.f;
    v *= row_scale;
    if (EPI == EPI_GATED) {
      if (!live) continue;
      float u = 0.f;
#pragma unroll
      for (int wv = 0; wv < SK_WAVES; ++wv)
        u += reinterpret_cast<const float*>(stage + (size_t)wv * STAGE_BYTES)[((1 * MT + tj) * 16 + nn) * 17 + mm];
      u *= row_scale;
      if (bias) {
        v += to_f32(bias[n]);
        u += to_f32(bias[tile2_offset + n]);
      }
      out[(size_t)m * ldo + n] = from_f32<OutT>(sk_activate(v, act) * u);
    } else if (EPI == EPI_ROPE) {
      if (bias && live) v += to_f32(bias[n]);
      const float partner = __shfl_xor(v, 1, WAVE);  // the other element of the rotary pair: N is a multiple of 16
      if (!live) continue;
      const int D = rope.head_dim;
      const int hh = n / D, d = n - hh * D;
      const int pos = s_pos[m], seq = s_seq[m];
      if (rope.cos_t != nullptr && hh < rope.nheads + rope.kvheads && d < rope.rot_dim) {
        const float c = pre_resid[rd], sn = pre_nw[rd];
        v = (d & 1) ? sn * partner + c * v : c * v - sn * partner;
      }
      if (hh < rope.nheads) {
        out[(size_t)m * ldo + n] = from_f32<OutT>(v);
      } else if (seq >= 0 && rope.k_cache != nullptr && s_page[m] >= 0) {
        const size_t page_elems = (size_t)rope.kvheads * PAGE_TOKENS * D;
        const int in_page = pos % PAGE_TOKENS;
        if (hh < rope.nheads + rope.kvheads) {
          const int kh = hh - rope.nheads;
          rope.k_cache[(size_t)s_page[m] * page_elems + ((size_t)kh * PAGE_TOKENS + in_page) * D + d] = (bf16)v;
        } else {
          const int kh = hh - rope.nheads - rope.kvheads;
          rope.v_cache[(size_t)s_page[m] * page_elems + ((size_t)kh * D + d) * PAGE_TOKENS + in_page] = (bf16)v;
        }
      }
    } else if (EPI == EPI_RESID) {
      float stream = 0.f;
      if (live) {
        if (bias) v += to_f32(bias[n]);
        stream = pre_resid[rd] + v;
        res.resid[(size_t)m * res.ldr + n] = stream;
        const float nw = (res.norm_w != nullptr && !res.norm_w_f32) ? to_f32(pre_nw16[rd]) : pre_nw[rd];
        out[(size_t)m * ldo + n] = from_f32<OutT>(stream * nw);
      }
      // the 16 columns of a tile sit in 16 neighbouring lanes
      float sq = stream * stream;
#pragma unroll
      for (int off = 8; off > 0; off >>= 1) sq += __shfl_xor(sq, off, WAVE);
      if (nn == 0 && m < M) res.partials[(size_t)m * res.tiles + blockIdx.x * NTB + ti] = sq;  // 0 for an empty tile
    } else {
      if (!live) continue;
      if (bias) v += to_f32(bias[n]);
      out[(size_t)m * ldo + n] = from_f32<OutT>(v);
    }
  }
}

template <int NTB, int MT, int EPI>
static void launch_skinny(const void* x, long ldx, const void* w, const void* bias, int bias_dtype, void* out,
                          int out_dtype, long ldo, int M, int N, int K, int tile2_offset, int act, int rows_per_block,
                          hipStream_t stream, RowScale scale, RopeEpilogue rope = RopeEpilogue{},
                          ResidEpilogue res = ResidEpilogue{}) {
  const int blocks = ceil_div(N, rows_per_block);
  const bool fb = bias != nullptr && bias_dtype == FMS_F32;
  constexpr int SK_WAVES = 8;
  constexpr int UNR = (NTB + MT) <= 2 ? 2 : 1;
#define FMS_SK(O, B)                                                                                 \
  skinny_bf16_kernel<SK_WAVES, UNR, NTB, MT, EPI, O, B><<<blocks, SK_WAVES * WAVE, 0, stream>>>(     \
      (const bf16*)x, ldx, (const bf16*)w, (const B*)bias, (O*)out, ldo, M, N, K, tile2_offset, act, rows_per_block,  \
      scale, rope, res)
  if (out_dtype == FMS_BF16) {
    if (fb)
      FMS_SK(bf16, float);
    else
      FMS_SK(bf16, bf16);
  } else if (EPI != EPI_ROPE && EPI != EPI_RESID) {
    if (fb)
      FMS_SK(float, float);
    else
      FMS_SK(float, bf16);
  }
#undef FMS_SK
}

// Rows of W per block.  The blocks are dealt over the compute units (one or two at a time on each, sharing its
// path to memory), and what a unit has to pull decides the time: its blocks' weight rows and, per block, the
// rows of x (read four rows an instruction).  The choice with the least of
//   blocks per unit (a whole number) x (rows of W + rows of x per block)
// wins: 6144 rows in blocks of 24 are one block a unit where blocks of 16 are one and a half; the gated product
// of 14336 columns in blocks of 14 gate rows and 14 up rows is four blocks a unit of 28 rows where blocks of 16
// and 16 are three and a half - that is, four for some - of 32.
#define SK_COMPUTE_UNITS 256
static int skinny_x_rows(int M) { return ceil_div(M, 4) * 4; }

// 17 to 32 rows of x and a short K: the kernel above with two tiles of x a wave beats the kernels of
// gemm_wide.hip, which have to cut so short a K into slices that meet in memory and need a second kernel
// (measured at K = 4096: 13.5 against 17.2 us for 6144 weight rows, 11.3 against 14.5 for 4096; at K = 14336, and
// from 33 rows on, where every block reads more of x than of W, the wide kernels win).
static bool skinny_takes_many_rows(int M, int N, int K) { return M > 16 && M <= 32 && K <= 8192; }

static int skinny_rows_per_block(int N, int M) {
  int best = 0;
  long best_cost = 0;
  for (int rows = 12; rows <= 32; rows += 2) {
    const long cost = (long)ceil_div(ceil_div(N, rows), SK_COMPUTE_UNITS) * (rows + skinny_x_rows(M));
    if (best == 0 || cost <= best_cost) best = rows, best_cost = cost;  // a tie goes to the larger blocks
  }
  return best;
}

// gate rows (and as many up rows) per block of the gated product
static int skinny_gated_rows_per_block(int hidden, int M) {
  int best = 0;
  long best_cost = 0;
  for (int rows = 12; rows <= 16; ++rows) {
    const long cost = (long)ceil_div(ceil_div(hidden, rows), SK_COMPUTE_UNITS) * (2 * rows + skinny_x_rows(M));
    if (best == 0 || cost <= best_cost) best = rows, best_cost = cost;
  }
  return best;
}

// Checks a deferred row norm and turns it into the kernel's argument.
static int row_scale_of(const fmsamd_row_scale* in, int K, RowScale* out) {
  *out = RowScale{nullptr, 0, 0.f, 0.f};
  if (in == nullptr || in->partials == nullptr) return 0;
  FMS_REQUIRE(in->count > 0 && in->eps >= 0.f, "deferred row norm: %d partial sums, eps %g", in->count, (double)in->eps);
  *out = RowScale{in->partials, in->count, 1.f / (float)K, in->eps};
  return 0;
}

// out[M, N] = x[M, K] w[N, K]^T (+ bias).  M <= 192.
extern "C" int fmsamd_gemm_skinny_bf16(const void* x, long ldx, const void* w, const void* bias, int bias_dtype,
                                       void* out, int out_dtype, long ldo, int M, int N, int K,
                                       const fmsamd_row_scale* row_scale, void* workspace, long workspace_bytes,
                                       hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  RowScale scale;
  if (row_scale_of(row_scale, K, &scale)) return -1;
  FMS_REQUIRE(M > 0 && M <= FMS_SKINNY_MAX_ROWS && N > 0 && K > 0, "gemm_skinny_bf16: bad sizes M=%d N=%d K=%d (M <= 192)", M, N, K);
  FMS_REQUIRE(K % 8 == 0 && ldx % 8 == 0, "gemm_skinny_bf16: K=%d and the row stride %ld must be multiples of 8", K, ldx);
  FMS_REQUIRE(ldx >= K && ldo >= N, "gemm_skinny_bf16: leading dimensions too small");
  FMS_REQUIRE(out_dtype == FMS_BF16 || out_dtype == FMS_F32, "gemm_skinny_bf16: unknown output dtype %d", out_dtype);
  if (M > 16 && !skinny_takes_many_rows(M, N, K))
    return wide_product(EPI_PLAIN, x, ldx, w, bias, bias_dtype, out, out_dtype, ldo, M, N, K, 0, 0, scale, RopeEpilogue{},
                        ResidEpilogue{}, workspace, workspace_bytes, stream);
  const int rows = skinny_rows_per_block(N, M);
#define FMS_LS(NTB, MT) \
  launch_skinny<NTB, MT, EPI_PLAIN>(x, ldx, w, bias, bias_dtype, out, out_dtype, ldo, M, N, K, 0, 0, rows, stream, scale)
#define FMS_LS_MT(NTB)  \
  do {                  \
    if (M <= 16)        \
      FMS_LS(NTB, 1);   \
    else                \
      FMS_LS(NTB, 2);   \
  } while (0)
  if (rows > 16)
    FMS_LS_MT(2);
  else
    FMS_LS_MT(1);
#undef FMS_LS_MT
#undef FMS_LS
  FMS_LAUNCH_CHECK("gemm_skinny_bf16");
  return 0;
}

// out[M, hidden] = act(x Wg^T + bg) * (x Wu^T + bu) with w = [Wg; Wu] stacked, [2*hidden, K].  M <= 192.
extern "C" int fmsamd_gemm_skinny_gated_bf16(const void* x, long ldx, const void* w, const void* bias,
                                             int bias_dtype, void* out, int out_dtype, long ldo, int M, int hidden,
                                             int K, int act, const fmsamd_row_scale* row_scale, void* workspace,
                                             long workspace_bytes, hipStream_t stream) {
  if (M == 0 || hidden == 0) return 0;
  RowScale scale;
  if (row_scale_of(row_scale, K, &scale)) return -1;
  FMS_REQUIRE(M > 0 && M <= FMS_SKINNY_MAX_ROWS && hidden > 0 && K > 0, "gemm_skinny_gated_bf16: bad sizes M=%d hidden=%d K=%d (M <= 192)",
              M, hidden, K);
  FMS_REQUIRE(K % 8 == 0 && ldx % 8 == 0, "gemm_skinny_gated_bf16: K=%d and the row stride %ld must be multiples of 8", K,
              ldx);
  FMS_REQUIRE(ldx >= K && ldo >= hidden, "gemm_skinny_gated_bf16: leading dimensions too small");
  FMS_REQUIRE(out_dtype == FMS_BF16 || out_dtype == FMS_F32, "gemm_skinny_gated_bf16: unknown output dtype %d", out_dtype);
  FMS_REQUIRE(act >= FMS_ACT_SILU && act <= FMS_ACT_LAST, "gemm_skinny_gated_bf16: unknown activation %d", act);
  if (M > 16)
    return wide_product(EPI_GATED, x, ldx, w, bias, bias_dtype, out, out_dtype, ldo, M, hidden, K, hidden, act, scale,
                        RopeEpilogue{}, ResidEpilogue{}, workspace, workspace_bytes, stream);
#define FMS_LG(MT) \
  launch_skinny<2, MT, EPI_GATED>(x, ldx, w, bias, bias_dtype, out, out_dtype, ldo, M, hidden, K, hidden, act,     \
                                  skinny_gated_rows_per_block(hidden, M), stream, scale)
  FMS_LG(1);
#undef FMS_LG
  FMS_LAUNCH_CHECK("gemm_skinny_gated_bf16");
  return 0;
}

// qkv[M, (H+2K)*D] = x W^T (+ bias) with the rotation of q and k and the cache write of k and v fused into
// the epilogue: the decode-time twin of fmsamd_gemm_skinny_bf16 followed by fmsamd_rope_kv_write.  Only the
// query columns of `out` are written.  M <= 192.
extern "C" int fmsamd_qkv_rope_skinny_bf16(const void* x, long ldx, const void* w, const void* bias, int bias_dtype,
                                           void* out, long ldo, int M, int K, const int* positions,
                                           const int* seq_of_token, const int* block_table, int table_stride,
                                           const float* cos_t, const float* sin_t, int rot_dim, int max_pos,
                                           void* k_cache, void* v_cache, int nheads, int kvheads, int head_dim,
                                           const fmsamd_row_scale* row_scale, void* workspace, long workspace_bytes,
                                           hipStream_t stream) {
  if (M == 0) return 0;
  const int N = (nheads + 2 * kvheads) * head_dim;
  RowScale scale;
  if (row_scale_of(row_scale, K, &scale)) return -1;
  FMS_REQUIRE(M > 0 && M <= FMS_SKINNY_MAX_ROWS && K > 0 && nheads > 0 && kvheads > 0 && head_dim > 0,
              "qkv_rope_skinny_bf16: bad sizes M=%d K=%d (M <= 192)", M, K);
  FMS_REQUIRE(K % 8 == 0 && ldx % 8 == 0, "qkv_rope_skinny_bf16: K=%d and the row stride %ld must be multiples of 8", K, ldx);
  FMS_REQUIRE(ldx >= K && ldo >= N, "qkv_rope_skinny_bf16: leading dimensions too small");
  FMS_REQUIRE(head_dim % 2 == 0 && N % 16 == 0, "qkv_rope_skinny_bf16: head size %d must be even and the row a multiple of 16",
              head_dim);
  FMS_REQUIRE(rot_dim % 2 == 0 && rot_dim >= 0 && rot_dim <= head_dim, "qkv_rope_skinny_bf16: rotary size %d does not fit",
              rot_dim);
  FMS_REQUIRE((k_cache == nullptr) == (v_cache == nullptr), "qkv_rope_skinny_bf16: key and value cache must come together");
  FMS_REQUIRE(cos_t == nullptr || (max_pos > 0 && sin_t != nullptr), "qkv_rope_skinny_bf16: empty rotary table");
  RopeEpilogue rope{positions, seq_of_token, block_table, table_stride, rot_dim > 0 ? cos_t : nullptr, sin_t, rot_dim,
                    max_pos, (bf16*)k_cache, (bf16*)v_cache, nheads, kvheads, head_dim};
  if (M > 16 && !skinny_takes_many_rows(M, N, K))
    return wide_product(EPI_ROPE, x, ldx, w, bias, bias_dtype, out, FMS_BF16, ldo, M, N, K, 0, 0, scale, rope,
                        ResidEpilogue{}, workspace, workspace_bytes, stream);
  const int rows = skinny_rows_per_block(N, M);
#define FMS_LR(NTB, MT) \
  launch_skinny<NTB, MT, EPI_ROPE>(x, ldx, w, bias, bias_dtype, out, FMS_BF16, ldo, M, N, K, 0, 0, rows, stream, scale, rope)
#define FMS_LR_MT(NTB)  \
  do {                  \
    if (M <= 16)        \
      FMS_LR(NTB, 1);   \
    else                \
      FMS_LR(NTB, 2);   \
  } while (0)
  if (rows > 16)
    FMS_LR_MT(2);
  else
    FMS_LR_MT(1);
#undef FMS_LR_MT
#undef FMS_LR
  FMS_LAUNCH_CHECK("qkv_rope_skinny_bf16");
  return 0;
}

// The last product of a residual branch, fused with what follows it in a pre-norm block:
//   resid[M, N] += x w^T (+ bias)                      float32, in place
//   scaled[M, N] = resid * norm_w                      bfloat16: the next norm's input, not yet divided by its
//                                                      root mean square
//   partials[m, i] = sums of resid[m]^2 over groups of up to 16 columns, the unused ones zero
//                    [M, partial_count], partial_count >= fmsamd_gemm_skinny_residual_partials(M, N, K)
// A product that takes `scaled` with these partials as its deferred row norm then equals the product of the
// normed stream.  M <= 192.
extern "C" int fmsamd_gemm_skinny_residual_partials(int M, int N, int K) {
  if (M > 16 && !skinny_takes_many_rows(M, N, K)) return ceil_div(N, 16);
  const int rows = skinny_rows_per_block(N, M);
  return ceil_div(N, rows) * (rows > 16 ? 2 : 1);
}

// Bytes of workspace that the products for at most 192 rows need (none up to 16 rows).  rows: all rows of W.
extern "C" long fmsamd_gemm_skinny_workspace(int M, int rows, int K) {
  return M > 16 && M <= FMS_SKINNY_MAX_ROWS ? wide_workspace_bytes(M, rows, K) : 0;  // enough for every product of this shape
}

extern "C" int fmsamd_gemm_skinny_residual_bf16(const void* x, long ldx, const void* w, const void* bias,
                                                int bias_dtype, float* resid, long ldr, const void* norm_w,
                                                int norm_w_dtype, void* scaled, long ldo, float* partials,
                                                int partial_count, int M, int N, int K,
                                                const fmsamd_row_scale* row_scale, void* workspace,
                                                long workspace_bytes, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  FMS_REQUIRE(M > 0 && M <= FMS_SKINNY_MAX_ROWS && N > 0 && K > 0, "gemm_skinny_residual_bf16: bad sizes M=%d N=%d K=%d (M <= 192)", M, N, K);
  FMS_REQUIRE(K % 8 == 0 && ldx % 8 == 0, "gemm_skinny_residual_bf16: K=%d and the row stride %ld must be multiples of 8",
              K, ldx);
  FMS_REQUIRE(ldx >= K && ldo >= N && ldr >= N, "gemm_skinny_residual_bf16: leading dimensions too small");
  FMS_REQUIRE(norm_w == nullptr || norm_w_dtype == FMS_BF16 || norm_w_dtype == FMS_F32,
              "gemm_skinny_residual_bf16: unknown norm weight dtype %d", norm_w_dtype);
  FMS_REQUIRE(resid != nullptr && scaled != nullptr && partials != nullptr, "gemm_skinny_residual_bf16: null buffer");
  RowScale scale;
  if (row_scale_of(row_scale, K, &scale)) return -1;
  const int rows = skinny_rows_per_block(N, M);
  const int tiles = fmsamd_gemm_skinny_residual_partials(M, N, K);
  FMS_REQUIRE(partial_count >= tiles, "gemm_skinny_residual_bf16: room for %d partial sums per row, %d needed",
              partial_count, tiles);
  ResidEpilogue res{resid, ldr, norm_w, norm_w_dtype == FMS_F32, partials, partial_count};
  if (M > 16 && !skinny_takes_many_rows(M, N, K)) {
    res.tiles = tiles;  // the finish kernel writes exactly these
    FMS_REQUIRE(partial_count == tiles, "gemm_skinny_residual_bf16: %d partial sums per row, %d expected", partial_count,
                tiles);
    return wide_product(EPI_RESID, x, ldx, w, bias, bias_dtype, scaled, FMS_BF16, ldo, M, N, K, 0, 0, scale,
                        RopeEpilogue{}, res, workspace, workspace_bytes, stream);
  }
#define FMS_LX(NTB, MT)                                                                                              \
  launch_skinny<NTB, MT, EPI_RESID>(x, ldx, w, bias, bias_dtype, scaled, FMS_BF16, ldo, M, N, K, 0, 0, rows, stream, \
                                    scale, RopeEpilogue{}, res)
#define FMS_LX_MT(NTB)  \
  do {                  \
    if (M <= 16)        \
      FMS_LX(NTB, 1);   \
    else                \
      FMS_LX(NTB, 2);   \
  } while (0)
  if (rows > 16)
    FMS_LX_MT(2);
  else
    FMS_LX_MT(1);
#undef FMS_LX_MT
#undef FMS_LX
  FMS_LAUNCH_CHECK("gemm_skinny_residual_bf16");
  return 0;
}
