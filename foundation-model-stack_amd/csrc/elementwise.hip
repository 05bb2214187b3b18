// Embedding gather, residual-add + norm, gated activation, casts and bias adds.
// All statistics and sums are float32; storage types are template parameters.
#include <stdarg.h>
#include <stdio.h>

#include "common.h"
#include "fmsamd.h"

// --------------------------------------------------------------------------
// error string
// --------------------------------------------------------------------------
static thread_local char g_error[512] = "";

void fmsamd_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

extern "C" const char* fmsamd_last_error() { return g_error; }

extern "C" int fmsamd_abi_version() { return FMSAMD_ABI_VERSION; }

// --------------------------------------------------------------------------
// embedding: resid[t, :] = float(table[ids[t], :])
// --------------------------------------------------------------------------
template <typename TableT>
__global__ void embed_kernel(const int* __restrict__ ids, const TableT* __restrict__ table, float* __restrict__ out,
                             int width, int vocab) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);  // the host has checked the range; never read outside
  const TableT* row = table + (size_t)id * width;
  float* o = out + (size_t)t * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) o[i] = to_f32(row[i]);
}

extern "C" int fmsamd_embed(const int* ids, const void* table, int table_dtype, float* out, int n_tokens, int width,
                            int vocab, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && width > 0 && vocab > 0, "embed: bad sizes T=%d width=%d vocab=%d", n_tokens, width, vocab);
  const int threads = width >= 1024 ? 256 : 64;
  if (table_dtype == FMS_F32)
    embed_kernel<float><<<n_tokens, threads, 0, stream>>>(ids, (const float*)table, out, width, vocab);
  else if (table_dtype == FMS_BF16)
    embed_kernel<bf16><<<n_tokens, threads, 0, stream>>>(ids, (const bf16*)table, out, width, vocab);
  else
    FMS_REQUIRE(false, "embed: unknown table dtype %d", table_dtype);
  FMS_LAUNCH_CHECK("embed");
  return 0;
}

// --------------------------------------------------------------------------
// add + norm.  One block per output row.
//   s = resid[r] (+ branch[r])            float32 sum, written back to resid
//   s = s - mean(s)                       if use_mean
//   y = s * rsqrt(mean(s^2) + eps) (* weight) (+ bias)
// With `rows`, output row i is computed from stream row rows[i] and the
// residual is not written back (the stream is not used again).
// --------------------------------------------------------------------------
// VEC consecutive elements as float, from float or bfloat16 storage
template <int VEC, typename T>
__device__ __forceinline__ void load_vec(const T* p, float (&v)[VEC]) {
  if constexpr (VEC == 4 && sizeof(T) == 4) {
    const f32x4 t = *reinterpret_cast<const f32x4*>(p);
    v[0] = t[0], v[1] = t[1], v[2] = t[2], v[3] = t[3];
  } else if constexpr (VEC == 4 && sizeof(T) == 2) {
    const bf16x4 t = *reinterpret_cast<const bf16x4*>(p);
    v[0] = (float)t[0], v[1] = (float)t[1], v[2] = (float)t[2], v[3] = (float)t[3];
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = to_f32(p[i]);
  }
}

template <int VEC, typename T>
__device__ __forceinline__ void store_vec(T* p, const float (&v)[VEC]) {
  if constexpr (VEC == 4 && sizeof(T) == 4) {
    *reinterpret_cast<f32x4*>(p) = f32x4{v[0], v[1], v[2], v[3]};
  } else if constexpr (VEC == 4 && sizeof(T) == 2) {
    *reinterpret_cast<bf16x4*>(p) = bf16x4{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) p[i] = from_f32<T>(v[i]);
  }
}

// A thread keeps KEEP vectors of VEC elements in registers (and their weights, fetched before the
// reduction so that they do not wait for it); a wider row is read again.  The loops over the kept
// values have compile-time trip counts: the arrays must never be indexed by a run-time value, or
// they are addressed through relative register indexing.
template <int VEC, typename BranchT, typename WeightT, typename OutT>
__global__ void __launch_bounds__(1024) add_norm_kernel(float* __restrict__ resid, const BranchT* __restrict__ branch,
                                                        const WeightT* __restrict__ weight,
                                                        const WeightT* __restrict__ bias, OutT* __restrict__ out,
                                                        const int* __restrict__ rows, int width, float eps,
                                                        int use_mean) {
  __shared__ float scratch[17];
  const int r = rows ? rows[blockIdx.x] : blockIdx.x;
  float* x = resid + (size_t)r * width;
  const BranchT* b = branch ? branch + (size_t)r * width : nullptr;
  OutT* o = out + (size_t)blockIdx.x * width;

  constexpr int KEEP = VEC == 4 ? 4 : 16;
  const int stride = blockDim.x * VEC;  // elements covered by the block in one sweep
  float keep[KEEP][VEC], wkeep[KEEP][VEC], bkeep[KEEP][VEC];
  const int tail = threadIdx.x * VEC + KEEP * stride;
  float sum = 0.f, sq = 0.f;
#pragma unroll
  for (int n = 0; n < KEEP; ++n) {
    const int i = threadIdx.x * VEC + n * stride;
#pragma unroll
    for (int e = 0; e < VEC; ++e) keep[n][e] = 0.f, wkeep[n][e] = 1.f, bkeep[n][e] = 0.f;
    if (i < width) {  // width is a multiple of VEC
      load_vec<VEC>(x + i, keep[n]);
      if (weight) load_vec<VEC>(weight + i, wkeep[n]);
      if (bias) load_vec<VEC>(bias + i, bkeep[n]);
      if (b) {
        float bv[VEC];
        load_vec<VEC>(b + i, bv);
#pragma unroll
        for (int e = 0; e < VEC; ++e) keep[n][e] += bv[e];
        if (!rows) store_vec<VEC>(x + i, keep[n]);
      }
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      sum += keep[n][e];
      sq += keep[n][e] * keep[n][e];
    }
  }
  for (int i = tail; i < width; i += stride) {
    float v[VEC];
    load_vec<VEC>(x + i, v);
    if (b) {
      float bv[VEC];
      load_vec<VEC>(b + i, bv);
#pragma unroll
      for (int e = 0; e < VEC; ++e) v[e] += bv[e];
      if (!rows) store_vec<VEC>(x + i, v);
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      sum += v[e];
      sq += v[e] * v[e];
    }
  }
  const bool reread_adds = rows != nullptr && b != nullptr;  // the stream was not updated: add again
  float mean = 0.f;
  if (use_mean) {
    mean = block_sum(sum, scratch) / (float)width;
    sq = 0.f;  // second moment about the mean
#pragma unroll
    for (int n = 0; n < KEEP; ++n) {
      const int i = threadIdx.x * VEC + n * stride;
      if (i < width) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) sq += (keep[n][e] - mean) * (keep[n][e] - mean);
      }
    }
    for (int i = tail; i < width; i += stride) {
      float v[VEC];
      load_vec<VEC>(x + i, v);
      if (reread_adds) {
        float bv[VEC];
        load_vec<VEC>(b + i, bv);
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[e] += bv[e];
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e) sq += (v[e] - mean) * (v[e] - mean);
    }
  }
  const float ms = block_sum(sq, scratch) / (float)width;
  const float scale = rsqrtf(ms + eps);
#pragma unroll
  for (int n = 0; n < KEEP; ++n) {
    const int i = threadIdx.x * VEC + n * stride;
    if (i < width) {
      float v[VEC];
#pragma unroll
      for (int e = 0; e < VEC; ++e) v[e] = (keep[n][e] - mean) * scale * wkeep[n][e] + bkeep[n][e];
      store_vec<VEC>(o + i, v);
    }
  }
  for (int i = tail; i < width; i += stride) {
    float v[VEC], wv[VEC], bv[VEC];
    load_vec<VEC>(x + i, v);
    if (reread_adds) {
      load_vec<VEC>(b + i, bv);
#pragma unroll
      for (int e = 0; e < VEC; ++e) v[e] += bv[e];
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) wv[e] = 1.f, bv[e] = 0.f;
    if (weight) load_vec<VEC>(weight + i, wv);
    if (bias) load_vec<VEC>(bias + i, bv);
#pragma unroll
    for (int e = 0; e < VEC; ++e) v[e] = (v[e] - mean) * scale * wv[e] + bv[e];
    store_vec<VEC>(o + i, v);
  }
}

template <typename BranchT, typename WeightT, typename OutT>
static void launch_add_norm(float* resid, const void* branch, const void* weight, const void* bias, void* out,
                            const int* rows, int n_out, int width, float eps, int use_mean, hipStream_t stream) {
  const bool aligned = (((size_t)resid | (size_t)branch | (size_t)weight | (size_t)bias | (size_t)out) & 15) == 0;
  if (width % 4 == 0 && aligned) {
    // 4 vectors of 4 per thread cover the row up to 16 elements per thread; wider rows take more threads
    int threads = (width / 16 + 63) / 64 * 64;
    threads = threads < 64 ? 64 : (threads > 1024 ? 1024 : threads);
    add_norm_kernel<4, BranchT, WeightT, OutT><<<n_out, threads, 0, stream>>>(
        resid, (const BranchT*)branch, (const WeightT*)weight, (const WeightT*)bias, (OutT*)out, rows, width, eps,
        use_mean);
  } else {
    const int threads = width > 4096 ? 1024 : (width >= 2048 ? 256 : (width >= 512 ? 128 : 64));
    add_norm_kernel<1, BranchT, WeightT, OutT><<<n_out, threads, 0, stream>>>(
        resid, (const BranchT*)branch, (const WeightT*)weight, (const WeightT*)bias, (OutT*)out, rows, width, eps,
        use_mean);
  }
}

extern "C" int fmsamd_add_norm(float* resid, const void* branch, int act_dtype, const void* weight, const void* bias,
                               int weight_dtype, void* out, const int* rows, int n_out, int width, float eps,
                               int use_mean, hipStream_t stream) {
  if (n_out == 0) return 0;
  FMS_REQUIRE(n_out > 0 && width > 0, "add_norm: bad sizes rows=%d width=%d", n_out, width);
  FMS_REQUIRE(eps >= 0.f, "add_norm: eps %g is negative", (double)eps);
#define FMS_AN(B, W, O)                                                                               \
  launch_add_norm<B, W, O>(resid, branch, weight, bias, out, rows, n_out, width, eps, use_mean, stream)
  if (act_dtype == FMS_F32 && weight_dtype == FMS_F32)
    FMS_AN(float, float, float);
  else if (act_dtype == FMS_BF16 && weight_dtype == FMS_BF16)
    FMS_AN(bf16, bf16, bf16);
  else if (act_dtype == FMS_BF16 && weight_dtype == FMS_F32)
    FMS_AN(bf16, float, bf16);
  else if (act_dtype == FMS_F32 && weight_dtype == FMS_BF16)
    FMS_AN(float, bf16, float);
  else
    FMS_REQUIRE(false, "add_norm: unknown dtypes act=%d weight=%d", act_dtype, weight_dtype);
#undef FMS_AN
  FMS_LAUNCH_CHECK("add_norm");
  return 0;
}

// --------------------------------------------------------------------------
// gated activation: out[t, j] = act(gu[t, j] + bg[j]) * (gu[t, hidden + j] + bu[j])
// --------------------------------------------------------------------------
__device__ __forceinline__ float activate(float x, int kind) { return fms_activate(x, kind); }

// VEC elements per thread and step: 16 bytes of the activation type when the row length allows it
template <int VEC, typename T, typename BiasT>
__global__ void gated_act_kernel(const T* __restrict__ gu, const BiasT* __restrict__ bias, T* __restrict__ out,
                                 int hidden, int act) {
  const size_t t = blockIdx.y;
  const T* g = gu + t * 2 * hidden;
  const T* u = g + hidden;
  T* o = out + t * hidden;
  for (int j = (blockIdx.x * blockDim.x + threadIdx.x) * VEC; j < hidden; j += gridDim.x * blockDim.x * VEC) {
    __attribute__((aligned(16))) T gv[VEC], uv[VEC], ov[VEC];
    if constexpr (VEC * sizeof(T) == 16) {
      *reinterpret_cast<f32x4*>(gv) = *reinterpret_cast<const f32x4*>(g + j);
      *reinterpret_cast<f32x4*>(uv) = *reinterpret_cast<const f32x4*>(u + j);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) gv[e] = g[j + e], uv[e] = u[j + e];
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      float a = to_f32(gv[e]), b = to_f32(uv[e]);
      if (bias) {
        a += to_f32(bias[j + e]);
        b += to_f32(bias[hidden + j + e]);
      }
      ov[e] = from_f32<T>(activate(a, act) * b);
    }
    if constexpr (VEC * sizeof(T) == 16) {
      *reinterpret_cast<f32x4*>(o + j) = *reinterpret_cast<const f32x4*>(ov);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) o[j + e] = ov[e];
    }
  }
}

template <typename T, typename BiasT>
static void launch_gated_act(const void* gu, const void* bias, void* out, int n_tokens, int hidden, int act,
                             hipStream_t stream) {
  constexpr int VEC = 16 / sizeof(T);
  const bool wide = hidden % VEC == 0 && (((size_t)gu | (size_t)out) & 15) == 0;
  const int per_thread = wide ? VEC : 1;
  const int blocks = ceil_div(hidden, 256 * per_thread);
  dim3 grid(blocks > 64 ? 64 : blocks, n_tokens);
  if (wide)
    gated_act_kernel<VEC, T, BiasT><<<grid, 256, 0, stream>>>((const T*)gu, (const BiasT*)bias, (T*)out, hidden, act);
  else
    gated_act_kernel<1, T, BiasT><<<grid, 256, 0, stream>>>((const T*)gu, (const BiasT*)bias, (T*)out, hidden, act);
}

extern "C" int fmsamd_gated_act(const void* gu, const void* bias, int bias_dtype, void* out, int dtype, int n_tokens,
                                int hidden, int act, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && hidden > 0, "gated_act: bad sizes T=%d hidden=%d", n_tokens, hidden);
  FMS_REQUIRE(act >= FMS_ACT_SILU && act <= FMS_ACT_LAST, "gated_act: unknown activation %d", act);
  FMS_REQUIRE(n_tokens <= 65535, "gated_act: %d tokens exceed one launch (65535)", n_tokens);
  if (dtype == FMS_F32 && (bias == nullptr || bias_dtype == FMS_F32))
    launch_gated_act<float, float>(gu, bias, out, n_tokens, hidden, act, stream);
  else if (dtype == FMS_BF16 && (bias == nullptr || bias_dtype == FMS_BF16))
    launch_gated_act<bf16, bf16>(gu, bias, out, n_tokens, hidden, act, stream);
  else if (dtype == FMS_BF16 && bias_dtype == FMS_F32)
    launch_gated_act<bf16, float>(gu, bias, out, n_tokens, hidden, act, stream);
  else if (dtype == FMS_F32 && bias_dtype == FMS_BF16)
    launch_gated_act<float, bf16>(gu, bias, out, n_tokens, hidden, act, stream);
  else
    FMS_REQUIRE(false, "gated_act: unknown dtypes %d/%d", dtype, bias_dtype);
  FMS_LAUNCH_CHECK("gated_act");
  return 0;
}

// --------------------------------------------------------------------------
// cast and bias add
// --------------------------------------------------------------------------
template <typename A, typename B>
__global__ void cast_kernel(const A* __restrict__ in, B* __restrict__ out, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    out[i] = from_f32<B>(to_f32(in[i]));
}

extern "C" int fmsamd_cast(const void* in, int in_dtype, void* out, int out_dtype, long n, hipStream_t stream) {
  if (n == 0) return 0;
  FMS_REQUIRE(n > 0, "cast: negative count");
  const int blocks = ceil_div(n, 256) > 4096 ? 4096 : ceil_div(n, 256);
  if (in_dtype == FMS_F32 && out_dtype == FMS_BF16)
    cast_kernel<float, bf16><<<blocks, 256, 0, stream>>>((const float*)in, (bf16*)out, (size_t)n);
  else if (in_dtype == FMS_BF16 && out_dtype == FMS_F32)
    cast_kernel<bf16, float><<<blocks, 256, 0, stream>>>((const bf16*)in, (float*)out, (size_t)n);
  else
    FMS_REQUIRE(false, "cast: unsupported %d -> %d", in_dtype, out_dtype);
  FMS_LAUNCH_CHECK("cast");
  return 0;
}

template <typename T, typename BiasT>
__global__ void bias_add_kernel(T* __restrict__ x, const BiasT* __restrict__ bias, int cols) {
  T* row = x + (size_t)blockIdx.x * cols;
  for (int j = threadIdx.x; j < cols; j += blockDim.x) row[j] = from_f32<T>(to_f32(row[j]) + to_f32(bias[j]));
}

extern "C" int fmsamd_bias_add(void* x, int dtype, const void* bias, int bias_dtype, int rows, int cols,
                               hipStream_t stream) {
  if (rows == 0) return 0;
  FMS_REQUIRE(rows > 0 && cols > 0, "bias_add: bad sizes");
  if (dtype == FMS_F32 && bias_dtype == FMS_F32)
    bias_add_kernel<float, float><<<rows, 256, 0, stream>>>((float*)x, (const float*)bias, cols);
  else if (dtype == FMS_BF16 && bias_dtype == FMS_BF16)
    bias_add_kernel<bf16, bf16><<<rows, 256, 0, stream>>>((bf16*)x, (const bf16*)bias, cols);
  else if (dtype == FMS_BF16 && bias_dtype == FMS_F32)
    bias_add_kernel<bf16, float><<<rows, 256, 0, stream>>>((bf16*)x, (const float*)bias, cols);
  else if (dtype == FMS_F32 && bias_dtype == FMS_BF16)
    bias_add_kernel<float, bf16><<<rows, 256, 0, stream>>>((float*)x, (const bf16*)bias, cols);
  else
    FMS_REQUIRE(false, "bias_add: unknown dtypes");
  FMS_LAUNCH_CHECK("bias_add");
  return 0;
}

// --------------------------------------------------------------------------
// positions[i] += 1 for the live rows of a fixed-size decode batch, so that a
// captured step can be replayed without the host touching its index data
// --------------------------------------------------------------------------
__global__ void advance_positions_kernel(int* __restrict__ positions, const int* __restrict__ seq_of_token, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n && seq_of_token[i] >= 0) positions[i] += 1;
}

extern "C" int fmsamd_advance_positions(int* positions, const int* seq_of_token, int n, hipStream_t stream) {
  if (n == 0) return 0;
  FMS_REQUIRE(n > 0, "advance_positions: negative count");
  advance_positions_kernel<<<ceil_div(n, 256), 256, 0, stream>>>(positions, seq_of_token, n);
  FMS_LAUNCH_CHECK("advance_positions");
  return 0;
}
