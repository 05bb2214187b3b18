// Shared device helpers for the gfx950 kernels: types, wave and block
// reductions, launch checking.  Wavefronts are 64 lanes wide throughout.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16;
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define WAVE 64

// Tokens per cache page.  The Python side (cache/pages.py) uses the same number.
#define PAGE_TOKENS 64

// --------------------------------------------------------------------------
// error reporting: every entry point returns 0 or a negative code and leaves a
// message that fmsamd_last_error() returns.
// --------------------------------------------------------------------------
void fmsamd_set_error(const char* fmt, ...);

#define FMS_REQUIRE(cond, ...)          \
  do {                                  \
    if (!(cond)) {                      \
      fmsamd_set_error(__VA_ARGS__);    \
      return -1;                        \
    }                                   \
  } while (0)

#define FMS_LAUNCH_CHECK(name)                                                   \
  do {                                                                           \
    hipError_t e_ = hipGetLastError();                                           \
    if (e_ != hipSuccess) {                                                      \
      fmsamd_set_error("%s: launch failed: %s", name, hipGetErrorString(e_));    \
      return -2;                                                                 \
    }                                                                            \
  } while (0)

// A block-table entry below zero marks a page that is not there: never handed out, or given back by a window.
// No kernel needs such a page for a key it can see or a token it writes; if the host's bookkeeping is ever
// wrong, a read goes to page 0 and a write is dropped, instead of leaving the cache's memory.
__device__ __forceinline__ size_t readable_page(int entry) { return entry < 0 ? 0 : (size_t)entry; }

// --------------------------------------------------------------------------
// conversions
// --------------------------------------------------------------------------
__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(bf16 x) { return (float)x; }

template <typename T>
__device__ __forceinline__ T from_f32(float x);
template <>
__device__ __forceinline__ float from_f32<float>(float x) {
  return x;
}
template <>
__device__ __forceinline__ bf16 from_f32<bf16>(float x) {
  return (bf16)x;  // round to nearest even (v_cvt_pk_bf16_f32)
}

// --------------------------------------------------------------------------
// activation functions (the codes are FMS_ACT_* of fmsamd.h), in float32
// --------------------------------------------------------------------------
__device__ __forceinline__ float fms_activate(float x, int kind) {
  switch (kind) {
    case 0:  // silu
      return x / (1.f + expf(-x));
    case 1:  // gelu
      return 0.5f * x * (1.f + erff(x * 0.70710678118654752f));
    case 2:  // relu
      return fmaxf(x, 0.f);
    case 4:  // sigmoid
      return 1.f / (1.f + expf(-x));
    case 5:  // tanh
      return tanhf(x);
    case 6:  // mish; log(1 + e^x) is x itself beyond 20, as the reference's library has it
      return x * tanhf(x > 20.f ? x : log1pf(expf(x)));
    case 7:  // gelu, tanh approximation
      return 0.5f * x * (1.f + tanhf(0.79788456080286536f * (x + 0.044715f * x * x * x)));
    default:  // identity
      return x;
  }
}

// --------------------------------------------------------------------------
// reductions
// --------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.
// `scratch` is shared memory with room for 17 floats.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int wave = threadIdx.x / WAVE;
  const int nwaves = (blockDim.x + WAVE - 1) / WAVE;
  v = wave_sum(v);
  __syncthreads();  // scratch may still be read from an earlier call
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  if (wave == 0) {
    float t = lane < nwaves ? scratch[lane] : 0.f;
    t = wave_sum(t);
    if (lane == 0) scratch[16] = t;
  }
  __syncthreads();
  return scratch[16];
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int wave = threadIdx.x / WAVE;
  const int nwaves = (blockDim.x + WAVE - 1) / WAVE;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  if (wave == 0) {
    float t = lane < nwaves ? scratch[lane] : -INFINITY;
    t = wave_max(t);
    if (lane == 0) scratch[16] = t;
  }
  __syncthreads();
  return scratch[16];
}

// A load through the scalar unit, for a value that every lane of the wave reads from the same address and
// that nothing writes while the kernel runs (positions, block tables).  The scalar path has a cache of its
// own and does not queue behind the vector loads of the compute unit: under a stream of page loads a
// dependent vector load of four bytes was measured to take 6 microseconds.  (An address that differs
// between lanes still loads correctly, through the vector path.)
__device__ __forceinline__ int uniform_load(const int* p) {
  return *(const __attribute__((address_space(4))) int*)p;
}

// A block-wide barrier that orders LDS traffic only: every wave's LDS writes are done before any wave goes
// on.  Unlike __syncthreads() it does not wait for global loads in flight, which a kernel that keeps loads
// of later steps under way while it works on this one must not do.
__device__ __forceinline__ void block_sync_lds() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

static inline int ceil_div(long a, long b) { return (int)((a + b - 1) / b); }
