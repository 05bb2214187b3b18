// Two kernels that measure the GPU they run on, for the benchmark's "of the measured peak" fractions:
// a pure read of a buffer (what the memory system delivers to a kernel that does nothing else) and a loop of
// matrix instructions on registers (what the matrix cores deliver at the clock they hold under load).
#include "common.h"
#include "fmsamd.h"

#define PROBE_THREADS 512
#define PROBE_UNROLL 8

// Every thread reads 16 bytes at a time, PROBE_UNROLL loads under way, non-temporally (each byte is read once).
// contiguous: a block reads one stretch of the buffer from end to end (a wave's load covers 1 KB of it); otherwise
// the whole grid sweeps the buffer together.
__global__ void __launch_bounds__(PROBE_THREADS)
    probe_read_kernel(const f32x4* __restrict__ p, long n, int contiguous, float* __restrict__ out) {
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  long i, end, stride;
  if (contiguous) {
    const long per_block = (n + gridDim.x - 1) / gridDim.x;
    i = (long)blockIdx.x * per_block + threadIdx.x;
    end = (long)(blockIdx.x + 1) * per_block < n ? (long)(blockIdx.x + 1) * per_block : n;
    stride = blockDim.x;
  } else {
    i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    end = n;
    stride = (long)gridDim.x * blockDim.x;
  }
  for (; i < end; i += PROBE_UNROLL * stride) {
    f32x4 v[PROBE_UNROLL];
#pragma unroll
    for (int u = 0; u < PROBE_UNROLL; ++u) {
      const long at = i + u * stride;
      v[u] = __builtin_nontemporal_load(p + (at < end ? at : i));
    }
#pragma unroll
    for (int u = 0; u < PROBE_UNROLL; ++u) acc += v[u];
  }
  // a result that depends on every load, stored by (almost) no thread
  if (acc[0] + acc[1] + acc[2] + acc[3] == 12345.678f) out[0] = 1.f;
}

// bytes of `buffer` are read once by `blocks` blocks; `out` is one float that may be written.
extern "C" int fmsamd_probe_read(const void* buffer, long bytes, int blocks, int contiguous, float* out, hipStream_t stream) {
  FMS_REQUIRE(buffer != nullptr && out != nullptr && bytes >= 16 && blocks > 0 && blocks <= 65535,
              "probe_read: a buffer of at least 16 bytes and 1 to 65535 blocks are needed");
  FMS_REQUIRE(((uintptr_t)buffer & 15) == 0, "probe_read: the buffer must start 16-byte aligned");
  probe_read_kernel<<<blocks, PROBE_THREADS, 0, stream>>>((const f32x4*)buffer, bytes / 16, contiguous, out);
  FMS_LAUNCH_CHECK("probe_read");
  return 0;
}

// Independent accumulators, so that the matrix unit never waits for a result.  LARGE: 32x32x16 products (four
// accumulators of 16 registers), otherwise 16x16x32 (eight of 4); either is 2 * 16384 / 2 flops a lane group.
template <bool LARGE>
__global__ void __launch_bounds__(256) probe_mfma_kernel(int iterations, float* __restrict__ out) {
  const int lane = threadIdx.x & (WAVE - 1);
  bf16x8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (bf16)(0.001f * (float)(lane + i));
    b[i] = (bf16)(0.002f * (float)(lane ^ i));
  }
  float sum = 0.f;
  if (LARGE) {
    f32x16 acc[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[k][e] = 0.f;
    for (int it = 0; it < iterations; ++it) {
#pragma unroll
      for (int k = 0; k < 4; ++k) acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[k], 0, 0, 0);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
      for (int e = 0; e < 16; ++e) sum += acc[k][e];
  } else {
    f32x4 acc[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) acc[k] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iterations; ++it) {
#pragma unroll
      for (int k = 0; k < 8; ++k) acc[k] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[k], 0, 0, 0);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) sum += acc[k][0] + acc[k][1] + acc[k][2] + acc[k][3];
  }
  if (sum == 12345.678f) out[0] = sum;
}

// blocks x 4 waves x iterations x (8 products of 16x16x32 or 4 of 32x32x16); the caller divides the flops
// (returned through *flops) by the time.
extern "C" int fmsamd_probe_mfma(int blocks, int iterations, int large, float* out, double* flops, hipStream_t stream) {
  FMS_REQUIRE(out != nullptr && blocks > 0 && blocks <= 65535 && iterations > 0, "probe_mfma: bad sizes");
  if (large)
    probe_mfma_kernel<true><<<blocks, 256, 0, stream>>>(iterations, out);
  else
    probe_mfma_kernel<false><<<blocks, 256, 0, stream>>>(iterations, out);
  FMS_LAUNCH_CHECK("probe_mfma");
  if (flops != nullptr) *flops = (double)blocks * 4.0 * (double)iterations * (large ? 4.0 * 32768.0 : 8.0 * 16384.0);
  return 0;
}
