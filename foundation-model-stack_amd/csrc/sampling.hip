// Token choice from float32 logits, one block per row:
//   greedy      argmax (the lowest index among equal maxima)
//   sampling    logits / temperature; keep values >= the k-th largest (ties at
//               the threshold survive); softmax; inverse CDF in index order at
//               a uniform number drawn from a counter-based generator.
// The generator state of a row is (seed, counter) in device memory; the
// kernel advances the counter, so that a captured graph can be replayed.
#include <mutex>

#include "common.h"
#include "fmsamd.h"

#define SMP_THREADS 1024

__device__ __forceinline__ unsigned int float_key(float x) {
  // larger float <=> larger unsigned key
  const unsigned int b = __float_as_uint(x);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

__device__ __forceinline__ float uniform_from(unsigned long long seed, unsigned long long counter) {
  // splitmix64 of (seed, counter); the top 24 bits make a number in [0, 1)
  unsigned long long z = seed + (counter + 1ull) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z = z ^ (z >> 31);
  return (float)(z >> 40) * (1.0f / 16777216.0f);
}

__global__ void __launch_bounds__(SMP_THREADS)
    sample_kernel(const float* __restrict__ logits, long ld, int vocab, int do_sample, float temperature, int top_k,
                  unsigned long long* __restrict__ rng, int* __restrict__ out_tokens) {
  __shared__ float scratch[17];
  __shared__ unsigned int hist[256];
  __shared__ float seg_sum[SMP_THREADS];
  __shared__ unsigned int sh_prefix, sh_k;
  __shared__ int sh_arg;
  __shared__ float sh_target;
  const int row = blockIdx.x;
  const float* x = logits + (size_t)row * ld;
  const int tid = threadIdx.x;

  if (!do_sample) {
    float best = -INFINITY;
    int arg = 0x7fffffff;
    for (int i = tid; i < vocab; i += SMP_THREADS) {
      const float v = x[i];
      if (v > best || (v == best && i < arg)) {
        best = v;
        arg = i;
      }
    }
    const float mx = block_max(best, scratch);
    if (tid == 0) sh_arg = 0x7fffffff;
    __syncthreads();
    if (best == mx && arg != 0x7fffffff) atomicMin(&sh_arg, arg);
    __syncthreads();
    if (tid == 0) out_tokens[row] = sh_arg == 0x7fffffff ? 0 : sh_arg;
    return;
  }

  // ---- threshold: key of the k-th largest scaled logit -------------------
  unsigned int thr_key = 0u;
  if (top_k > 0 && top_k < vocab) {
    if (tid == 0) {
      sh_prefix = 0u;
      sh_k = (unsigned int)top_k;
    }
    for (int pass = 0; pass < 4; ++pass) {
      const int shift = 24 - 8 * pass;
      if (tid < 256) hist[tid] = 0u;
      __syncthreads();
      const unsigned int prefix = sh_prefix;
      const unsigned int mask = pass == 0 ? 0u : (0xFFFFFFFFu << (shift + 8));
      for (int i = tid; i < vocab; i += SMP_THREADS) {
        const unsigned int key = float_key(x[i] / temperature);
        if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
      }
      __syncthreads();
      if (tid == 0) {
        unsigned int need = sh_k, seen = 0u;
        int bin = 255;
        for (; bin > 0; --bin) {
          if (seen + hist[bin] >= need) break;
          seen += hist[bin];
        }
        sh_k = need - seen;
        sh_prefix = prefix | ((unsigned int)bin << shift);
      }
      __syncthreads();
    }
    thr_key = sh_prefix;
  }

  // ---- softmax over the kept values --------------------------------------
  float mx = -INFINITY;
  for (int i = tid; i < vocab; i += SMP_THREADS) mx = fmaxf(mx, x[i] / temperature);
  mx = block_max(mx, scratch);

  // thread `tid` owns the contiguous indices [tid*seg, (tid+1)*seg)
  const int seg = (vocab + SMP_THREADS - 1) / SMP_THREADS;
  const int begin = tid * seg;
  const int end = begin + seg < vocab ? begin + seg : vocab;
  float mine = 0.f;
  for (int i = begin; i < end; ++i) {
    const float s = x[i] / temperature;
    if (float_key(s) >= thr_key) mine += expf(s - mx);
  }
  seg_sum[tid] = mine;
  const float total = block_sum(mine, scratch);
  if (tid == 0) {
    unsigned long long counter = rng[2 * row + 1];
    sh_target = uniform_from(rng[2 * row], counter) * total;
    rng[2 * row + 1] = counter + 1ull;
    sh_arg = -1;
  }
  __syncthreads();
  // one wave finds the segment in which the running sum passes the target
  if (tid == 0) {
    const float target = sh_target;
    float run = 0.f;
    int owner = -1;
    for (int s = 0; s < SMP_THREADS; ++s) {
      if (seg_sum[s] > 0.f) {
        owner = s;  // the last segment with mass catches a target that rounding left above the total
        if (run + seg_sum[s] > target) break;
        run += seg_sum[s];
      }
    }
    sh_arg = owner;
    sh_target = target - run;
  }
  __syncthreads();
  if (tid == sh_arg) {
    const float target = sh_target;
    float run = 0.f;
    int chosen = -1;
    for (int i = begin; i < end; ++i) {
      const float s = x[i] / temperature;
      if (float_key(s) >= thr_key) {
        const float p = expf(s - mx);
        if (p > 0.f) {
          chosen = i;
          run += p;
          if (run > target) break;
        }
      }
    }
    out_tokens[row] = chosen < 0 ? 0 : chosen;
  }
  if (sh_arg < 0 && tid == 0) out_tokens[row] = 0;
}

// ---- greedy over a large vocabulary: many blocks per row, then one -------------------------
#define ARG_THREADS 256
#define ARG_CHUNK 2048  // logits per block of the first stage

__global__ void __launch_bounds__(ARG_THREADS)
    argmax_partial_kernel(const float* __restrict__ logits, long ld, int vocab, float* __restrict__ part_val,
                          int* __restrict__ part_idx, int chunks) {
  __shared__ float scratch[17];
  __shared__ int sh_arg;
  const int row = blockIdx.y, chunk = blockIdx.x;
  const float* x = logits + (size_t)row * ld;
  const int begin = chunk * ARG_CHUNK;
  const int end = begin + ARG_CHUNK < vocab ? begin + ARG_CHUNK : vocab;
  float best = -INFINITY;
  int arg = 0x7fffffff;
  for (int i = begin + threadIdx.x; i < end; i += ARG_THREADS) {
    const float v = x[i];
    if (v > best || (v == best && i < arg)) best = v, arg = i;
  }
  const float mx = block_max(best, scratch);
  if (threadIdx.x == 0) sh_arg = 0x7fffffff;
  __syncthreads();
  if (best == mx && arg != 0x7fffffff) atomicMin(&sh_arg, arg);
  __syncthreads();
  if (threadIdx.x == 0) {
    part_val[(size_t)row * chunks + chunk] = mx;
    part_idx[(size_t)row * chunks + chunk] = sh_arg;
  }
}

__global__ void __launch_bounds__(ARG_THREADS)
    argmax_final_kernel(const float* __restrict__ part_val, const int* __restrict__ part_idx, int chunks,
                        int* __restrict__ out_tokens) {
  __shared__ float scratch[17];
  __shared__ int sh_arg;
  const int row = blockIdx.x;
  float best = -INFINITY;
  int arg = 0x7fffffff;
  for (int c = threadIdx.x; c < chunks; c += ARG_THREADS) {
    const float v = part_val[(size_t)row * chunks + c];
    const int i = part_idx[(size_t)row * chunks + c];
    if (v > best || (v == best && i < arg)) best = v, arg = i;
  }
  const float mx = block_max(best, scratch);
  if (threadIdx.x == 0) sh_arg = 0x7fffffff;
  __syncthreads();
  if (best == mx && arg != 0x7fffffff) atomicMin(&sh_arg, arg);
  __syncthreads();
  if (threadIdx.x == 0) out_tokens[row] = sh_arg == 0x7fffffff ? 0 : sh_arg;
}

extern "C" long fmsamd_argmax_workspace(int rows, int vocab) {
  return (long)rows * ceil_div(vocab, ARG_CHUNK) * 8;
}

// greedy choice with a workspace of fmsamd_argmax_workspace(rows, vocab) bytes
extern "C" int fmsamd_argmax(const float* logits, long ld, int rows, int vocab, void* workspace, long workspace_bytes,
                             int* out_tokens, hipStream_t stream) {
  if (rows == 0) return 0;
  FMS_REQUIRE(rows > 0 && vocab > 0 && ld >= vocab, "argmax: bad sizes rows=%d vocab=%d ld=%ld", rows, vocab, ld);
  FMS_REQUIRE(rows <= 65535, "argmax: %d rows exceed one launch", rows);
  const int chunks = ceil_div(vocab, ARG_CHUNK);
  FMS_REQUIRE(workspace != nullptr && workspace_bytes >= fmsamd_argmax_workspace(rows, vocab),
              "argmax: workspace of %ld bytes, %ld needed", workspace_bytes, fmsamd_argmax_workspace(rows, vocab));
  float* part_val = (float*)workspace;
  int* part_idx = (int*)(part_val + (size_t)rows * chunks);
  argmax_partial_kernel<<<dim3(chunks, rows), ARG_THREADS, 0, stream>>>(logits, ld, vocab, part_val, part_idx, chunks);
  FMS_LAUNCH_CHECK("argmax_partial");
  argmax_final_kernel<<<rows, ARG_THREADS, 0, stream>>>(part_val, part_idx, chunks, out_tokens);
  FMS_LAUNCH_CHECK("argmax_final");
  return 0;
}

// ---- the same greedy choice for callers that cannot allocate ---------------------------------
// The partial maxima of the first stage live in an array of the library's own instead of a workspace of the
// caller's.  In host code the array's name is only a handle: its address on the current GPU is asked for
// once per device (every GPU holds a copy of its own) and that address is what the kernels get.
static __device__ __align__(256) unsigned char scratch[FMSAMD_ARGMAX_STATIC_BYTES];

#define ARG_MAX_DEVICES 64
static void* scratch_of_device[ARG_MAX_DEVICES];
static std::mutex scratch_lock;

static int scratch_address(void** out) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  FMS_REQUIRE(e == hipSuccess, "argmax_static: hipGetDevice failed: %s", hipGetErrorString(e));
  FMS_REQUIRE(device >= 0 && device < ARG_MAX_DEVICES, "argmax_static: device %d is beyond the %d this library keeps track of",
              device, ARG_MAX_DEVICES);
  std::lock_guard<std::mutex> guard(scratch_lock);
  if (scratch_of_device[device] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    FMS_REQUIRE(e == hipSuccess && ptr != nullptr, "argmax_static: the scratch array has no address on device %d: %s", device,
                hipGetErrorString(e));
    scratch_of_device[device] = ptr;
  }
  *out = scratch_of_device[device];
  return 0;
}

extern "C" int fmsamd_argmax_static(const float* logits, long ld, int rows, int vocab, int* out_tokens,
                                    hipStream_t stream) {
  if (rows == 0) return 0;
  FMS_REQUIRE(rows > 0 && vocab > 0 && ld >= vocab, "argmax_static: bad sizes rows=%d vocab=%d ld=%ld", rows, vocab, ld);
  FMS_REQUIRE(rows <= 65535, "argmax_static: %d rows exceed one launch", rows);
  FMS_REQUIRE(logits != nullptr && out_tokens != nullptr, "argmax_static: null logits or output");
  const int chunks = ceil_div(vocab, ARG_CHUNK);
  const long need = fmsamd_argmax_workspace(rows, vocab);
  FMS_REQUIRE(need <= (long)FMSAMD_ARGMAX_STATIC_BYTES,
              "argmax_static: %d rows of %d logits need %ld bytes of partial results, the library's array holds %ld "
              "(rows x ceil(vocab / %d) <= %ld): use fmsamd_argmax with a workspace",
              rows, vocab, need, (long)FMSAMD_ARGMAX_STATIC_BYTES, ARG_CHUNK, (long)FMSAMD_ARGMAX_STATIC_BYTES / 8);
  void* base = nullptr;
  if (scratch_address(&base) != 0) return -1;
  // every entry that the second stage reads is written by the first: nothing has to start at zero
  float* part_val = (float*)base;
  int* part_idx = (int*)(part_val + (size_t)rows * chunks);
  argmax_partial_kernel<<<dim3(chunks, rows), ARG_THREADS, 0, stream>>>(logits, ld, vocab, part_val, part_idx, chunks);
  FMS_LAUNCH_CHECK("argmax_static (first stage)");
  argmax_final_kernel<<<rows, ARG_THREADS, 0, stream>>>(part_val, part_idx, chunks, out_tokens);
  FMS_LAUNCH_CHECK("argmax_static (second stage)");
  return 0;
}

extern "C" int fmsamd_sample(const float* logits, long ld, int rows, int vocab, int do_sample, float temperature,
                             int top_k, void* rng_state, int* out_tokens, hipStream_t stream) {
  if (rows == 0) return 0;
  FMS_REQUIRE(rows > 0 && vocab > 0 && ld >= vocab, "sample: bad sizes rows=%d vocab=%d ld=%ld", rows, vocab, ld);
  if (do_sample) {
    FMS_REQUIRE(temperature > 0.f, "sample: temperature %g must be positive", (double)temperature);
    FMS_REQUIRE(top_k >= 0, "sample: top_k %d is negative", top_k);
    FMS_REQUIRE(rng_state != nullptr, "sample: sampling needs generator state");
  }
  sample_kernel<<<rows, SMP_THREADS, 0, stream>>>(logits, ld, vocab, do_sample, temperature, top_k,
                                                  (unsigned long long*)rng_state, out_tokens);
  FMS_LAUNCH_CHECK("sample");
  return 0;
}
