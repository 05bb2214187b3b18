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
#define SMP_WAVES (SMP_THREADS / WAVE)
#define SMP_SHORT_K 512       // the largest top_k that is served from a short list of candidates
#define SMP_CANDIDATES 1024   // room in that list: one candidate per thread

__device__ __forceinline__ unsigned int float_key(float x) {
  // larger float <=> larger unsigned key
  const unsigned int b = __float_as_uint(x);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

__device__ __forceinline__ float key_float(unsigned int key) {
  // the float that float_key() made the key from
  return __uint_as_float((key & 0x80000000u) ? (key & 0x7FFFFFFFu) : ~key);
}

__device__ __forceinline__ float uniform_from(unsigned long long seed, unsigned long long counter) {
  // splitmix64 of (seed, counter); the top 24 bits make a number in [0, 1)
  unsigned long long z = seed + (counter + 1ull) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z = z ^ (z >> 31);
  return (float)(z >> 40) * (1.0f / 16777216.0f);
}

// The k-th largest of the keys that the block's threads hold together, by a radix selection of four passes
// over eight bits each.  `for_each_key(count)` calls count(key) for every key of this thread; it is called
// once per pass.  k is at least 1 and at most the number of keys.  Every thread of the block calls this and
// gets the result.  hist: 256 counters, wave_total: 4, state: 2, all in shared memory.
template <typename ForEachKey>
__device__ __forceinline__ unsigned int kth_largest_key(unsigned int k, unsigned int* hist, unsigned int* wave_total,
                                                        unsigned int* state, ForEachKey for_each_key) {
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  unsigned int prefix = 0u, need = k;
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    const unsigned int mask = pass == 0 ? 0u : (0xFFFFFFFFu << (shift + 8));
    __syncthreads();  // the counters and the state of the pass before have been read
    if (tid < 256) hist[tid] = 0u;
    __syncthreads();
    for_each_key([&](unsigned int key) {
      if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
    });
    __syncthreads();
    // thread b < 256 learns how many keys lie in the bins b and above: a suffix scan inside each of the four
    // waves that hold the bins, then the totals of the waves above
    unsigned int mine = 0u, suffix = 0u;
    if (tid < 256) {
      mine = hist[tid];
      suffix = mine;
#pragma unroll
      for (int off = 1; off < WAVE; off <<= 1) {
        const unsigned int other = __shfl_down(suffix, off, WAVE);
        if (lane + off < WAVE) suffix += other;
      }
      if (lane == 0) wave_total[tid / WAVE] = suffix;
    }
    __syncthreads();
    if (tid < 256) {
      for (int w = tid / WAVE + 1; w < 4; ++w) suffix += wave_total[w];
      const unsigned int higher = suffix - mine;  // keys in the bins above this one
      if (higher < need && need <= suffix) {       // the bin of the key that is looked for: exactly one thread
        state[0] = prefix | ((unsigned int)tid << shift);
        state[1] = need - higher;
      } else if (tid == 0 && suffix < need) {      // fewer keys than k: the lowest bin, so that everything is kept
        state[0] = prefix;
        state[1] = 1u;
      }
    }
    __syncthreads();
    prefix = state[0];
    need = state[1];
  }
  return prefix;
}

// f(value, index) for every index in [begin, end), shared out among `count` threads of which this is number `me`.
// With `quads` (the row starts at a multiple of 16 bytes, and begin is a multiple of 4) four values come with
// one load: a pass over a long row is bound by the number of loads that a compute unit has under way.
template <typename F>
__device__ __forceinline__ void for_each_value(const float* __restrict__ x, int begin, int end, int me, int count,
                                               bool quads, F f) {
  if (quads) {
    const int n = (end - begin) / 4;
    const float4* x4 = (const float4*)(x + begin);
#pragma unroll 4
    for (int q = me; q < n; q += count) {
      const float4 v = x4[q];
      const int i = begin + 4 * q;
      f(v.x, i);
      f(v.y, i + 1);
      f(v.z, i + 2);
      f(v.w, i + 3);
    }
    for (int i = begin + 4 * n + me; i < end; i += count) f(x[i], i);
  } else {
#pragma unroll 4
    for (int i = begin + me; i < end; i += count) f(x[i], i);
  }
}

// One block per row.  The row is read in passes whose loads are coalesced.
//   Always: the largest value.
//   top_k up to 512: each thread's largest value as well.  At least k values are as large as the k-th largest
//   of these 1024, so the k-th largest of the row is no smaller than that bound, and the values at or above
//   the bound are few (about k (1 + k / 2048)) unless many are equal.  A second pass collects them, with
//   their indices, and the rest happens on that list: the threshold, the order by index, the running sum of
//   the exponentials, the place where it passes the target.
//   No top_k, a larger one, or a list that overflows: the threshold by a selection over the whole row; then
//   the sum of the kept exponentials by sixteen stretches of consecutive indices, one per wave; the stretch in
//   which the running sum passes the target is cut into sixteen again, down to 64 indices, which a wave scans.
// Dividing by the temperature keeps the order of the values, so the largest value and the bound are found on
// the logits as they are, and only values that pass a bound lowered by a little are divided and compared exactly.
__global__ void __launch_bounds__(SMP_THREADS)
    sample_kernel(const float* __restrict__ logits, long ld, int vocab, int do_sample, float temperature, int top_k,
                  unsigned long long* __restrict__ rng, int* __restrict__ out_tokens) {
  __shared__ float scratch[17];
  __shared__ unsigned int hist[256];
  __shared__ unsigned int wave_total[4];
  __shared__ unsigned int state[2];
  __shared__ unsigned int cand_key[SMP_CANDIDATES];
  __shared__ int cand_index[SMP_CANDIDATES];
  __shared__ int sorted_index[SMP_CANDIDATES];
  __shared__ float sorted_p[SMP_CANDIDATES];
  __shared__ unsigned int n_candidates;
  __shared__ float stretch_sum[SMP_WAVES];
  __shared__ int sh_arg, sh_last;
  __shared__ float sh_target;
  const int row = blockIdx.x;
  const float* x = logits + (size_t)row * ld;
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;

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

  // ---- the largest logit, and each thread's own largest ---------------------
  const bool quads = ((size_t)x & 15) == 0;
  float best = -INFINITY;
  for_each_value(x, 0, vocab, tid, SMP_THREADS, quads, [&](float v, int) { best = fmaxf(best, v); });
  const float mx = block_max(best, scratch) / temperature;  // the largest scaled logit

  const bool with_top_k = top_k > 0 && top_k < vocab;
  if (with_top_k && top_k <= SMP_SHORT_K) {
    const unsigned int my_key = float_key(best);
    const float bound = key_float(kth_largest_key((unsigned int)top_k, hist, wave_total, state,
                                                  [&](auto count) { count(my_key); }));
    const unsigned int bound_key = float_key(bound / temperature);
    // two logits whose quotients round to the same number differ by a few units in the last place at most
    const float loose = bound - fmaxf(fabsf(bound) * 0x1p-20f, 1e-30f);
    if (tid == 0) n_candidates = 0u;
    __syncthreads();
    for_each_value(x, 0, vocab, tid, SMP_THREADS, quads, [&](float v, int i) {
      if (v >= loose) {
        const unsigned int key = float_key(v / temperature);
        if (key >= bound_key) {
          const unsigned int at = atomicAdd(&n_candidates, 1u);
          if (at < SMP_CANDIDATES) {
            cand_key[at] = key;
            cand_index[at] = i;
          }
        }
      }
    });
    __syncthreads();
    const int n = (int)n_candidates;
    if (n <= SMP_CANDIDATES) {
      const unsigned int thr_key = kth_largest_key((unsigned int)top_k, hist, wave_total, state, [&](auto count) {
        if (tid < n) count(cand_key[tid]);
      });
      // The list is in the order in which the threads got to it.  Candidate `tid` goes to the place that its
      // index has among the indices, so that the sums below are taken in the order of the indices whatever
      // the order of arrival was.
      if (tid < n) {
        const int mine = cand_index[tid];
        int place = 0;
        for (int j = 0; j < n; ++j) place += cand_index[j] < mine ? 1 : 0;
        const unsigned int key = cand_key[tid];
        sorted_index[place] = mine;
        sorted_p[place] = key >= thr_key ? expf(key_float(key) - mx) : 0.f;
      }
      if (tid == 0) {
        sh_arg = 0x7fffffff;
        sh_last = -1;
      }
      __syncthreads();
      const float p = tid < n ? sorted_p[tid] : 0.f;
      float upto = p;  // the sum of p over this place and the places before it
#pragma unroll
      for (int off = 1; off < WAVE; off <<= 1) {
        const float other = __shfl_up(upto, off, WAVE);
        if (lane >= off) upto += other;
      }
      if (lane == WAVE - 1) stretch_sum[wave] = upto;
      __syncthreads();
      float before = 0.f, total = 0.f;
      for (int w = 0; w < SMP_WAVES; ++w) {
        if (w == wave) before = total;
        total += stretch_sum[w];
      }
      upto += before;
      if (tid == 0) {
        const unsigned long long counter = rng[2 * row + 1];
        sh_target = uniform_from(rng[2 * row], counter) * total;
        rng[2 * row + 1] = counter + 1ull;
      }
      __syncthreads();
      if (p > 0.f) {
        if (upto > sh_target) atomicMin(&sh_arg, tid);
        atomicMax(&sh_last, tid);  // the last place with mass catches a target that rounding left above the total
      }
      __syncthreads();
      if (tid == 0) {
        const int place = sh_arg != 0x7fffffff ? sh_arg : sh_last;
        out_tokens[row] = place < 0 ? 0 : sorted_index[place];
      }
      return;
    }
  }

  // ---- threshold: key of the k-th largest scaled logit, over the whole row -------------------
  unsigned int thr_key = 0u;
  if (with_top_k) {
    thr_key = kth_largest_key((unsigned int)top_k, hist, wave_total, state, [&](auto count) {
      for_each_value(x, 0, vocab, tid, SMP_THREADS, quads, [&](float v, int) { count(float_key(v / temperature)); });
    });
  }

  // ---- softmax over the kept values and the inverse of its running sum ---------------------
  int lo = 0, hi = vocab;
  float target = 0.f;
  bool whole_row = true;
  while (whole_row || hi - lo > WAVE) {
    // wave w sums the indices [lo + w * len, lo + (w + 1) * len)
    int len = (hi - lo + SMP_WAVES - 1) / SMP_WAVES;
    len = (len + WAVE - 1) / WAVE * WAVE;
    const int begin = lo + wave * len;
    const int end = begin + len < hi ? begin + len : hi;
    float mine = 0.f;
    if (begin < end) {  // lo is a multiple of 64 at every level, and so is begin
      for_each_value(x, begin, end, lane, WAVE, quads, [&](float v, int) {
        const float s = v / temperature;
        if (float_key(s) >= thr_key) mine += expf(s - mx);
      });
    }
    mine = wave_sum(mine);
    __syncthreads();  // the sums of the level before have been read
    if (lane == 0) stretch_sum[wave] = mine;
    __syncthreads();
    if (whole_row) {
      float total = 0.f;
      for (int w = 0; w < SMP_WAVES; ++w) total += stretch_sum[w];
      if (tid == 0) {
        const unsigned long long counter = rng[2 * row + 1];
        sh_target = uniform_from(rng[2 * row], counter) * total;
        rng[2 * row + 1] = counter + 1ull;
      }
      __syncthreads();
      target = sh_target;
      whole_row = false;
    }
    // every thread walks the sixteen sums alike
    float run = 0.f;
    int owner = -1;
    for (int w = 0; w < SMP_WAVES; ++w) {
      const float sum = stretch_sum[w];
      if (sum > 0.f) {
        owner = w;  // the last stretch with mass catches a target that rounding left above the total
        if (run + sum > target) break;
        run += sum;
      }
    }
    if (owner < 0) {  // no mass anywhere (logits that are not numbers)
      if (tid == 0) out_tokens[row] = 0;
      return;
    }
    target -= run;
    lo += owner * len;
    hi = lo + len < hi ? lo + len : hi;
  }
  if (wave == 0) {
    const int i = lo + lane;
    float p = 0.f;
    if (i < hi) {
      const float s = x[i] / temperature;
      if (float_key(s) >= thr_key) p = expf(s - mx);
    }
    float upto = p;  // the sum of p over this lane and the lanes below
#pragma unroll
    for (int off = 1; off < WAVE; off <<= 1) {
      const float other = __shfl_up(upto, off, WAVE);
      if (lane >= off) upto += other;
    }
    const unsigned long long passed = __ballot(p > 0.f && upto > target);
    const unsigned long long mass = __ballot(p > 0.f);
    int chosen = 0;
    if (passed != 0ull) {
      chosen = lo + __ffsll(passed) - 1;
    } else if (mass != 0ull) {
      chosen = lo + 63 - __clzll(mass);  // the last index with mass catches a target that rounding left above the sum
    }
    if (lane == 0) out_tokens[row] = chosen;
  }
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
