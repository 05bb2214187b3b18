// Causal attention over the paged cache, with grouped kv heads and an
// optional sliding window.
//
//   * attn_generic_kernel: any element type (float32 here), any even head
//     size up to 256, plain FMA arithmetic.  It is the true 32-bit path.
//   * attn_prefill_lds_kernel (pages through LDS, shared by the heads of a kv
//     group; head sizes up to 128), attn_prefill_bf16_kernel (straight from
//     global memory; head sizes above 128) and
//     attn_decode_bf16_kernel (+ merge): bfloat16 storage, float32 softmax and
//     accumulation, MFMA 16x16x32.
//
// The MFMA kernels compute S^T = K Q^T (rows: keys, columns: queries) so that
// the probabilities come out of the accumulator already in the operand layout
// of the second product O^T = V^T P^T; no round trip through LDS is needed.
// Cache layout: see rope.hip.
#include "common.h"
#include "fmsamd.h"

// ==========================================================================
// generic kernel: one block per (head, token)
// ==========================================================================
#define GEN_THREADS 256

// TERMS: the scores carry further terms (fms/modules/positions.py:9-36, the reference's adjusted_mask): a soft cap
// cap * tanh(score / cap), and a bias slope[head] * (key position - query position), which is zero or negative.
// Without TERMS neither is compiled in.
template <typename T, bool TERMS>
__global__ void __launch_bounds__(GEN_THREADS)
    attn_generic_kernel(const T* __restrict__ q, long q_stride, T* __restrict__ out, long out_stride,
                        const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                        const int* __restrict__ block_table, int table_stride, const T* __restrict__ k_cache,
                        const T* __restrict__ v_cache, int nheads, int kvheads, int head_dim, float scale, int window,
                        const float* __restrict__ slopes, float soft_cap) {
  __shared__ float qs[256];
  __shared__ float ps[GEN_THREADS];
  __shared__ float scratch[17];
  const int h = blockIdx.x;
  const int t = blockIdx.y;
  const int seq = seq_of_token[t];
  T* o = out + (size_t)t * out_stride + (size_t)h * head_dim;
  if (seq < 0) {
    for (int d = threadIdx.x; d < head_dim; d += blockDim.x) o[d] = from_f32<T>(0.f);
    return;
  }
  const int pos = positions[t];
  const int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;
  const int kh = h / (nheads / kvheads);
  const int* bt = block_table + (size_t)seq * table_stride;
  const size_t page_elems = (size_t)kvheads * PAGE_TOKENS * head_dim;

  const T* qrow = q + (size_t)t * q_stride + (size_t)h * head_dim;
  for (int d = threadIdx.x; d < head_dim; d += blockDim.x) qs[d] = to_f32(qrow[d]);
  __syncthreads();

  float m_run = -1e30f, l_run = 0.f, acc = 0.f;  // acc: this thread's output element d = threadIdx.x
  for (int base = lo; base <= pos; base += GEN_THREADS) {
    const int j = base + threadIdx.x;
    float s = -INFINITY;
    if (j <= pos) {
      const T* krow = k_cache + readable_page(bt[j / PAGE_TOKENS]) * page_elems +
                      ((size_t)kh * PAGE_TOKENS + j % PAGE_TOKENS) * head_dim;
      float dot = 0.f;
      for (int d = 0; d < head_dim; ++d) dot = fmaf(qs[d], to_f32(krow[d]), dot);
      s = dot * scale;
      if (TERMS) {
        if (soft_cap > 0.f) s = soft_cap * tanhf(s / soft_cap);
        if (slopes != nullptr) s = fmaf(slopes[h], (float)(j - pos), s);
      }
    }
    const float m_new = fmaxf(m_run, block_max(s, scratch));
    const float p = j <= pos ? expf(s - m_new) : 0.f;
    const float alpha = expf(m_run - m_new);
    ps[threadIdx.x] = p;
    const float psum = block_sum(p, scratch);  // has the barriers that publish ps
    l_run = l_run * alpha + psum;
    m_run = m_new;
    if ((int)threadIdx.x < head_dim) {
      const int d = threadIdx.x;
      float a = acc * alpha;
      const int n = pos - base + 1 < GEN_THREADS ? pos - base + 1 : GEN_THREADS;
      for (int i = 0; i < n; ++i) {
        const int jj = base + i;
        const T* vrow = v_cache + readable_page(bt[jj / PAGE_TOKENS]) * page_elems +
                        ((size_t)kh * head_dim + d) * PAGE_TOKENS + jj % PAGE_TOKENS;
        a = fmaf(ps[i], to_f32(*vrow), a);
      }
      acc = a;
    }
    __syncthreads();  // ps is overwritten by the next chunk
  }
  if ((int)threadIdx.x < head_dim) o[threadIdx.x] = from_f32<T>(l_run > 0.f ? acc / l_run : 0.f);
}

#define LOG2E 1.4426950408889634f
// the maximum that a partial result of the decode kernel carries when it holds no key at all
#define DECODE_EMPTY -1e30f

// Maxima as single instructions.  fmaxf() first passes each operand through a max with itself (it must quiet a
// signalling NaN), which tripled the instructions of the score maxima; the scores here come out of the matrix unit
// and are never signalling NaNs.
__device__ __forceinline__ float max2f(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
// The maximum over the four lanes l, l ^ 16, l ^ 32, l ^ 48 (a score column's four lane groups), in all four:
// two swaps of lane halves and rows between a register and its copy, in the vector unit (a shuffle through
// LDS takes a round trip to LDS for each of the two steps, in the middle of the softmax's chain).
__device__ __forceinline__ float max_over_lane_groups(float x) {
  const unsigned u = __float_as_uint(x);
  const auto halves = __builtin_amdgcn_permlane32_swap(u, u, false, false);  // [lo, lo] and [hi, hi]
  float m;
  asm("v_max_f32 %0, %1, %2" : "=v"(m) : "v"(__uint_as_float(halves[0])), "v"(__uint_as_float(halves[1])));
  const unsigned um = __float_as_uint(m);
  const auto rows = __builtin_amdgcn_permlane16_swap(um, um, false, false);  // rows [0, 0, 2, 2] and [1, 1, 3, 3]
  asm("v_max_f32 %0, %1, %2" : "=v"(m) : "v"(__uint_as_float(rows[0])), "v"(__uint_as_float(rows[1])));
  return m;
}
__device__ __forceinline__ float max3f(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// ==========================================================================
// MFMA core.  One wave owns 16*QT query columns and walks over pages of keys.
// ==========================================================================
template <int MAXDT, int QT>
struct WaveState {
  f32x4 acc[QT][MAXDT];  // O^T tiles: rows d = dt*16 + (lane/16)*4 + i, column = lane%16
  float m[QT];           // running maximum of this lane's column (equal in the 4 lanes of a column)
  float l[QT];           // this lane's share of the running sum of its column
};

__device__ __forceinline__ bf16x8 load_bf16x8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }

// One step of the online softmax over 32 keys for the 16*QT query columns of a wave.
// qreg[qt][c]: this lane's 8 query elements d = c*32 + (lane/16)*8 .. +8 of its column (zero when absent).
// qpos/qlo: visible keys of this lane's column are qlo <= key <= qpos (qpos < 0: no key).
// kbase: key row 0 of the 32 keys, rows k_stride elements apart; vbase: column 0 of the 32 keys in the
// transposed values, rows (head_dim of them) v_stride elements apart.  Global memory or LDS.
// scale2 = softmax scale * log2(e): scores and running maxima live in the base-2 domain (exp2 is the
// hardware's native exponential).  `full`: every one of the 32 keys is visible to every column of the
// wave, so no mask is applied (true for all but the steps at the causal edge or a window's edge).
// The three parts of a step: scores S^T = K Q^T of 32 keys (matrix unit), the online softmax of those scores
// (vector unit), and O^T += V^T P^T (matrix unit).
template <int MAXDT, int QT>
__device__ __forceinline__ void step_scores(f32x4 (&sa)[QT], f32x4 (&sb)[QT], const bf16x8 (&qreg)[QT][(MAXDT + 1) / 2],
                                            const bf16* kbase, int k_stride, int head_dim) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int r = lane & 15;
  const int g = lane >> 4;
  const int nchunk = (head_dim + 31) / 32;
  // Which key sits in which row of the two score tiles is free, as long as the second product pairs every
  // probability with its value.  Rows are dealt so that lane group g ends up with the probabilities of the
  // 8 consecutive keys 8 g .. 8 g + 7 (tile a: 8 g + i, tile b: 8 g + 4 + i): their values are then one
  // 16-byte read per row of the transposed values.
  const int key_a = (r >> 2) * 8 + (r & 3);
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    sa[qt] = f32x4{0.f, 0.f, 0.f, 0.f};
    sb[qt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
#pragma unroll
  for (int c = 0; c < (MAXDT + 1) / 2; ++c) {
    if (c < nchunk) {
      const int d = c * 32 + g * 8;
      bf16x8 ka = {0, 0, 0, 0, 0, 0, 0, 0}, kb = {0, 0, 0, 0, 0, 0, 0, 0};
      if (d < head_dim) {
        ka = load_bf16x8(kbase + (size_t)key_a * k_stride + d);
        kb = load_bf16x8(kbase + (size_t)(key_a + 4) * k_stride + d);
      }
#pragma unroll
      for (int qt = 0; qt < QT; ++qt) {
        sa[qt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qreg[qt][c], sa[qt], 0, 0, 0);
        sb[qt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb, qreg[qt][c], sb[qt], 0, 0, 0);
      }
    }
  }
}

template <int MAXDT, int QT>
__device__ __forceinline__ void step_softmax(WaveState<MAXDT, QT>& st, f32x4 (&sa)[QT], f32x4 (&sb)[QT],
                                             bf16x8 (&pmat)[QT], const int (&qpos)[QT], const int (&qlo)[QT], int key0,
                                             int head_dim, float scale2, bool full) {
  const int g = (threadIdx.x & (WAVE - 1)) >> 4;
  const int ndt = head_dim / 16;
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    // maxima of the raw scores, scaled once (the scale is positive); every probability is then one fused
    // multiply-add and one exponential: exp2(s * scale2 - m)
    if (!full) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int ja = key0 + g * 8 + i;  // the accumulator's rows 4 g + i hold these keys
        const int jb = ja + 4;
        sa[qt][i] = (ja <= qpos[qt] && ja >= qlo[qt]) ? sa[qt][i] : -INFINITY;
        sb[qt][i] = (jb <= qpos[qt] && jb >= qlo[qt]) ? sb[qt][i] : -INFINITY;
      }
    }
    float mx = max3f(max3f(sa[qt][0], sa[qt][1], sa[qt][2]), max3f(sa[qt][3], sb[qt][0], sb[qt][1]), max2f(sb[qt][2], sb[qt][3]));
    mx = max_over_lane_groups(mx);
    const float m_new = max2f(st.m[qt], mx * scale2);
    const float alpha = __builtin_amdgcn_exp2f(st.m[qt] - m_new);
    st.m[qt] = m_new;
    float psum = 0.f;
    float pa[4], pb[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      pa[i] = __builtin_amdgcn_exp2f(fmaf(sa[qt][i], scale2, -m_new));
      pb[i] = __builtin_amdgcn_exp2f(fmaf(sb[qt][i], scale2, -m_new));
      psum += pa[i] + pb[i];
    }
    st.l[qt] = st.l[qt] * alpha + psum;
    pmat[qt] = bf16x8{(bf16)pa[0], (bf16)pa[1], (bf16)pa[2], (bf16)pa[3],
                      (bf16)pb[0], (bf16)pb[1], (bf16)pb[2], (bf16)pb[3]};
    // the running maximum seldom moves after the first keys: rescale only when some column's did
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int dt = 0; dt < MAXDT; ++dt)
        if (dt < ndt) st.acc[qt][dt] *= alpha;
    }
  }
}

template <int MAXDT, int QT>
__device__ __forceinline__ void step_accumulate(WaveState<MAXDT, QT>& st, const bf16x8 (&pmat)[QT], const bf16* vbase,
                                                int v_stride, int head_dim) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int r = lane & 15;
  const int g = lane >> 4;
  const int ndt = head_dim / 16;
#pragma unroll
  for (int dt = 0; dt < MAXDT; ++dt) {
    if (dt < ndt) {
      const bf16x8 v = load_bf16x8(vbase + (size_t)(dt * 16 + r) * v_stride + g * 8);
#pragma unroll
      for (int qt = 0; qt < QT; ++qt)
        st.acc[qt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v, pmat[qt], st.acc[qt][dt], 0, 0, 0);
    }
  }
}

template <int MAXDT, int QT>
__device__ __forceinline__ void half_step(WaveState<MAXDT, QT>& st, const bf16x8 (&qreg)[QT][(MAXDT + 1) / 2],
                                          const int (&qpos)[QT], const int (&qlo)[QT], int key0, const bf16* kbase,
                                          int k_stride, const bf16* vbase, int v_stride, int head_dim, float scale2,
                                          bool full) {
  f32x4 sa[QT], sb[QT];
  bf16x8 pmat[QT];
  step_scores<MAXDT, QT>(sa, sb, qreg, kbase, k_stride, head_dim);
  step_softmax<MAXDT, QT>(st, sa, sb, pmat, qpos, qlo, key0, head_dim, scale2, full);
  step_accumulate<MAXDT, QT>(st, pmat, vbase, v_stride, head_dim);
}

// The pages page_first, page_first + page_step, ... of a sequence, straight from global memory.
template <int MAXDT, int QT>
__device__ __forceinline__ void attn_wave_pages(WaveState<MAXDT, QT>& st, const bf16x8 (&qreg)[QT][(MAXDT + 1) / 2],
                                                const int (&qpos)[QT], const int (&qlo)[QT], int key_lo, int key_hi,
                                                int page_first, int page_step, const int* __restrict__ bt,
                                                const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
                                                size_t page_elems, int kh, int head_dim, float scale, int full_lo,
                                                int full_hi) {
  // full_lo..full_hi: the keys that every column of the wave sees (no mask needed inside)
  if (key_hi < key_lo) return;
  const int page_last = key_hi / PAGE_TOKENS;
  for (int pi = page_first; pi <= page_last; pi += page_step) {
    const size_t phys = readable_page(bt[pi]);
    const bf16* kp = k_cache + phys * page_elems + (size_t)kh * PAGE_TOKENS * head_dim;
    const bf16* vp = v_cache + phys * page_elems + (size_t)kh * head_dim * PAGE_TOKENS;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int key0 = pi * PAGE_TOKENS + half * 32;
      if (key0 > key_hi || key0 + 31 < key_lo) continue;  // uniform over the wave
      half_step<MAXDT, QT>(st, qreg, qpos, qlo, key0, kp + (size_t)half * 32 * head_dim, head_dim, vp + half * 32,
                           PAGE_TOKENS, head_dim, scale * LOG2E, key0 + 31 <= full_hi && key0 >= full_lo);
    }
  }
}

template <int MAXDT, int QT>
__device__ __forceinline__ void wave_state_init(WaveState<MAXDT, QT>& st) {
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    st.m[qt] = -1e30f;
    st.l[qt] = 0.f;
#pragma unroll
    for (int dt = 0; dt < MAXDT; ++dt) st.acc[qt][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
}

template <int MAXDT>
__device__ __forceinline__ void load_query(bf16x8 (&dst)[(MAXDT + 1) / 2], const bf16* row, int head_dim) {
  const int g = (threadIdx.x & (WAVE - 1)) >> 4;
#pragma unroll
  for (int c = 0; c < (MAXDT + 1) / 2; ++c) {
    const int d = c * 32 + g * 8;
    bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (row != nullptr && d < head_dim) v = load_bf16x8(row + d);
    dst[c] = v;
  }
}

// ==========================================================================
// prefill: a block is WAVES waves, each with 16*QT consecutive query
// tokens of one sequence, for one query head.  Keys come from the cache, so a
// chunk that continues a cached prefix works the same way.
// ==========================================================================
// A block covers PREFILL_QBLOCK tokens as WAVES waves of 16*QT tokens; large head sizes take
// fewer tokens per wave so that the accumulators stay in registers.
#define PREFILL_QBLOCK 128

template <int MAXDT, int QT, int WAVES>
__global__ void __launch_bounds__(WAVES* WAVE)
    attn_prefill_bf16_kernel(const bf16* __restrict__ q, long q_stride, bf16* __restrict__ out, long out_stride,
                             const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                             const int* __restrict__ qblock_start, const int* __restrict__ qblock_len,
                             const int* __restrict__ block_table, int table_stride, const bf16* __restrict__ k_cache,
                             const bf16* __restrict__ v_cache, int nheads, int kvheads, int head_dim, float scale,
                             int window) {
  static_assert(WAVES * QT * 16 == PREFILL_QBLOCK, "a block covers PREFILL_QBLOCK tokens");
  const int h = blockIdx.y;
  const int wave = threadIdx.x / WAVE;
  const int lane = threadIdx.x & (WAVE - 1);
  const int r = lane & 15;
  const int g = lane >> 4;
  const int t_begin = qblock_start[blockIdx.x];
  const int t_end = t_begin + qblock_len[blockIdx.x];
  const int t0 = t_begin + wave * QT * 16;
  if (t0 >= t_end) return;
  const int seq = seq_of_token[t0];
  if (seq < 0) return;
  const int kh = h / (nheads / kvheads);
  const int* bt = block_table + (size_t)seq * table_stride;
  const size_t page_elems = (size_t)kvheads * PAGE_TOKENS * head_dim;

  bf16x8 qreg[QT][(MAXDT + 1) / 2];
  int qpos[QT], qlo[QT];
  int key_hi = -1, key_lo = 0x7fffffff;
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int t = t0 + qt * 16 + r;
    const bool valid = t < t_end;
    load_query<MAXDT>(qreg[qt], valid ? q + (size_t)t * q_stride + (size_t)h * head_dim : nullptr, head_dim);
    qpos[qt] = valid ? positions[t] : -1;
    qlo[qt] = (valid && window > 0 && qpos[qt] - window + 1 > 0) ? qpos[qt] - window + 1 : 0;
  }
  // key range of the wave: tokens of a block are consecutive positions of one sequence
  {
    const int t_last = (t0 + QT * 16 < t_end ? t0 + QT * 16 : t_end) - 1;
    key_hi = positions[t_last];
    const int first = positions[t0];
    key_lo = (window > 0 && first - window + 1 > 0) ? first - window + 1 : 0;
  }

  WaveState<MAXDT, QT> st;
  wave_state_init(st);
  // every column sees the keys from the last token's window start up to the first token's position
  const int full_hi = positions[t0];
  const int full_lo = (window > 0 && key_hi - window + 1 > 0) ? key_hi - window + 1 : 0;
  attn_wave_pages<MAXDT, QT>(st, qreg, qpos, qlo, key_lo, key_hi, key_lo / PAGE_TOKENS, 1, bt, k_cache, v_cache,
                             page_elems, kh, head_dim, scale, full_lo, full_hi);

  const int ndt = head_dim / 16;
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    float l = st.l[qt];
    l += __shfl_xor(l, 16, WAVE);
    l += __shfl_xor(l, 32, WAVE);
    const int t = t0 + qt * 16 + r;
    if (t < t_end) {
      const float inv = l > 0.f ? 1.f / l : 0.f;
      bf16* orow = out + (size_t)t * out_stride + (size_t)h * head_dim;
#pragma unroll
      for (int dt = 0; dt < MAXDT; ++dt) {
        if (dt < ndt) {
          const f32x4 a = st.acc[qt][dt];
          const bf16x4 o = {(bf16)(a[0] * inv), (bf16)(a[1] * inv), (bf16)(a[2] * inv), (bf16)(a[3] * inv)};
          *reinterpret_cast<bf16x4*>(orow + dt * 16 + g * 4) = o;
        }
      }
    }
  }
}

// ==========================================================================
// prefill through LDS.  A block stages the pages of keys and values in LDS,
// two at a time: one is multiplied while the next is written.  It has four
// units: `hb` query heads of one kv group (they share the page) times 4/hb runs
// of 16*QT consecutive query tokens; a unit is two waves that take one half of
// every page each and meet at the end, which halves the chain of dependent
// steps of the longest block of a causal step.  Pages are fetched into
// registers two ahead of the one that is multiplied.
// ==========================================================================
#define LDS_PAD 8  // elements: rows 16 bytes apart from a multiple of the bank count

// EXACT: the head size is MAXDT * 16, known at compile time: the checks that let a smaller head size through
// the same code (a quarter of the vector instructions of a step) fall away.
template <int MAXDT, int QT, int UNITS, bool EXACT>
__global__ void __launch_bounds__(UNITS * 2 * WAVE) __attribute__((amdgpu_waves_per_eu(2, 2)))
    attn_prefill_lds_kernel(const bf16* __restrict__ q, long q_stride, bf16* __restrict__ out, long out_stride,
                            const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                            const int* __restrict__ qblock_start, const int* __restrict__ qblock_len,
                            int n_qblocks, const int* __restrict__ block_table, int table_stride,
                            const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache, int nheads,
                            int kvheads, int head_dim_arg, float scale, int window, int hb) {
  const int head_dim = EXACT ? MAXDT * 16 : head_dim_arg;
  constexpr int KS = MAXDT * 16 + LDS_PAD;    // LDS row stride of the key page [64][KS]
  constexpr int VS = PAGE_TOKENS + LDS_PAD;   // LDS row stride of the transposed value page [head_dim][VS]
  constexpr int THREADS = UNITS * 2 * WAVE;
  constexpr int CH = (MAXDT * 128 + THREADS - 1) / THREADS;  // 16-byte chunks a thread moves per page and operand (at most)
  constexpr int K_ELEMS = PAGE_TOKENS * KS, V_ELEMS = MAXDT * 16 * VS;
  // at the end the same memory carries one wave's state to its partner: UNITS waves x 64 lanes x (MAXDT * 4 + 2) floats
  constexpr int MERGE_BYTES = UNITS * WAVE * (MAXDT * 4 + 2) * 4;
  // two pages: one is multiplied while the next one is written
  constexpr int PAGE_ELEMS = K_ELEMS + V_ELEMS;
  constexpr int STAGE_BYTES = 2 * PAGE_ELEMS * 2 > MERGE_BYTES ? 2 * PAGE_ELEMS * 2 : MERGE_BYTES;
  __shared__ __attribute__((aligned(16))) unsigned char stage[STAGE_BYTES];
  bf16* const ks = reinterpret_cast<bf16*>(stage);  // page b: keys at ks + b * PAGE_ELEMS, values at vs + b * PAGE_ELEMS
  bf16* const vs = ks + K_ELEMS;

  // Blocks of a causal step differ in length, and the longest sets the time of the whole kernel: they go
  // first (workgroups are handed out in linear order), and the short ones fill in behind them.
  const int group = nheads / kvheads;
  const int tiles = group / hb;
  const int per_qb = kvheads * tiles;                 // blocks that share a query block
  const int qb = n_qblocks - 1 - (int)(blockIdx.x / per_qb);
  const int y = blockIdx.x % per_qb;
  const int kh = y / tiles;
  const int wave = threadIdx.x / WAVE;
  const int unit = wave % UNITS;  // which head and run of query tokens
  const int khalf = wave / UNITS; // the two waves of a unit take the two halves (32 keys each) of every page
  const int lane = threadIdx.x & (WAVE - 1);
  const int r = lane & 15;
  const int g = lane >> 4;
  const int h = kh * group + (y % tiles) * hb + unit % hb;
  const int t_begin = qblock_start[qb];
  const int t_end = t_begin + qblock_len[qb];
  const int seq = seq_of_token[t_begin];
  if (seq < 0) return;  // whole block: uniform
  const int* bt = block_table + (size_t)seq * table_stride;
  const size_t page_elems = (size_t)kvheads * PAGE_TOKENS * head_dim;

  // this wave's queries
  const int t0 = t_begin + (unit / hb) * QT * 16;
  const bool has_work = t0 < t_end;
  bf16x8 qreg[QT][(MAXDT + 1) / 2];
  int qpos[QT], qlo[QT];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int t = t0 + qt * 16 + r;
    const bool valid = t < t_end;
    load_query<MAXDT>(qreg[qt], valid ? q + (size_t)t * q_stride + (size_t)h * head_dim : nullptr, head_dim);
    qpos[qt] = valid ? positions[t] : -1;
    qlo[qt] = (valid && window > 0 && qpos[qt] - window + 1 > 0) ? qpos[qt] - window + 1 : 0;
  }
  int wave_hi = -1, wave_lo = 0, full_hi = -1, full_lo = 0;  // keys some / every column of the wave sees
  if (has_work) {
    const int t_last = (t0 + QT * 16 < t_end ? t0 + QT * 16 : t_end) - 1;
    wave_hi = positions[t_last];
    full_hi = positions[t0];
    wave_lo = (window > 0 && full_hi - window + 1 > 0) ? full_hi - window + 1 : 0;
    full_lo = (window > 0 && wave_hi - window + 1 > 0) ? wave_hi - window + 1 : 0;
  }
  // the block's keys: tokens of a block are consecutive positions of one sequence
  const int blk_first = positions[t_begin];
  const int blk_hi = positions[t_end - 1];
  const int blk_lo = (window > 0 && blk_first - window + 1 > 0) ? blk_first - window + 1 : 0;
  const int page_first = blk_lo / PAGE_TOKENS, page_last = blk_hi / PAGE_TOKENS;

  // cooperative copy: chunk id -> (row, 16-byte column) of the page in global memory and in LDS
  const int k_chunks = PAGE_TOKENS * head_dim / 8;  // per page; the value page has as many
  const int k_cols = head_dim / 8;
  // Pages are fetched PF pages ahead of the one that is multiplied (a page's loads take longer to arrive than
  // a page takes to multiply): PF sets of registers, used in turn.
  constexpr int PF = 2;
  bf16x8 kbuf[PF][CH], vbuf[PF][CH];
  auto fetch = [&](int pi, bf16x8 (&kb)[CH], bf16x8 (&vb)[CH]) {
    const size_t phys = readable_page(bt[pi]);
    const bf16* kp = k_cache + phys * page_elems + (size_t)kh * PAGE_TOKENS * head_dim;
    const bf16* vp = v_cache + phys * page_elems + (size_t)kh * head_dim * PAGE_TOKENS;
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      const int id = threadIdx.x + j * THREADS;
      const size_t at = id < k_chunks ? (size_t)id * 8 : 0;  // the page is contiguous; never a load behind a branch
      kb[j] = load_bf16x8(kp + at);
      vb[j] = load_bf16x8(vp + at);
    }
  };
  auto stash = [&](int which, const bf16x8 (&kb)[CH], const bf16x8 (&vb)[CH]) {
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      const int id = threadIdx.x + j * THREADS;
      if (id < k_chunks) {
        *reinterpret_cast<bf16x8*>(ks + which * PAGE_ELEMS + (id / k_cols) * KS + (id % k_cols) * 8) = kb[j];
        *reinterpret_cast<bf16x8*>(vs + which * PAGE_ELEMS + (id / 8) * VS + (id % 8) * 8) = vb[j];
      }
    }
  };

  WaveState<MAXDT, QT> st;
  wave_state_init(st);
  // (a fetch past the last page reads the last page again: cheaper than a branch around loads, behind which
  // the compiler loses count of the loads in flight and waits for all of them)
  // kbuf[i % PF], vbuf[i % PF]: page page_first + i on its way from memory.  The first page goes to LDS before
  // the loop; in the loop a page is multiplied while the next one is written to the other half of LDS and the
  // one PF further on is asked for: one barrier a page.
  fetch(page_first, kbuf[0], vbuf[0]);
  stash(0, kbuf[0], vbuf[0]);
#pragma unroll
  for (int d = 0; d < PF; ++d) fetch(page_first + 1 + d <= page_last ? page_first + 1 + d : page_last, kbuf[(1 + d) % PF], vbuf[(1 + d) % PF]);
  block_sync_lds();  // not __syncthreads(): the pages under way must not be waited for
  for (int p0 = page_first; p0 <= page_last; p0 += PF) {
#pragma unroll
    for (int d = 0; d < PF; ++d) {
      const int pi = p0 + d;  // past the last page (the loop runs in steps of PF pages): nothing but the barrier
      const int cur = d & 1;  // PF is even: the page's half of LDS
      if (pi + 1 <= page_last) stash(cur ^ 1, kbuf[(d + 1) % PF], vbuf[(d + 1) % PF]);
      fetch(pi + 1 + PF <= page_last ? pi + 1 + PF : page_last, kbuf[(d + 1) % PF], vbuf[(d + 1) % PF]);
      const int key0 = pi * PAGE_TOKENS + khalf * 32;
      if (has_work && pi <= page_last && !(key0 > wave_hi || key0 + 31 < wave_lo))  // uniform over the wave
        half_step<MAXDT, QT>(st, qreg, qpos, qlo, key0, ks + cur * PAGE_ELEMS + khalf * 32 * KS, KS,
                             vs + cur * PAGE_ELEMS + khalf * 32, VS, head_dim, scale * LOG2E,
                             key0 + 31 <= full_hi && key0 >= full_lo);
      block_sync_lds();  // the page just multiplied is overwritten after the next one
    }
  }
  __syncthreads();  // the loads still under way, before the memory changes its use

  // ---- the two waves of a unit meet: the second hands its state over, one run of 16 columns at a time ----
  const int ndt = head_dim / 16;
  float* const hand = reinterpret_cast<float*>(stage) + (size_t)(unit * WAVE + lane) * (MAXDT * 4 + 2);
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    if (khalf == 1) {
#pragma unroll
      for (int dt = 0; dt < MAXDT; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i) hand[dt * 4 + i] = st.acc[qt][dt][i];
      hand[MAXDT * 4] = st.m[qt];
      hand[MAXDT * 4 + 1] = st.l[qt];
    }
    __syncthreads();
    if (khalf == 0 && has_work) {
      const float m1 = hand[MAXDT * 4], l1 = hand[MAXDT * 4 + 1];
      const float m = fmaxf(st.m[qt], m1);
      const float f0 = __builtin_amdgcn_exp2f(st.m[qt] - m), f1 = __builtin_amdgcn_exp2f(m1 - m);  // base-2 maxima
      float l = st.l[qt] * f0 + l1 * f1;
      l += __shfl_xor(l, 16, WAVE);
      l += __shfl_xor(l, 32, WAVE);
      const int t = t0 + qt * 16 + r;
      if (t < t_end) {
        const float inv = l > 0.f ? 1.f / l : 0.f;
        bf16* orow = out + (size_t)t * out_stride + (size_t)h * head_dim;
#pragma unroll
        for (int dt = 0; dt < MAXDT; ++dt) {
          if (dt < ndt) {
            const f32x4 a = st.acc[qt][dt];
            const float* b = hand + dt * 4;
            const bf16x4 o = {(bf16)((a[0] * f0 + b[0] * f1) * inv), (bf16)((a[1] * f0 + b[1] * f1) * inv),
                              (bf16)((a[2] * f0 + b[2] * f1) * inv), (bf16)((a[3] * f0 + b[3] * f1) * inv)};
            *reinterpret_cast<bf16x4*>(orow + dt * 16 + g * 4) = o;
          }
        }
      }
    }
    __syncthreads();  // the memory carries the next run
  }
}

// ==========================================================================
// prefill through LDS with 32x32x16 products, for head sizes that are multiples of 32 up to 128.  The block is
// that of attn_prefill_lds_kernel (four units of two waves, pages staged two at a time, fetched two ahead); a
// wave's 32 query columns are one tile column.  On this GPU the 32x32x16 product runs at close to twice the
// rate of the 16x16x32 one for the same operand bytes, and the prefill is bound by the matrix unit.
//
// S^T = K Q^T: a tile of 32 keys x 32 queries; lane (j = lane % 32, hb = lane / 32) holds query column j and
// the 16 tile rows 8 (v / 4) + 4 hb + v % 4, v < 16.  Which key sits in which tile row is free: rows are dealt
// so that those 16 are the keys 8 hb .. 8 hb + 7 (v < 8) and 16 + 8 hb .. 16 + 8 hb + 7 (v >= 8), each eight
// the B operand of one step of O^T += V^T P^T, whose A operand is then one 16-byte read of a row of the
// transposed value page.
// ==========================================================================
template <int DT32>
struct WaveState32 {
  f32x16 acc[DT32];  // O^T: d = dt * 32 + 8 (v / 4) + 4 hb + v % 4, query column j
  float m, l;        // running maximum of the column (equal in its two lanes), this lane's share of the running sum
};

template <int DT32>
__device__ __forceinline__ void half_step32(WaveState32<DT32>& st, const bf16x8 (&qreg)[DT32 * 2], int qpos, int qlo,
                                            int key0, const bf16* kbase, int k_stride, const bf16* vbase, int v_stride,
                                            float scale2, bool full) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int j = lane & 31, hb = lane >> 5;
  // the key of tile row i = lane % 32 (this lane's row of the A operand): i = 8 blk + 4 h + e
  const int key_row = 16 * (j >> 4) + 8 * ((j >> 2) & 1) + 4 * ((j >> 3) & 1) + (j & 3);
  f32x16 sc;
#pragma unroll
  for (int v = 0; v < 16; ++v) sc[v] = 0.f;
  {
    bf16x8 ka[DT32 * 2];
#pragma unroll
    for (int c = 0; c < DT32 * 2; ++c) ka[c] = load_bf16x8(kbase + (size_t)key_row * k_stride + c * 16 + hb * 8);
#pragma unroll
    for (int c = 0; c < DT32 * 2; ++c) sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[c], qreg[c], sc, 0, 0, 0);
  }
  if (!full) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int key = key0 + 16 * (v >> 3) + 8 * hb + (v & 7);
      sc[v] = (key <= qpos && key >= qlo) ? sc[v] : -INFINITY;
    }
  }
  float mx = max3f(max3f(sc[0], sc[1], sc[2]), max3f(sc[3], sc[4], sc[5]), max3f(sc[6], sc[7], sc[8]));
  mx = max3f(mx, max3f(sc[9], sc[10], sc[11]), max3f(sc[12], sc[13], max2f(sc[14], sc[15])));
  {
    const unsigned u = __float_as_uint(mx);
    const auto halves = __builtin_amdgcn_permlane32_swap(u, u, false, false);  // the column's other lane
    mx = max2f(__uint_as_float(halves[0]), __uint_as_float(halves[1]));
  }
  const float m_new = max2f(st.m, mx * scale2);  // the scale is positive: scaled once, after the maximum
  const float alpha = __builtin_amdgcn_exp2f(st.m - m_new);
  st.m = m_new;
  float p[16], psum = 0.f;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    p[v] = __builtin_amdgcn_exp2f(fmaf(sc[v], scale2, -m_new));
    psum += p[v];
  }
  st.l = st.l * alpha + psum;
  bf16x8 pmat[2];
#pragma unroll
  for (int h = 0; h < 2; ++h)
    pmat[h] = bf16x8{(bf16)p[8 * h], (bf16)p[8 * h + 1], (bf16)p[8 * h + 2], (bf16)p[8 * h + 3],
                     (bf16)p[8 * h + 4], (bf16)p[8 * h + 5], (bf16)p[8 * h + 6], (bf16)p[8 * h + 7]};
  if (__any(alpha != 1.f)) {  // the running maximum seldom moves after the first keys
#pragma unroll
    for (int dt = 0; dt < DT32; ++dt) st.acc[dt] *= alpha;
  }
#pragma unroll
  for (int dt = 0; dt < DT32; ++dt) {
    bf16x8 va[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) va[h] = load_bf16x8(vbase + (size_t)(dt * 32 + j) * v_stride + 16 * h + 8 * hb);
#pragma unroll
    for (int h = 0; h < 2; ++h) st.acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[h], pmat[h], st.acc[dt], 0, 0, 0);
  }
}

template <int DT32, int UNITS>
__global__ void __launch_bounds__(UNITS * 2 * WAVE) __attribute__((amdgpu_waves_per_eu(2, 2)))
    attn_prefill_lds32_kernel(const bf16* __restrict__ q, long q_stride, bf16* __restrict__ out, long out_stride,
                              const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                              const int* __restrict__ qblock_start, const int* __restrict__ qblock_len,
                              int n_qblocks, const int* __restrict__ block_table, int table_stride,
                              const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache, int nheads,
                              int kvheads, float scale, int window, int hb) {
  constexpr int head_dim = DT32 * 32;
  constexpr int KS = head_dim + LDS_PAD;      // LDS row stride of the key page [64][KS]
  constexpr int VS = PAGE_TOKENS + LDS_PAD;   // LDS row stride of the transposed value page [head_dim][VS]
  constexpr int THREADS = UNITS * 2 * WAVE;
  constexpr int k_chunks = PAGE_TOKENS * head_dim / 8;  // 16-byte chunks of a page and operand
  constexpr int k_cols = head_dim / 8;
  constexpr int CH = (k_chunks + THREADS - 1) / THREADS;
  constexpr int K_ELEMS = PAGE_TOKENS * KS, V_ELEMS = head_dim * VS;
  // at the end the same memory carries one wave's state to its partner: UNITS waves x 64 lanes x (DT32 * 16 + 2) floats
  constexpr int MERGE_BYTES = UNITS * WAVE * (DT32 * 16 + 2) * 4;
  constexpr int PAGE_ELEMS = K_ELEMS + V_ELEMS;
  constexpr int STAGE_BYTES = 2 * PAGE_ELEMS * 2 > MERGE_BYTES ? 2 * PAGE_ELEMS * 2 : MERGE_BYTES;
  __shared__ __attribute__((aligned(16))) unsigned char stage[STAGE_BYTES];
  bf16* const ks = reinterpret_cast<bf16*>(stage);
  bf16* const vs = ks + K_ELEMS;

  // the longest blocks of a causal step go first (workgroups are handed out in linear order)
  const int group = nheads / kvheads;
  const int tiles = group / hb;
  const int per_qb = kvheads * tiles;
  const int qb = n_qblocks - 1 - (int)(blockIdx.x / per_qb);
  const int y = blockIdx.x % per_qb;
  const int kh = y / tiles;
  const int wave = threadIdx.x / WAVE;
  const int unit = wave % UNITS;   // which head and run of 32 query tokens
  const int khalf = wave / UNITS;  // the two waves of a unit take the two halves (32 keys each) of every page
  const int lane = threadIdx.x & (WAVE - 1);
  const int j = lane & 31, hbit = lane >> 5;
  const int h = kh * group + (y % tiles) * hb + unit % hb;
  const int t_begin = qblock_start[qb];
  const int t_end = t_begin + qblock_len[qb];
  const int seq = seq_of_token[t_begin];
  if (seq < 0) return;  // whole block: uniform
  const int* bt = block_table + (size_t)seq * table_stride;
  const size_t page_elems = (size_t)kvheads * PAGE_TOKENS * head_dim;

  // this wave's queries: column j is token t0 + j
  const int t0 = t_begin + (unit / hb) * 32;
  const bool has_work = t0 < t_end;
  const int t = t0 + j;
  const bool valid = t < t_end;
  bf16x8 qreg[DT32 * 2];
#pragma unroll
  for (int c = 0; c < DT32 * 2; ++c) {
    bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (valid) v = load_bf16x8(q + (size_t)t * q_stride + (size_t)h * head_dim + c * 16 + hbit * 8);
    qreg[c] = v;
  }
  const int qpos = valid ? positions[t] : -1;
  const int qlo = (valid && window > 0 && qpos - window + 1 > 0) ? qpos - window + 1 : 0;
  int wave_hi = -1, wave_lo = 0, full_hi = -1, full_lo = 0;  // keys some / every column of the wave sees
  if (has_work) {
    const int t_last = (t0 + 32 < t_end ? t0 + 32 : t_end) - 1;
    wave_hi = positions[t_last];
    full_hi = positions[t0];
    wave_lo = (window > 0 && full_hi - window + 1 > 0) ? full_hi - window + 1 : 0;
    full_lo = (window > 0 && wave_hi - window + 1 > 0) ? wave_hi - window + 1 : 0;
  }
  const int blk_first = positions[t_begin];
  const int blk_hi = positions[t_end - 1];
  const int blk_lo = (window > 0 && blk_first - window + 1 > 0) ? blk_first - window + 1 : 0;
  const int page_first = blk_lo / PAGE_TOKENS, page_last = blk_hi / PAGE_TOKENS;

  constexpr int PF = 2;
  bf16x8 kbuf[PF][CH], vbuf[PF][CH];
  auto fetch = [&](int pi, bf16x8 (&kb)[CH], bf16x8 (&vb)[CH]) {
    const size_t phys = readable_page(bt[pi]);
    const bf16* kp = k_cache + phys * page_elems + (size_t)kh * PAGE_TOKENS * head_dim;
    const bf16* vp = v_cache + phys * page_elems + (size_t)kh * head_dim * PAGE_TOKENS;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int id = threadIdx.x + c * THREADS;
      const size_t at = id < k_chunks ? (size_t)id * 8 : 0;  // the page is contiguous; never a load behind a branch
      kb[c] = load_bf16x8(kp + at);
      vb[c] = load_bf16x8(vp + at);
    }
  };
  auto stash = [&](int which, const bf16x8 (&kb)[CH], const bf16x8 (&vb)[CH]) {
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int id = threadIdx.x + c * THREADS;
      if (id < k_chunks) {
        *reinterpret_cast<bf16x8*>(ks + which * PAGE_ELEMS + (id / k_cols) * KS + (id % k_cols) * 8) = kb[c];
        *reinterpret_cast<bf16x8*>(vs + which * PAGE_ELEMS + (id / 8) * VS + (id % 8) * 8) = vb[c];
      }
    }
  };

  WaveState32<DT32> st;
  st.m = -1e30f, st.l = 0.f;
#pragma unroll
  for (int dt = 0; dt < DT32; ++dt)
#pragma unroll
    for (int v = 0; v < 16; ++v) st.acc[dt][v] = 0.f;

  fetch(page_first, kbuf[0], vbuf[0]);
  stash(0, kbuf[0], vbuf[0]);
#pragma unroll
  for (int d = 0; d < PF; ++d) fetch(page_first + 1 + d <= page_last ? page_first + 1 + d : page_last, kbuf[(1 + d) % PF], vbuf[(1 + d) % PF]);
  block_sync_lds();  // not __syncthreads(): the pages under way must not be waited for
  for (int p0 = page_first; p0 <= page_last; p0 += PF) {
#pragma unroll
    for (int d = 0; d < PF; ++d) {
      const int pi = p0 + d;  // past the last page (the loop runs in steps of PF pages): nothing but the barrier
      const int cur = d & 1;  // PF is even: the page's half of LDS
      if (pi + 1 <= page_last) stash(cur ^ 1, kbuf[(d + 1) % PF], vbuf[(d + 1) % PF]);
      fetch(pi + 1 + PF <= page_last ? pi + 1 + PF : page_last, kbuf[(d + 1) % PF], vbuf[(d + 1) % PF]);
      const int key0 = pi * PAGE_TOKENS + khalf * 32;
      if (has_work && pi <= page_last && !(key0 > wave_hi || key0 + 31 < wave_lo))  // uniform over the wave
        half_step32<DT32>(st, qreg, qpos, qlo, key0, ks + cur * PAGE_ELEMS + khalf * 32 * KS, KS,
                          vs + cur * PAGE_ELEMS + khalf * 32, VS, scale * LOG2E, key0 + 31 <= full_hi && key0 >= full_lo);
      block_sync_lds();  // the page just multiplied is overwritten after the next one
    }
  }
  __syncthreads();  // the loads still under way, before the memory changes its use

  // ---- the two waves of a unit meet: the second hands its state over ----
  float* const hand = reinterpret_cast<float*>(stage) + (size_t)(unit * WAVE + lane) * (DT32 * 16 + 2);
  if (khalf == 1) {
#pragma unroll
    for (int dt = 0; dt < DT32; ++dt)
#pragma unroll
      for (int v = 0; v < 16; ++v) hand[dt * 16 + v] = st.acc[dt][v];
    hand[DT32 * 16] = st.m;
    hand[DT32 * 16 + 1] = st.l;
  }
  __syncthreads();
  if (khalf == 0 && has_work) {
    const float m1 = hand[DT32 * 16], l1 = hand[DT32 * 16 + 1];
    const float m = fmaxf(st.m, m1);
    const float f0 = __builtin_amdgcn_exp2f(st.m - m), f1 = __builtin_amdgcn_exp2f(m1 - m);  // base-2 maxima
    float l = st.l * f0 + l1 * f1;
    l += __shfl_xor(l, 32, WAVE);
    if (valid) {
      const float inv = l > 0.f ? 1.f / l : 0.f;
      bf16* orow = out + (size_t)t * out_stride + (size_t)h * head_dim;
#pragma unroll
      for (int dt = 0; dt < DT32; ++dt) {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const float* o1 = hand + dt * 16 + b * 4;
          const bf16x4 o = {(bf16)((st.acc[dt][b * 4] * f0 + o1[0] * f1) * inv), (bf16)((st.acc[dt][b * 4 + 1] * f0 + o1[1] * f1) * inv),
                            (bf16)((st.acc[dt][b * 4 + 2] * f0 + o1[2] * f1) * inv), (bf16)((st.acc[dt][b * 4 + 3] * f0 + o1[3] * f1) * inv)};
          *reinterpret_cast<bf16x4*>(orow + dt * 32 + b * 8 + hbit * 4) = o;
        }
      }
    }
  }
}

// ==========================================================================
// decode: one query token per sequence.  Grid (split, kv head x head tile,
// token); the 16 columns of a wave's tiles are query heads that share the kv
// head.  Every sequence deals its own pages out over the splits; the waves of
// a block (up to 8) take the pages of its split in turn and meet in LDS; the
// splits of a token meet in attn_decode_merge_kernel.  For a small batch many
// small blocks keep the whole cache in flight at once; for a large one a block
// takes a whole sequence, and the long sequences go first.
// ==========================================================================
// The arithmetic of HALVES halves of 32 keys starting at key0, for operands that are already in registers:
// kreg[hf][tile][c] the keys of the two score tiles (rows dealt as key_a below says), vreg[hf][dt] the values.
template <int MAXDT, int HALVES>
__device__ __forceinline__ void decode_math(WaveState<MAXDT, 1>& st, const bf16x8 (&qreg)[(MAXDT + 1) / 2], int qpos,
                                            int qlo, int key0, const bf16x8 (&kreg)[HALVES][2][(MAXDT + 1) / 2],
                                            const bf16x8 (&vreg)[HALVES][MAXDT], int head_dim, float scale2) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int g = lane >> 4;
  const int ndt = head_dim / 16;
  const int nchunk = (head_dim + 31) / 32;
#pragma unroll
  for (int hf = 0; hf < HALVES; ++hf) {
    const int k0 = key0 + hf * 32;
    f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < (MAXDT + 1) / 2; ++c) {
      if (c < nchunk) {
        sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kreg[hf][0][c], qreg[c], sa, 0, 0, 0);
        sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kreg[hf][1][c], qreg[c], sb, 0, 0, 0);
      }
    }
    if (!(k0 + 31 <= qpos && k0 >= qlo)) {  // uniform: not all 32 keys are visible
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int ja = k0 + g * 8 + i;  // the accumulator's rows 4 g + i hold these keys
        const int jb = ja + 4;
        sa[i] = (ja <= qpos && ja >= qlo) ? sa[i] : -INFINITY;
        sb[i] = (jb <= qpos && jb >= qlo) ? sb[i] : -INFINITY;
      }
    }
    float mx = max3f(max3f(sa[0], sa[1], sa[2]), max3f(sa[3], sb[0], sb[1]), max2f(sb[2], sb[3]));
    mx = max_over_lane_groups(mx);
    const float m_new = max2f(st.m[0], mx * scale2);  // the scale is positive: scaled once, after the maximum
    const float alpha = __builtin_amdgcn_exp2f(st.m[0] - m_new);
    st.m[0] = m_new;
    float pa[4], pb[4], psum = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      pa[i] = __builtin_amdgcn_exp2f(fmaf(sa[i], scale2, -m_new));
      pb[i] = __builtin_amdgcn_exp2f(fmaf(sb[i], scale2, -m_new));
      psum += pa[i] + pb[i];
    }
    st.l[0] = st.l[0] * alpha + psum;
    const bf16x8 pmat = {(bf16)pa[0], (bf16)pa[1], (bf16)pa[2], (bf16)pa[3],
                         (bf16)pb[0], (bf16)pb[1], (bf16)pb[2], (bf16)pb[3]};
    if (__any(alpha != 1.f)) {  // the running maximum seldom moves after the first keys
#pragma unroll
      for (int dt = 0; dt < MAXDT; ++dt)
        if (dt < ndt) st.acc[0][dt] *= alpha;
    }
#pragma unroll
    for (int dt = 0; dt < MAXDT; ++dt) {
      if (dt < ndt) st.acc[0][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vreg[hf][dt], pmat, st.acc[0][dt], 0, 0, 0);
    }
  }
}

template <int MAXDT, int HALVES>
__device__ __forceinline__ void decode_keys(WaveState<MAXDT, 1>& st, const bf16x8 (&qreg)[(MAXDT + 1) / 2], int qpos,
                                            int qlo, int key0, const bf16* __restrict__ kp,
                                            const bf16* __restrict__ vp, int head_dim, float scale2) {
  // HALVES halves of 32 keys starting at key0 (kp/vp point at the page, `first` is the half inside it)
  const int lane = threadIdx.x & (WAVE - 1);
  const int r = lane & 15;
  const int g = lane >> 4;
  const int ndt = head_dim / 16;
  const int nchunk = (head_dim + 31) / 32;
  const int first = (key0 % PAGE_TOKENS) / 32;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  // Which key sits in which row of the two score tiles is free, as long as the second product pairs every
  // probability with its value.  Rows are dealt so that lane group g ends up with the probabilities of the
  // 8 consecutive keys 8 g .. 8 g + 7 (tile a: 8 g + i, tile b: 8 g + 4 + i): their values are then one
  // 16-byte load per row of the transposed page.
  const int key_a = (r >> 2) * 8 + (r & 3);
  bf16x8 kreg[HALVES][2][(MAXDT + 1) / 2];
  bf16x8 vreg[HALVES][MAXDT];
#pragma unroll
  for (int hf = 0; hf < HALVES; ++hf) {
#pragma unroll
    for (int c = 0; c < (MAXDT + 1) / 2; ++c) {
      const int d = c * 32 + g * 8;
      const bool ok = c < nchunk && d < head_dim;
      kreg[hf][0][c] = ok ? load_bf16x8(kp + (size_t)((first + hf) * 32 + key_a) * head_dim + d) : zero8;
      kreg[hf][1][c] = ok ? load_bf16x8(kp + (size_t)((first + hf) * 32 + key_a + 4) * head_dim + d) : zero8;
    }
#pragma unroll
    for (int dt = 0; dt < MAXDT; ++dt)
      vreg[hf][dt] = dt < ndt ? load_bf16x8(vp + (size_t)(dt * 16 + r) * PAGE_TOKENS + (first + hf) * 32 + g * 8) : zero8;
  }
  decode_math<MAXDT, HALVES>(st, qreg, qpos, qlo, key0, kreg, vreg, head_dim, scale2);
}

// Pages of head size 128 by way of the wave's own 16 KB of LDS.  The page of a kv head is 16 KB of keys and
// 16 KB of values, each contiguous: the wave loads them 1 KB an instruction (what the memory system streams
// best; the operand layout takes 64 bytes from each of 16 rows and fetches every line twice), writes them to
// LDS as loaded and reads the MFMA operands back: first the keys, then, through the same buffer, the values.
// 16-byte pieces are XOR-swizzled so that both directions spread over the banks.
//
// The wave's pages are a pipeline through one set of 16 load registers: as soon as the keys of a page are in
// LDS the registers take the loads of its values, and as soon as those are in LDS, the loads of the next
// page's keys; so the memory always works on the wave's next 16 KB while the matrix unit works on the last.
// A compute unit's loads queue up behind one another (16 KB asked for when the unit's other waves have just
// asked for theirs take some microseconds); a wave that asks again the moment its registers are free keeps
// that queue full instead of waiting at its end once a page.
__device__ __forceinline__ void staged_load(bf16x8 (&raw)[16], const bf16* __restrict__ p) {
  const int lane = threadIdx.x & (WAVE - 1);
#pragma unroll
  for (int i = 0; i < 16; ++i) raw[i] = load_bf16x8(p + i * 512 + lane * 8);
}

// One page: its keys are on their way into raw; vp points at its values, kn (PREFETCH) at the next page's
// keys.  The softmax takes the page's 64 keys at once.
template <bool PREFETCH>
__device__ __forceinline__ void staged_page_step(WaveState<8, 1>& st, const bf16x8 (&qreg)[4], int qpos, int qlo,
                                                 int key0, bf16x8 (&raw)[16], const bf16* __restrict__ vp,
                                                 const bf16* __restrict__ kn, bf16* __restrict__ buf, float scale2) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int r = lane & 15;
  const int g = lane >> 4;
  // keys: row = token (256 bytes = 16 pieces), piece ^ key(token); the 16 tokens of a score tile have the keys 0..15
  {
    const int piece = lane & 15;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int token = i * 4 + (lane >> 4);
      const int key = (((token >> 3) & 3) << 2) | (token & 3);
      *reinterpret_cast<bf16x8*>(buf + token * 128 + ((piece ^ key) & 15) * 8) = raw[i];
    }
  }
  __builtin_amdgcn_wave_barrier();
  staged_load(raw, vp);
  // Which key sits in which row of the two score tiles: see decode_keys.  The swizzle key of row key_a is r,
  // and so is that of key_a + 4.
  const int key_a = (r >> 2) * 8 + (r & 3);
  f32x4 sa[2], sb[2];
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    bf16x8 ka[4], kb[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      ka[c] = *reinterpret_cast<const bf16x8*>(buf + (hf * 32 + key_a) * 128 + (((c * 4 + g) ^ r) & 15) * 8);
      kb[c] = *reinterpret_cast<const bf16x8*>(buf + (hf * 32 + key_a + 4) * 128 + (((c * 4 + g) ^ r) & 15) * 8);
    }
    sa[hf] = f32x4{0.f, 0.f, 0.f, 0.f};
    sb[hf] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      sa[hf] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[c], qreg[c], sa[hf], 0, 0, 0);
      sb[hf] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb[c], qreg[c], sb[hf], 0, 0, 0);
    }
  }

  if (!(key0 + PAGE_TOKENS - 1 <= qpos && key0 >= qlo)) {  // uniform: not all 64 keys are visible
#pragma unroll
    for (int hf = 0; hf < 2; ++hf)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int ja = key0 + hf * 32 + g * 8 + i;  // the accumulator's rows 4 g + i hold these keys
        const int jb = ja + 4;
        sa[hf][i] = (ja <= qpos && ja >= qlo) ? sa[hf][i] : -INFINITY;
        sb[hf][i] = (jb <= qpos && jb >= qlo) ? sb[hf][i] : -INFINITY;
      }
  }
  float mx = -INFINITY;
#pragma unroll
  for (int hf = 0; hf < 2; ++hf)
    mx = max3f(max3f(mx, sa[hf][0], sa[hf][1]), max3f(sa[hf][2], sa[hf][3], sb[hf][0]), max3f(sb[hf][1], sb[hf][2], sb[hf][3]));
  mx = max_over_lane_groups(mx);
  const float m_new = max2f(st.m[0], mx * scale2);  // the scale is positive: scaled once, after the maximum
  const float alpha = __builtin_amdgcn_exp2f(st.m[0] - m_new);
  st.m[0] = m_new;
  bf16x8 pmat[2];
  float psum = 0.f;
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    float pa[4], pb[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      pa[i] = __builtin_amdgcn_exp2f(fmaf(sa[hf][i], scale2, -m_new));
      pb[i] = __builtin_amdgcn_exp2f(fmaf(sb[hf][i], scale2, -m_new));
      psum += pa[i] + pb[i];
    }
    pmat[hf] = bf16x8{(bf16)pa[0], (bf16)pa[1], (bf16)pa[2], (bf16)pa[3], (bf16)pb[0], (bf16)pb[1], (bf16)pb[2], (bf16)pb[3]};
  }
  st.l[0] = st.l[0] * alpha + psum;
  if (__any(alpha != 1.f)) {  // the running maximum seldom moves after the first keys
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) st.acc[0][dt] *= alpha;
  }

  __builtin_amdgcn_wave_barrier();  // the keys have been read: the buffer takes the values
  // values: row = d (128 bytes = 8 pieces of 8 tokens), piece ^ (d / 2): two rows fill the banks once
  {
    const int piece = lane & 7;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int d = i * 8 + (lane >> 3);
      *reinterpret_cast<bf16x8*>(buf + d * 64 + ((piece ^ (d >> 1)) & 7) * 8) = raw[i];
    }
  }
  __builtin_amdgcn_wave_barrier();
  if (PREFETCH) staged_load(raw, kn);
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    bf16x8 vreg[8];
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) {
      const int d = dt * 16 + r;
      vreg[dt] = *reinterpret_cast<const bf16x8*>(buf + d * 64 + (((hf * 4 + g) ^ (d >> 1)) & 7) * 8);
    }
#pragma unroll
    for (int dt = 0; dt < 8; ++dt)
      st.acc[0][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vreg[dt], pmat[hf], st.acc[0][dt], 0, 0, 0);
  }
  __builtin_amdgcn_wave_barrier();  // the values have been read: the buffer is free for the next page's keys
}

// The pages first, first + stride, ... <= last of a sequence, for kv head kh.
__device__ __forceinline__ void decode_pages_staged(WaveState<8, 1>& st, const bf16x8 (&qreg)[4], int qpos, int qlo,
                                                    int first, int stride, int last, const int* __restrict__ bt,
                                                    const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
                                                    size_t page_elems, int kh, bf16* __restrict__ buf, float scale2) {
  if (first > last) return;
  const size_t head_off = (size_t)kh * PAGE_TOKENS * 128;
  bf16x8 raw[16];
  size_t phys = readable_page(uniform_load(bt + first));
  staged_load(raw, k_cache + phys * page_elems + head_off);
  int pi = first;
  for (; pi + stride <= last; pi += stride) {
    const size_t next = readable_page(uniform_load(bt + pi + stride));
    staged_page_step<true>(st, qreg, qpos, qlo, pi * PAGE_TOKENS, raw, v_cache + phys * page_elems + head_off,
                           k_cache + next * page_elems + head_off, buf, scale2);
    phys = next;
  }
  staged_page_step<false>(st, qreg, qpos, qlo, pi * PAGE_TOKENS, raw, v_cache + phys * page_elems + head_off, nullptr,
                          buf, scale2);
}

// The pages that split `split` of `n_splits` takes of a sequence whose visible keys are lo..pos: every
// sequence's own pages are dealt out evenly, so that in a batch of unequal lengths every block has work in
// proportion to its sequence.  Returns the number of splits that have pages at all (the first ones).
__device__ __forceinline__ int split_pages(int lo, int pos, int n_splits, int split, int* page_lo, int* page_hi) {
  const int first_page = lo / PAGE_TOKENS, last_page = pos / PAGE_TOKENS;
  const int span = last_page - first_page + 1;
  const int per = (span + n_splits - 1) / n_splits;
  *page_lo = first_page + split * per;
  *page_hi = *page_lo + per - 1 < last_page ? *page_lo + per - 1 : last_page;
  return (span + per - 1) / per;
}

// Grid (split, kv head x head tile, token).  The waves of a block take the pages of its split in turn and
// meet in LDS; the splits of a token meet in the merge kernel.  (Merging in the block that finishes last,
// behind a device-wide fence and a counter, was measured four times slower: the fence writes back and
// invalidates the whole L2 of the block's XCD while the other blocks stream through it.)
// STAGED (head size 128 only): pages go through LDS (decode_page_staged), 16 KB a wave.
template <int MAXDT, int MAXW, bool STAGED>
__global__ void __launch_bounds__(MAXW* WAVE) __attribute__((amdgpu_waves_per_eu(MAXDT <= 8 ? 2 : 1)))
    attn_decode_bf16_kernel(const bf16* __restrict__ q, long q_stride, bf16* __restrict__ out, long out_stride,
                            float* __restrict__ part_o, float* __restrict__ part_ml, int n_splits,
                            const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                            const int* __restrict__ block_table, int table_stride, const bf16* __restrict__ k_cache,
                            const bf16* __restrict__ v_cache, int nheads, int kvheads, int head_dim, float scale,
                            int window, int tile_cols, const int* __restrict__ row_order) {
  extern __shared__ float lds_dynamic[];  // not staged: [wave][tile_cols columns][head_dim + 2]
  __shared__ __attribute__((aligned(16))) bf16 stage[STAGED ? MAXW * 8192 : 8];
  // where the waves' partial results meet: a region of its own, or (staged) the head of each wave's page buffer
  float* const lds = STAGED ? reinterpret_cast<float*>(stage) : lds_dynamic;
  const int wave_stride = STAGED ? 4096 : tile_cols * (head_dim + 2);  // floats
  const int split = blockIdx.x;
  const int group = nheads / kvheads;
  const int tiles_per_kv = (group + tile_cols - 1) / tile_cols;
  const int kh = blockIdx.y / tiles_per_kv;
  const int ht = blockIdx.y % tiles_per_kv;
  // blocks are handed out in the order of their index: with the rows sorted by length the long ones go first
  const int t = row_order != nullptr ? uniform_load(row_order + blockIdx.z) : (int)blockIdx.z;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);  // uniform: table entries load as scalars
  const int n_waves = blockDim.x / WAVE;
  const int lane = threadIdx.x & (WAVE - 1);
  const int r = lane & 15;
  const int g = lane >> 4;
  const int seq = uniform_load(seq_of_token + t);
  const int cols = group - ht * tile_cols < tile_cols ? group - ht * tile_cols : tile_cols;  // query heads here
  const int head0 = kh * group + ht * tile_cols;
  // A block without keys (a padding row, or a split beyond the sequence's pages) leaves a maximum that marks its
  // partial result as empty: the merge kernel then needs no index data to tell which splits count.
  auto leave_empty = [&]() {
    if (n_splits > 1 && (int)threadIdx.x < cols) {
      const size_t base = ((size_t)t * nheads + head0 + threadIdx.x) * n_splits + split;
      part_ml[base * 2] = DECODE_EMPTY;
      part_ml[base * 2 + 1] = 0.f;
    }
  };
  if (seq < 0) {
    if (n_splits == 1)
      for (int i = threadIdx.x; i < cols * head_dim; i += blockDim.x)
        out[(size_t)t * out_stride + (size_t)head0 * head_dim + i] = (bf16)0.f;
    leave_empty();
    return;
  }
  const int pos = uniform_load(positions + t);
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  int page_lo, page_hi;
  if (split >= split_pages(lo, pos, n_splits, split, &page_lo, &page_hi)) {
    leave_empty();
    return;
  }

  const int* bt = block_table + (size_t)seq * table_stride;
  const size_t page_elems = (size_t)kvheads * PAGE_TOKENS * head_dim;

  bf16x8 qreg[(MAXDT + 1) / 2];
  load_query<MAXDT>(qreg, r < cols ? q + (size_t)t * q_stride + (size_t)(head0 + r) * head_dim : nullptr, head_dim);

  WaveState<MAXDT, 1> st;
  wave_state_init(st);
  if (STAGED) {
    if constexpr (MAXDT == 8)
      decode_pages_staged(st, qreg, pos, lo, page_lo + wave, n_waves, page_hi, bt, k_cache, v_cache, page_elems, kh,
                          stage + wave * 8192, scale * LOG2E);
  } else {
    for (int pi = page_lo + wave; pi <= page_hi; pi += n_waves) {
      const size_t phys = readable_page(uniform_load(bt + pi));
      const bf16* kp = k_cache + phys * page_elems + (size_t)kh * PAGE_TOKENS * head_dim;
      const bf16* vp = v_cache + phys * page_elems + (size_t)kh * head_dim * PAGE_TOKENS;
      if (MAXDT <= 8) {
        decode_keys<MAXDT, 2>(st, qreg, pos, lo, pi * PAGE_TOKENS, kp, vp, head_dim, scale * LOG2E);
      } else {  // large heads: half a page at a time keeps the loads in registers
        decode_keys<MAXDT, 1>(st, qreg, pos, lo, pi * PAGE_TOKENS, kp, vp, head_dim, scale * LOG2E);
        decode_keys<MAXDT, 1>(st, qreg, pos, lo, pi * PAGE_TOKENS + 32, kp, vp, head_dim, scale * LOG2E);
      }
    }
  }

  // ---- the waves of the block meet in LDS --------------------------------
  const int ndt = head_dim / 16;
  const int cstride = head_dim + 2;
  float l = st.l[0];
  l += __shfl_xor(l, 16, WAVE);
  l += __shfl_xor(l, 32, WAVE);
  if (r < cols) {
    float* dst = lds + (size_t)wave * wave_stride + r * cstride;
    if (g == 0) {
      dst[head_dim] = st.m[0];
      dst[head_dim + 1] = l;
    }
#pragma unroll
    for (int dt = 0; dt < MAXDT; ++dt)
      if (dt < ndt)
#pragma unroll
        for (int i = 0; i < 4; ++i) dst[dt * 16 + g * 4 + i] = st.acc[0][dt][i];
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < cols * head_dim; idx += blockDim.x) {
    const int c = idx / head_dim;
    const int d = idx % head_dim;
    float m = -1e30f;
    for (int w = 0; w < n_waves; ++w) m = fmaxf(m, lds[(size_t)w * wave_stride + c * cstride + head_dim]);
    float o = 0.f, lsum = 0.f;
    for (int w = 0; w < n_waves; ++w) {
      const float* src = lds + (size_t)w * wave_stride + c * cstride;
      const float f = __builtin_amdgcn_exp2f(src[head_dim] - m);  // maxima are base-2 logarithms
      o += f * src[d];
      lsum += f * src[head_dim + 1];
    }
    const int head = head0 + c;
    if (n_splits == 1) {
      out[(size_t)t * out_stride + (size_t)head * head_dim + d] = (bf16)(lsum > 0.f ? o / lsum : 0.f);
    } else {
      const size_t base = ((size_t)t * nheads + head) * n_splits + split;
      part_o[base * head_dim + d] = o;
      if (d == 0) {
        part_ml[base * 2] = m;
        part_ml[base * 2 + 1] = lsum;
      }
    }
  }
}

// one block per (head, token): combine the partial results of the splits.  The loads of four splits are
// issued together (a loop that loads, waits and combines split by split pays the memory's latency per split),
// and none of them waits for index data: a split without keys carries the maximum DECODE_EMPTY, and whatever
// its other numbers are, they are set aside (a row of which every split is empty, a padding row, becomes zeros).
__global__ void attn_decode_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                         bf16* __restrict__ out, long out_stride, int nheads, int head_dim, int n_splits) {
  const int h = blockIdx.x;
  const int t = blockIdx.y;
  const size_t base = ((size_t)t * nheads + h) * n_splits;
  for (int d = threadIdx.x; d < head_dim; d += blockDim.x) {
    float m = DECODE_EMPTY, o = 0.f, l = 0.f;  // running maximum (a base-2 logarithm), sum of values, sum of weights
    for (int s0 = 0; s0 < n_splits; s0 += 4) {
      float ms[4], ls[4], os[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int s = s0 + i < n_splits ? s0 + i : n_splits - 1;  // past the end: the last split again, given no weight
        ms[i] = part_ml[(base + s) * 2];
        ls[i] = part_ml[(base + s) * 2 + 1];
        os[i] = part_o[(base + s) * head_dim + d];
      }
      bool counts[4];
      float m_new = m;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        counts[i] = s0 + i < n_splits && ms[i] > 0.5f * DECODE_EMPTY;
        if (counts[i]) m_new = fmaxf(m_new, ms[i]);
      }
      const float keep = __builtin_amdgcn_exp2f(m - m_new);
      o *= keep;
      l *= keep;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float f = __builtin_amdgcn_exp2f(ms[i] - m_new);
        o += counts[i] ? f * os[i] : 0.f;
        l += counts[i] ? f * ls[i] : 0.f;
      }
      m = m_new;
    }
    out[(size_t)t * out_stride + (size_t)h * head_dim + d] = (bf16)(l > 0.f ? o / l : 0.f);
  }
}

// ==========================================================================
// host entry points
// ==========================================================================
static int check_common(const char* name, int n_tokens, int nheads, int kvheads, int head_dim, long q_stride,
                        long out_stride) {
  FMS_REQUIRE(n_tokens > 0 && nheads > 0 && kvheads > 0, "%s: bad sizes", name);
  FMS_REQUIRE(nheads % kvheads == 0, "%s: %d query heads are no multiple of %d kv heads", name, nheads, kvheads);
  FMS_REQUIRE(head_dim > 0 && head_dim <= 256, "%s: head size %d is outside 1..256", name, head_dim);
  FMS_REQUIRE(q_stride >= (long)nheads * head_dim && out_stride >= (long)nheads * head_dim,
              "%s: row strides are smaller than heads x head size", name);
  return 0;
}

extern "C" int fmsamd_attn_generic(const void* q, long q_stride, void* out, long out_stride, int dtype,
                                   const int* positions, const int* seq_of_token, const int* block_table,
                                   int table_stride, const void* k_cache, const void* v_cache, int n_tokens,
                                   int nheads, int kvheads, int head_dim, float scale, int window,
                                   const float* slopes, float soft_cap, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (check_common("attn_generic", n_tokens, nheads, kvheads, head_dim, q_stride, out_stride)) return -1;
  FMS_REQUIRE(n_tokens <= 65535, "attn_generic: %d tokens exceed one launch (65535)", n_tokens);
  FMS_REQUIRE(soft_cap >= 0.f, "attn_generic: soft cap %g is negative", (double)soft_cap);
  dim3 grid(nheads, n_tokens);
  const bool terms = slopes != nullptr || soft_cap > 0.f;
#define FMS_GEN(T, TERMS)                                                                                              \
  attn_generic_kernel<T, TERMS><<<grid, GEN_THREADS, 0, stream>>>(                                                     \
      (const T*)q, q_stride, (T*)out, out_stride, positions, seq_of_token, block_table, table_stride, (const T*)k_cache, \
      (const T*)v_cache, nheads, kvheads, head_dim, scale, window, slopes, soft_cap)
  if (dtype == FMS_F32) {
    if (terms)
      FMS_GEN(float, true);
    else
      FMS_GEN(float, false);
  } else if (dtype == FMS_BF16) {
    if (terms)
      FMS_GEN(bf16, true);
    else
      FMS_GEN(bf16, false);
  } else {
    FMS_REQUIRE(false, "attn_generic: unknown dtype %d", dtype);
  }
#undef FMS_GEN
  FMS_LAUNCH_CHECK("attn_generic");
  return 0;
}

// How the bfloat16 prefill kernel cuts a step: the heads of a kv group that share a block, and the
// query tokens a block covers.  Head sizes up to 128 go through LDS (4 units = hb heads x 4/hb runs of
// 32 tokens); larger ones keep the direct kernel (128 tokens).
#define LDS_QT 2
#define LDS_UNITS 4  // units of a block: heads of a kv group (at most) times runs of query tokens
static void prefill_shape(int nheads, int kvheads, int head_dim, int n_tokens, int* hb, int* qt, int* qblock) {
  const int group = nheads / kvheads;
  (void)n_tokens;
  if (head_dim > 128) {
    *hb = 1, *qt = 0, *qblock = PREFILL_QBLOCK;
    return;
  }
  *hb = (LDS_UNITS >= 4 && group % 4 == 0) ? 4 : (group % 2 == 0 ? 2 : 1);
  *qt = LDS_QT;
  *qblock = (LDS_UNITS / *hb) * *qt * 16;
}

extern "C" int fmsamd_attn_prefill_qblock(int nheads, int kvheads, int head_dim, int n_tokens) {
  int hb, qt, qblock;
  if (nheads <= 0 || kvheads <= 0 || nheads % kvheads) return PREFILL_QBLOCK;
  prefill_shape(nheads, kvheads, head_dim, n_tokens, &hb, &qt, &qblock);
  return qblock;
}

extern "C" int fmsamd_attn_prefill_bf16(const void* q, long q_stride, void* out, long out_stride,
                                        const int* positions, const int* seq_of_token, const int* qblock_start,
                                        const int* qblock_len, int n_qblocks, int qblock_tokens,
                                        const int* block_table, int table_stride, const void* k_cache,
                                        const void* v_cache, int n_tokens, int nheads, int kvheads, int head_dim,
                                        float scale, int window, hipStream_t stream) {
  if (n_tokens == 0 || n_qblocks == 0) return 0;
  if (check_common("attn_prefill_bf16", n_tokens, nheads, kvheads, head_dim, q_stride, out_stride)) return -1;
  FMS_REQUIRE(head_dim % 16 == 0, "attn_prefill_bf16: head size %d is no multiple of 16", head_dim);
  FMS_REQUIRE(q_stride % 8 == 0 && out_stride % 4 == 0, "attn_prefill_bf16: row strides must keep 16-byte alignment");
  FMS_REQUIRE(nheads <= 65535, "attn_prefill_bf16: too many heads");
  const int group = nheads / kvheads;
  if (head_dim > 128) {
    FMS_REQUIRE(qblock_tokens == PREFILL_QBLOCK, "attn_prefill_bf16: query blocks of %d tokens, %d expected",
                qblock_tokens, PREFILL_QBLOCK);
    dim3 grid(n_qblocks, nheads);
    attn_prefill_bf16_kernel<16, 1, 8><<<grid, dim3(8 * WAVE), 0, stream>>>(
        (const bf16*)q, q_stride, (bf16*)out, out_stride, positions, seq_of_token, qblock_start, qblock_len,
        block_table, table_stride, (const bf16*)k_cache, (const bf16*)v_cache, nheads, kvheads, head_dim, scale, window);
    FMS_LAUNCH_CHECK("attn_prefill_bf16");
    return 0;
  }
  int hb, qt_unused, qblock_expected;
  prefill_shape(nheads, kvheads, head_dim, n_tokens, &hb, &qt_unused, &qblock_expected);
  FMS_REQUIRE(qblock_tokens == qblock_expected, "attn_prefill_bf16: query blocks of %d tokens, %d expected",
              qblock_tokens, qblock_expected);
  const long blocks = (long)n_qblocks * kvheads * (group / hb);
  FMS_REQUIRE(blocks < (1l << 31), "attn_prefill_bf16: %ld blocks exceed one launch", blocks);
  dim3 grid((unsigned)blocks);
#define FMS_PL(M)                                                                                                  \
  do {                                                                                                             \
  if (head_dim == M * 16)                                                                                          \
    attn_prefill_lds_kernel<M, LDS_QT, LDS_UNITS, true><<<grid, dim3(LDS_UNITS * 2 * WAVE), 0, stream>>>(          \
        (const bf16*)q, q_stride, (bf16*)out, out_stride, positions, seq_of_token, qblock_start, qblock_len,       \
        n_qblocks, block_table, table_stride, (const bf16*)k_cache, (const bf16*)v_cache, nheads, kvheads,         \
        head_dim, scale, window, hb);                                                                              \
  else                                                                                                             \
    attn_prefill_lds_kernel<M, LDS_QT, LDS_UNITS, false><<<grid, dim3(LDS_UNITS * 2 * WAVE), 0, stream>>>(         \
      (const bf16*)q, q_stride, (bf16*)out, out_stride, positions, seq_of_token, qblock_start, qblock_len,         \
      n_qblocks, block_table, table_stride, (const bf16*)k_cache, (const bf16*)v_cache, nheads, kvheads, head_dim, \
      scale, window, hb);                                                                                          \
  } while (0)
#define FMS_PL32(D32)                                                                                              \
  attn_prefill_lds32_kernel<D32, LDS_UNITS><<<grid, dim3(LDS_UNITS * 2 * WAVE), 0, stream>>>(                      \
      (const bf16*)q, q_stride, (bf16*)out, out_stride, positions, seq_of_token, qblock_start, qblock_len, n_qblocks, \
      block_table, table_stride, (const bf16*)k_cache, (const bf16*)v_cache, nheads, kvheads, scale, window, hb)
  if (head_dim == 128)  // head sizes with a 32x32x16 kernel of their own
    FMS_PL32(4);
  else if (head_dim == 64)
    FMS_PL32(2);
  else if (head_dim <= 64)
    FMS_PL(4);
  else
    FMS_PL(8);
#undef FMS_PL32
#undef FMS_PL
  FMS_LAUNCH_CHECK("attn_prefill_bf16");
  return 0;
}

extern "C" long fmsamd_attn_decode_workspace(int n_tokens, int nheads, int head_dim, int n_splits) {
  if (n_splits <= 1) return 0;
  return (long)n_tokens * nheads * n_splits * (head_dim + 2) * (long)sizeof(float);
}

extern "C" int fmsamd_attn_decode_bf16(const void* q, long q_stride, void* out, long out_stride, void* workspace,
                                       long workspace_bytes, const int* positions, const int* seq_of_token,
                                       const int* block_table, int table_stride, const void* k_cache,
                                       const void* v_cache, int n_tokens, int nheads, int kvheads, int head_dim,
                                       float scale, int window, int max_context, int pages_per_split, int waves,
                                       int staged, const int* row_order, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (check_common("attn_decode_bf16", n_tokens, nheads, kvheads, head_dim, q_stride, out_stride)) return -1;
  FMS_REQUIRE(head_dim % 16 == 0, "attn_decode_bf16: head size %d is no multiple of 16", head_dim);
  FMS_REQUIRE(q_stride % 8 == 0, "attn_decode_bf16: query row stride must keep 16-byte alignment");
  FMS_REQUIRE(pages_per_split > 0 && max_context > 0, "attn_decode_bf16: bad split sizes");
  FMS_REQUIRE(waves >= 1 && waves <= 8, "attn_decode_bf16: %d waves per block (1..8)", waves);
  if (head_dim > 128 && waves > 4) waves = 4;
  FMS_REQUIRE(n_tokens <= 65535, "attn_decode_bf16: %d tokens exceed one launch (65535)", n_tokens);
  const int n_splits = ceil_div(ceil_div(max_context, PAGE_TOKENS), pages_per_split);
  const long need = fmsamd_attn_decode_workspace(n_tokens, nheads, head_dim, n_splits);
  FMS_REQUIRE(workspace_bytes >= need, "attn_decode_bf16: workspace of %ld bytes, %ld needed", workspace_bytes, need);
  const int group = nheads / kvheads;
  // the merge buffer [waves][columns][head_dim + 2] must fit 64 KB of LDS
  int tile_cols = 16;
  while (tile_cols > 1 && (size_t)waves * tile_cols * (head_dim + 2) * sizeof(float) > 65536) tile_cols /= 2;
  const size_t lds_bytes = (size_t)waves * tile_cols * (head_dim + 2) * sizeof(float);
  FMS_REQUIRE(lds_bytes <= 65536, "attn_decode_bf16: %d waves need %zu bytes of LDS", waves, lds_bytes);
  const int tiles_per_kv = (group + tile_cols - 1) / tile_cols;
  FMS_REQUIRE((long)kvheads * tiles_per_kv <= 65535, "attn_decode_bf16: too many heads");
  float* part_o = (float*)workspace;
  float* part_ml = part_o ? part_o + (size_t)n_tokens * nheads * n_splits * head_dim : nullptr;
  dim3 grid(n_splits, kvheads * tiles_per_kv, n_tokens);
#define FMS_DC(M, MAXW, STAGED, LDS)                                                                                 \
  attn_decode_bf16_kernel<M, MAXW, STAGED><<<grid, dim3(waves * WAVE), LDS, stream>>>(                               \
      (const bf16*)q, q_stride, (bf16*)out, out_stride, part_o, part_ml, n_splits, positions, seq_of_token,          \
      block_table, table_stride, (const bf16*)k_cache, (const bf16*)v_cache, nheads, kvheads, head_dim, scale,       \
      window, tile_cols, row_order)
  FMS_REQUIRE(staged == 0 || head_dim == 128, "attn_decode_bf16: pages go through LDS for head size 128 only");
  if (staged != 0) {
    // the waves' results meet in the page buffers: 16 KB a wave hold 16 columns of 130 floats
    if (waves <= 4)
      FMS_DC(8, 4, true, 0);
    else
      FMS_DC(8, 8, true, 0);
  } else if (head_dim <= 64)
    FMS_DC(4, 8, false, lds_bytes);
  else if (head_dim <= 128)
    FMS_DC(8, 8, false, lds_bytes);
  else
    FMS_DC(16, 4, false, lds_bytes);  // large heads need the registers of a smaller block
#undef FMS_DC
  FMS_LAUNCH_CHECK("attn_decode_bf16");
  if (n_splits > 1) {
    dim3 mgrid(nheads, n_tokens);
    attn_decode_merge_kernel<<<mgrid, head_dim <= 64 ? 64 : 128, 0, stream>>>(part_o, part_ml, (bf16*)out, out_stride, nheads,
                                                                              head_dim, n_splits);
    FMS_LAUNCH_CHECK("attn_decode_merge");
  }
  return 0;
}
