// Rotary position encoding: the cos/sin table, and the fused kernel that
// rotates queries in place and writes rotated keys and the values into the
// paged cache.
//
// Cache layout of one layer (PAGE_TOKENS tokens per page):
//   keys    [page][kv head][token in page][head_dim]
//   values  [page][kv head][head_dim][token in page]      (transposed)
// so that both the score product (contraction over head_dim) and the mixing
// product (contraction over tokens) read their contraction index contiguously.
#include "common.h"
#include "fmsamd.h"

// cos/sin of position * freq, float32: angle = float(p) * f, as the reference
// builds its table (outer product of positions and frequencies, then cos/sin).
__global__ void rope_table_kernel(const float* __restrict__ freqs, float* __restrict__ cos_t, float* __restrict__ sin_t,
                                  int max_pos, int half) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= max_pos * half) return;
  const int p = idx / half, i = idx % half;
  const float angle = (float)p * freqs[i];
  cos_t[idx] = cosf(angle);
  sin_t[idx] = sinf(angle);
}

extern "C" int fmsamd_rope_table(const float* freqs, float* cos_t, float* sin_t, int max_pos, int half,
                                 hipStream_t stream) {
  FMS_REQUIRE(max_pos > 0 && half > 0, "rope_table: bad sizes max_pos=%d half=%d", max_pos, half);
  FMS_REQUIRE((long)max_pos * half < (1L << 31), "rope_table: table too large");
  rope_table_kernel<<<ceil_div((long)max_pos * half, 256), 256, 0, stream>>>(freqs, cos_t, sin_t, max_pos, half);
  FMS_LAUNCH_CHECK("rope_table");
  return 0;
}

// One block per token, a pair of elements a thread: for any even head size and any alignment.
// qkv row = [H*D queries | K*D keys | K*D values].
template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, long row_stride, const int* __restrict__ positions,
                                     const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
                                     int table_stride, const float* __restrict__ cos_t,
                                     const float* __restrict__ sin_t, int rot_dim, int max_pos, T* __restrict__ k_cache,
                                     T* __restrict__ v_cache, int nheads, int kvheads, int head_dim) {
  const int t = blockIdx.x;
  const int seq = seq_of_token[t];
  if (seq < 0) return;  // padding row of a fixed-size batch
  int pos = positions[t];
  const int tpos = pos < 0 ? 0 : (pos < max_pos ? pos : max_pos - 1);  // the host has checked; never read outside the table
  const int half = head_dim / 2;
  const int rot_half = rot_dim / 2;
  T* row = qkv + (size_t)t * row_stride;

  long page = 0;
  int in_page = pos % PAGE_TOKENS;
  if (k_cache) {
    page = block_table[(size_t)seq * table_stride + pos / PAGE_TOKENS];
    if (page < 0) k_cache = nullptr, v_cache = nullptr;  // no page for this token: queries only
  }
  const size_t page_elems = (size_t)kvheads * PAGE_TOKENS * head_dim;

  const int total = (nheads + 2 * kvheads) * half;
  for (int idx = threadIdx.x; idx < total; idx += blockDim.x) {
    const int hh = idx / half;
    const int i = idx % half;
    T* p = row + (size_t)hh * head_dim + 2 * i;
    float a = to_f32(p[0]), b = to_f32(p[1]);
    if (hh < nheads + kvheads) {
      if (cos_t && i < rot_half) {
        const float c = cos_t[(size_t)tpos * rot_half + i];
        const float s = sin_t[(size_t)tpos * rot_half + i];
        const float ra = c * a - s * b;
        const float rb = s * a + c * b;
        a = ra;
        b = rb;
      }
      if (hh < nheads) {
        p[0] = from_f32<T>(a);
        p[1] = from_f32<T>(b);
      } else if (k_cache) {
        const int kh = hh - nheads;
        T* dst = k_cache + page * page_elems + ((size_t)kh * PAGE_TOKENS + in_page) * head_dim + 2 * i;
        dst[0] = from_f32<T>(a);
        dst[1] = from_f32<T>(b);
      }
    } else if (v_cache) {
      const int kh = hh - nheads - kvheads;
      T* dst = v_cache + page * page_elems + ((size_t)kh * head_dim + 2 * i) * PAGE_TOKENS + in_page;
      dst[0] = from_f32<T>(a);
      dst[PAGE_TOKENS] = from_f32<T>(b);
    }
  }
}

// The same for many tokens: a block takes RT consecutive token rows and one head (a query head, a key head or
// a value head), 16 bytes a thread and step where rows allow it (QV = 8 bfloat16 or 4 float32 elements, with
// their cosines and sines as 16-byte loads too; QV = 4 for bfloat16 rows that only allow 8 bytes).  Rows of q and
// k stay rows; the values of a head are turned over in LDS, so that the lanes of a store are neighbouring tokens
// of one row of the transposed page (tokens that follow one another in a sequence are neighbours there) instead
// of 2-byte writes 128 bytes apart.
template <typename T, int N>
struct VecOf {
  typedef T type __attribute__((ext_vector_type(N)));
};

template <typename T, int QV>
__global__ void __launch_bounds__(256)
    rope_kv_tile_kernel(T* __restrict__ qkv, long row_stride, const int* __restrict__ positions,
                        const int* __restrict__ seq_of_token, const int* __restrict__ block_table, int table_stride,
                        const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot_dim, int max_pos,
                        T* __restrict__ k_cache, T* __restrict__ v_cache, int nheads, int kvheads, int head_dim,
                        int n_tokens) {
  constexpr int RT = sizeof(T) == 4 ? 32 : 64;
  typedef typename VecOf<T, 4>::type vec4;
  typedef typename VecOf<T, QV>::type vecq;
  extern __shared__ __attribute__((aligned(16))) unsigned char tile_raw[];  // value heads: RT x (head_dim + 4)
  __shared__ int s_pos[RT];
  __shared__ long long s_page[RT];  // -1: the row is padding or past the end
  const int t0 = blockIdx.x * RT;
  const int hh = blockIdx.y;
  if (hh >= nheads && k_cache == nullptr) return;  // queries only
  if (threadIdx.x < RT) {
    const int t = t0 + threadIdx.x;
    int pos = 0;
    long long page = -1;
    if (t < n_tokens) {
      const int seq = seq_of_token[t];
      if (seq >= 0) {
        pos = positions[t];
        page = k_cache ? block_table[(size_t)seq * table_stride + pos / PAGE_TOKENS] : 0;
      }
    }
    s_pos[threadIdx.x] = pos;
    s_page[threadIdx.x] = page;
  }
  __syncthreads();
  const int quads = head_dim / 4;
  const int rot_half = rot_dim / 2;
  const size_t page_elems = (size_t)kvheads * PAGE_TOKENS * head_dim;

  if (hh < nheads + kvheads) {
    const int per_row = head_dim / QV;  // the host has checked that QV divides the head size
    for (int idx = threadIdx.x; idx < RT * per_row; idx += blockDim.x) {
      const int tok = idx / per_row, qd = idx - tok * per_row;
      if (s_page[tok] < 0) continue;
      const int pos = s_pos[tok];
      T* p = qkv + (size_t)(t0 + tok) * row_stride + (size_t)hh * head_dim + QV * qd;
      vecq v = *reinterpret_cast<const vecq*>(p);
      if (cos_t != nullptr) {
        const int tpos = pos < 0 ? 0 : (pos < max_pos ? pos : max_pos - 1);  // the host has checked; never read outside the table
        const int i0 = (QV / 2) * qd;  // the first pair (x[2i], x[2i+1]) of this piece
        float c[QV / 2], sn[QV / 2];
        if (QV == 8 && i0 + 4 <= rot_half && rot_half % 4 == 0) {  // four angles: 16 bytes each of cosines and sines
          const f32x4 c4 = *reinterpret_cast<const f32x4*>(cos_t + (size_t)tpos * rot_half + i0);
          const f32x4 s4 = *reinterpret_cast<const f32x4*>(sin_t + (size_t)tpos * rot_half + i0);
#pragma unroll
          for (int j = 0; j < QV / 2; ++j) c[j] = c4[j & 3], sn[j] = s4[j & 3];
        } else {
#pragma unroll
          for (int j = 0; j < QV / 2; ++j) {
            const bool rotates = i0 + j < rot_half;
            c[j] = rotates ? cos_t[(size_t)tpos * rot_half + i0 + j] : 1.f;
            sn[j] = rotates ? sin_t[(size_t)tpos * rot_half + i0 + j] : 0.f;
          }
        }
#pragma unroll
        for (int j = 0; j < QV / 2; ++j) {
          if (i0 + j < rot_half) {
            const float a = to_f32(v[2 * j]), b = to_f32(v[2 * j + 1]);
            v[2 * j] = from_f32<T>(c[j] * a - sn[j] * b);
            v[2 * j + 1] = from_f32<T>(sn[j] * a + c[j] * b);
          }
        }
      }
      if (hh < nheads) {
        *reinterpret_cast<vecq*>(p) = v;
      } else {
        const int kh = hh - nheads;
        T* dst = k_cache + (size_t)s_page[tok] * page_elems + ((size_t)kh * PAGE_TOKENS + pos % PAGE_TOKENS) * head_dim + QV * qd;
        *reinterpret_cast<vecq*>(dst) = v;
      }
    }
    return;
  }

  T* tile = reinterpret_cast<T*>(tile_raw);
  const int ld = head_dim + 4;
  for (int idx = threadIdx.x; idx < RT * quads; idx += blockDim.x) {
    const int tok = idx / quads, qd = idx - tok * quads;
    if (s_page[tok] < 0) continue;
    *reinterpret_cast<vec4*>(tile + tok * ld + 4 * qd) =
        *reinterpret_cast<const vec4*>(qkv + (size_t)(t0 + tok) * row_stride + (size_t)hh * head_dim + 4 * qd);
  }
  // TG tokens make 16 bytes of a row of the transposed page.  Where the TG tokens of a group follow one another
  // in one page, from a place that is a multiple of TG (a prompt's tokens do), they leave as one 16-byte store,
  // and the lanes of a wave fill whole rows of the page; other groups go element by element.
  constexpr int TG = (QV == 8 || sizeof(T) == 4) ? 16 / (int)sizeof(T) : 1;
  __shared__ int s_together[RT];
  if (TG > 1 && threadIdx.x < RT / TG) {
    const int tok0 = threadIdx.x * TG;
    bool together = s_page[tok0] >= 0 && (s_pos[tok0] % PAGE_TOKENS) % TG == 0;
    for (int j = 1; j < TG; ++j) together = together && s_page[tok0 + j] == s_page[tok0] && s_pos[tok0 + j] == s_pos[tok0] + j;
    s_together[threadIdx.x] = together ? 1 : 0;
  }
  __syncthreads();
  const int kh = hh - nheads - kvheads;
  if constexpr (TG > 1) {
    typedef typename VecOf<T, TG>::type vecg;
    constexpr int GROUPS = RT / TG;
    for (int idx = threadIdx.x; idx < GROUPS * head_dim; idx += blockDim.x) {
      const int tg = idx % GROUPS, d = idx / GROUPS;  // neighbouring lanes: neighbouring pieces of a row
      const int tok0 = tg * TG;
      if (s_together[tg]) {
        vecg v;
#pragma unroll
        for (int j = 0; j < TG; ++j) v[j] = tile[(tok0 + j) * ld + d];
        *reinterpret_cast<vecg*>(v_cache + (size_t)s_page[tok0] * page_elems + ((size_t)kh * head_dim + d) * PAGE_TOKENS +
                                 s_pos[tok0] % PAGE_TOKENS) = v;
      } else {
#pragma unroll
        for (int j = 0; j < TG; ++j) {
          const int tok = tok0 + j;
          if (s_page[tok] >= 0)
            v_cache[(size_t)s_page[tok] * page_elems + ((size_t)kh * head_dim + d) * PAGE_TOKENS + s_pos[tok] % PAGE_TOKENS] =
                tile[tok * ld + d];
        }
      }
    }
    return;
  }
  for (int idx = threadIdx.x; idx < RT * head_dim; idx += blockDim.x) {
    const int tok = idx % RT, d = idx / RT;  // neighbouring lanes: neighbouring tokens
    if (s_page[tok] < 0) continue;
    v_cache[(size_t)s_page[tok] * page_elems + ((size_t)kh * head_dim + d) * PAGE_TOKENS + s_pos[tok] % PAGE_TOKENS] = tile[tok * ld + d];
  }
}

extern "C" int fmsamd_rope_kv_write(void* qkv, int dtype, long row_stride, const int* positions,
                                    const int* seq_of_token, const int* block_table, int table_stride,
                                    const float* cos_t, const float* sin_t, int rot_dim, int max_pos, void* k_cache,
                                    void* v_cache, int n_tokens, int nheads, int kvheads, int head_dim,
                                    hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && nheads > 0 && kvheads > 0 && head_dim > 0, "rope_kv_write: bad sizes");
  FMS_REQUIRE(head_dim % 2 == 0, "rope_kv_write: head size %d is odd", head_dim);
  FMS_REQUIRE(rot_dim % 2 == 0 && rot_dim >= 0 && rot_dim <= head_dim, "rope_kv_write: rotary size %d does not fit head size %d",
              rot_dim, head_dim);
  FMS_REQUIRE(row_stride >= (long)(nheads + 2 * kvheads) * head_dim, "rope_kv_write: row stride too small");
  FMS_REQUIRE((k_cache == nullptr) == (v_cache == nullptr), "rope_kv_write: key and value cache must come together");
  FMS_REQUIRE(cos_t == nullptr || max_pos > 0, "rope_kv_write: empty table");
  const int threads = 256;
  const float* c = rot_dim > 0 ? cos_t : nullptr;
  const size_t elem = dtype == FMS_F32 ? 4 : 2;
  FMS_REQUIRE(dtype == FMS_F32 || dtype == FMS_BF16, "rope_kv_write: unknown dtype %d", dtype);
  // four elements a thread need rows that start at multiples of four elements
  const bool by_fours = head_dim % 4 == 0 && row_stride % 4 == 0 && (uintptr_t)qkv % (4 * elem) == 0 &&
                        (uintptr_t)k_cache % (4 * elem) == 0 && (uintptr_t)v_cache % (4 * elem) == 0;
  if (by_fours) {
    const int rt = dtype == FMS_F32 ? 32 : 64;
    FMS_REQUIRE(nheads + 2 * kvheads <= 65535, "rope_kv_write: too many heads");
    dim3 grid(ceil_div(n_tokens, rt), nheads + 2 * kvheads);
    const size_t lds = (size_t)rt * (head_dim + 4) * elem;
    // bfloat16 rows of q and k by eights (16 bytes) where heads, rows, tables and caches start at multiples of 16 bytes
    const bool by_eights = dtype == FMS_BF16 && head_dim % 8 == 0 && row_stride % 8 == 0 && (uintptr_t)qkv % 16 == 0 &&
                           (uintptr_t)k_cache % 16 == 0 && (uintptr_t)v_cache % 16 == 0 && (uintptr_t)cos_t % 16 == 0 &&
                           (uintptr_t)sin_t % 16 == 0;
    if (dtype == FMS_F32)
      rope_kv_tile_kernel<float, 4><<<grid, threads, lds, stream>>>(
          (float*)qkv, row_stride, positions, seq_of_token, block_table, table_stride, c, sin_t, rot_dim, max_pos,
          (float*)k_cache, (float*)v_cache, nheads, kvheads, head_dim, n_tokens);
    else if (by_eights)
      rope_kv_tile_kernel<bf16, 8><<<grid, threads, lds, stream>>>(
          (bf16*)qkv, row_stride, positions, seq_of_token, block_table, table_stride, c, sin_t, rot_dim, max_pos,
          (bf16*)k_cache, (bf16*)v_cache, nheads, kvheads, head_dim, n_tokens);
    else
      rope_kv_tile_kernel<bf16, 4><<<grid, threads, lds, stream>>>(
          (bf16*)qkv, row_stride, positions, seq_of_token, block_table, table_stride, c, sin_t, rot_dim, max_pos,
          (bf16*)k_cache, (bf16*)v_cache, nheads, kvheads, head_dim, n_tokens);
  } else if (dtype == FMS_F32)
    rope_kv_write_kernel<float><<<n_tokens, threads, 0, stream>>>(
        (float*)qkv, row_stride, positions, seq_of_token, block_table, table_stride, c, sin_t, rot_dim, max_pos,
        (float*)k_cache, (float*)v_cache, nheads, kvheads, head_dim);
  else
    rope_kv_write_kernel<bf16><<<n_tokens, threads, 0, stream>>>(
        (bf16*)qkv, row_stride, positions, seq_of_token, block_table, table_stride, c, sin_t, rot_dim, max_pos,
        (bf16*)k_cache, (bf16*)v_cache, nheads, kvheads, head_dim);
  FMS_LAUNCH_CHECK("rope_kv_write");
  return 0;
}
