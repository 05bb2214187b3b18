// C interface of the gfx950 kernel library.  Every function takes device
// pointers and a HIP stream, checks its arguments on the host, launches
// asynchronously, and returns 0 or a negative code; fmsamd_last_error()
// then holds the reason.  Nothing here allocates device memory.
#pragma once

#include <hip/hip_runtime.h>

#define FMSAMD_ABI_VERSION 2

// element types
#define FMS_F32 0
#define FMS_BF16 1

// activations of the gated feed-forward
#define FMS_ACT_SILU 0
#define FMS_ACT_GELU 1       // with the error function
#define FMS_ACT_RELU 2
#define FMS_ACT_IDENTITY 3
#define FMS_ACT_SIGMOID 4
#define FMS_ACT_TANH 5
#define FMS_ACT_MISH 6       // x tanh(log(1 + e^x))
#define FMS_ACT_GELU_TANH 7  // the tanh approximation
#define FMS_ACT_LAST FMS_ACT_GELU_TANH

#ifdef __cplusplus
extern "C" {
#endif

const char* fmsamd_last_error();
int fmsamd_abi_version();

// resid[t, :] = float(table[ids[t], :])
int fmsamd_embed(const int* ids, const void* table, int table_dtype, float* out, int n_tokens, int width, int vocab,
                 hipStream_t stream);

// resid += branch (float32 sum, written back unless `rows` is given); out = norm(resid) * weight + bias.
// branch, weight, bias and rows may be null.  act_dtype is the type of branch and out.
int fmsamd_add_norm(float* resid, const void* branch, int act_dtype, const void* weight, const void* bias,
                    int weight_dtype, void* out, const int* rows, int n_out, int width, float eps, int use_mean,
                    hipStream_t stream);

// out[t, j] = act(gu[t, j] + b[j]) * (gu[t, hidden + j] + b[hidden + j])
int fmsamd_gated_act(const void* gu, const void* bias, int bias_dtype, void* out, int dtype, int n_tokens, int hidden,
                     int act, hipStream_t stream);

// positions[i] += 1 where seq_of_token[i] >= 0
int fmsamd_advance_positions(int* positions, const int* seq_of_token, int n, hipStream_t stream);

int fmsamd_cast(const void* in, int in_dtype, void* out, int out_dtype, long n, hipStream_t stream);
int fmsamd_bias_add(void* x, int dtype, const void* bias, int bias_dtype, int rows, int cols, hipStream_t stream);

// cos/sin of position * freqs[i], float32, [max_pos, half]
int fmsamd_rope_table(const float* freqs, float* cos_t, float* sin_t, int max_pos, int half, hipStream_t stream);

// Rotate the queries of qkv in place; rotate the keys and write keys and values into the paged cache
// (k_cache/v_cache null: queries only).  cos_t null: no rotation.
int fmsamd_rope_kv_write(void* qkv, int dtype, long row_stride, const int* positions, const int* seq_of_token,
                         const int* block_table, int table_stride, const float* cos_t, const float* sin_t,
                         int rot_dim, int max_pos, void* k_cache, void* v_cache, int n_tokens, int nheads, int kvheads,
                         int head_dim, hipStream_t stream);

// causal attention over the cache; any element type, any even head size up to 256.  Further terms of the scores:
// slopes (float32 [nheads] or null): score += slopes[head] * (key position - query position); soft_cap (0: none):
// score = soft_cap * tanh(score / soft_cap), before the slope term.
int fmsamd_attn_generic(const void* q, long q_stride, void* out, long out_stride, int dtype, const int* positions,
                        const int* seq_of_token, const int* block_table, int table_stride, const void* k_cache,
                        const void* v_cache, int n_tokens, int nheads, int kvheads, int head_dim, float scale,
                        int window, const float* slopes, float soft_cap, hipStream_t stream);

// bfloat16 prefill: the step is cut into query blocks of at most fmsamd_attn_prefill_qblock(...) consecutive
// tokens of one sequence; the same number goes into the call as qblock_tokens
int fmsamd_attn_prefill_qblock(int nheads, int kvheads, int head_dim, int n_tokens);
int fmsamd_attn_prefill_bf16(const void* q, long q_stride, void* out, long out_stride, const int* positions,
                             const int* seq_of_token, const int* qblock_start, const int* qblock_len, int n_qblocks,
                             int qblock_tokens, const int* block_table, int table_stride, const void* k_cache, const void* v_cache,
                             int n_tokens, int nheads, int kvheads, int head_dim, float scale, int window,
                             hipStream_t stream);

// bfloat16 decode: one token per sequence.  The context bound max_context is cut into splits of
// `pages_per_split` pages, and every sequence deals its own pages out evenly over that many blocks of `waves`
// waves (which take them in turn and merge in LDS); with more than one split a second kernel merges the
// partial results.  staged != 0 (head size 128 only): pages are loaded in contiguous kilobytes and turned into
// the MFMA layout in LDS, which streams faster when there is much to read.  row_order (or null): the token rows in
// the order in which the blocks are to take them, e.g. longest context first; the result does not depend on it.
long fmsamd_attn_decode_workspace(int n_tokens, int nheads, int head_dim, int n_splits);
int fmsamd_attn_decode_bf16(const void* q, long q_stride, void* out, long out_stride, void* workspace,
                            long workspace_bytes, const int* positions, const int* seq_of_token,
                            const int* block_table, int table_stride, const void* k_cache, const void* v_cache,
                            int n_tokens, int nheads, int kvheads, int head_dim, float scale, int window,
                            int max_context, int pages_per_split, int waves, int staged, const int* row_order,
                            hipStream_t stream);

// c[M, N] = a[M, K] w[N, K]^T (+ bias[N])
int fmsamd_gemm_f32(const float* a, long lda, const float* w, const float* bias, float* c, long ldc, int M, int N,
                    int K, hipStream_t stream);
int fmsamd_gemm_bf16(const void* a, long lda, const void* w, const void* bias, int bias_dtype, void* c, int out_dtype,
                     long ldc, int M, int N, int K, hipStream_t stream);
// The same product for any K and any row stride (the MFMA kernels need multiples of 8): element loads and
// float32 FMA.  Slow; it exists so that no width a configuration allows is refused.
int fmsamd_gemm_bf16_any(const void* a, long lda, const void* w, const void* bias, int bias_dtype, void* c,
                         int out_dtype, long ldc, int M, int N, int K, hipStream_t stream);
// A row norm left to the product that reads the rows: the rows hold stream * norm weight, and the sums of
// squares of the stream come as `count` partial sums per row (partials[m * count + i]).  The product is
// multiplied by rsqrt(sum / K + eps) of its row before the bias.  A null pointer (or null partials): none.
typedef struct {
  const float* partials;
  int count;
  float eps;
} fmsamd_row_scale;

// At most 192 rows: the weights stream once through MFMA registers.  From 17 rows on the product needs a
// workspace of fmsamd_gemm_skinny_workspace(M, rows of W, K) bytes (slices of K meet there).
long fmsamd_gemm_skinny_workspace(int M, int rows, int K);
int fmsamd_gemm_skinny_bf16(const void* x, long ldx, const void* w, const void* bias, int bias_dtype, void* out,
                            int out_dtype, long ldo, int M, int N, int K, const fmsamd_row_scale* row_scale,
                            void* workspace, long workspace_bytes, hipStream_t stream);
int fmsamd_gemm_skinny_gated_bf16(const void* x, long ldx, const void* w, const void* bias, int bias_dtype, void* out,
                                  int out_dtype, long ldo, int M, int hidden, int K, int act,
                                  const fmsamd_row_scale* row_scale, void* workspace, long workspace_bytes,
                                  hipStream_t stream);
// resid += x W^T (+ bias) in float32; scaled = resid * norm_w in bfloat16; partials[M, partial_count] = sums
// of squares of resid by groups of columns (partial_count as fmsamd_gemm_skinny_residual_partials(M, N, K) says;
// every entry is written).  At most 192 rows.
int fmsamd_gemm_skinny_residual_partials(int M, int N, int K);
int fmsamd_gemm_skinny_residual_bf16(const void* x, long ldx, const void* w, const void* bias, int bias_dtype,
                                     float* resid, long ldr, const void* norm_w, int norm_w_dtype, void* scaled,
                                     long ldo, float* partials, int partial_count, int M, int N, int K,
                                     const fmsamd_row_scale* row_scale, void* workspace, long workspace_bytes,
                                     hipStream_t stream);

// qkv = x W^T (+ bias) for at most 192 rows with the rotation and the cache write fused into the epilogue;
// only the query columns of `out` are written
int fmsamd_qkv_rope_skinny_bf16(const void* x, long ldx, const void* w, const void* bias, int bias_dtype, void* out,
                                long ldo, int M, int K, const int* positions, const int* seq_of_token,
                                const int* block_table, int table_stride, const float* cos_t, const float* sin_t,
                                int rot_dim, int max_pos, void* k_cache, void* v_cache, int nheads, int kvheads,
                                int head_dim, const fmsamd_row_scale* row_scale, void* workspace, long workspace_bytes,
                                hipStream_t stream);

// token choice; rng_state is [rows][2] uint64 (seed, counter), advanced by the kernel
int fmsamd_sample(const float* logits, long ld, int rows, int vocab, int do_sample, float temperature, int top_k,
                  void* rng_state, int* out_tokens, hipStream_t stream);

// greedy choice over many blocks per row; workspace of fmsamd_argmax_workspace(rows, vocab) bytes
long fmsamd_argmax_workspace(int rows, int vocab);
int fmsamd_argmax(const float* logits, long ld, int rows, int vocab, void* workspace, long workspace_bytes,
                  int* out_tokens, hipStream_t stream);

// The greedy choice of fmsamd_argmax without a workspace, for callers that cannot allocate device memory:
// code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart
// in the reference.  The partial results of the first stage go to an array of FMSAMD_ARGMAX_STATIC_BYTES
// that the library holds on every GPU it runs on until the process ends; rows * ceil(vocab / 2048) * 8 bytes
// must fit (32768 partial results: 256 rows of a vocabulary of 262144, 1024 rows of one of 65536), larger
// inputs are refused.  The call allocates nothing and frees nothing.  All calls on one GPU share that GPU's
// array: calls that overlap in time on one GPU (two streams, two threads) race; calls on one stream do not.
// The first call on a device looks the array's address up (hipGetSymbolAddress), so make it outside a capture.
#define FMSAMD_ARGMAX_STATIC_BYTES (256 * 1024)
int fmsamd_argmax_static(const float* logits, long ld, int rows, int vocab, int* out_tokens, hipStream_t stream);

// Measurements of the GPU itself, for a benchmark's "of the measured peak": a pure read of `bytes` bytes by
// `blocks` blocks, and blocks x 4 waves x iterations x 8 matrix instructions on registers (*flops: how many
// floating-point operations that is).  `out` is a float on the device that may be written.
// contiguous: every block reads one stretch of the buffer instead of the grid sweeping it together; large: 32x32x16
// products instead of 16x16x32.
int fmsamd_probe_read(const void* buffer, long bytes, int blocks, int contiguous, float* out, hipStream_t stream);
int fmsamd_probe_mfma(int blocks, int iterations, int large, float* out, double* flops, hipStream_t stream);

#ifdef __cplusplus
}
#endif
