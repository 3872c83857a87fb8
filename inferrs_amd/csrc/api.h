// C entry points of the kernel library.  Every function takes device pointers and a HIP
// stream, launches asynchronously on it, returns 0 on success and a non-zero code after
// leaving a message for ia_last_error().  dtype arguments: 0 = float32, 1 = bfloat16.
#pragma once

#include <hip/hip_runtime.h>

#define IA_ABI_VERSION 1

#ifdef __cplusplus
extern "C" {
#endif

const char* ia_last_error(void);
int ia_abi_version(void);

int ia_embed_gather(void* out, const void* table, const int* ids, int n, int hidden, int vocab,
                    int dtype, hipStream_t stream);
int ia_gather_rows(void* out, const void* x, const int* rows, int n, int cols, int dtype,
                   hipStream_t stream);
int ia_rmsnorm(void* out, const void* x, const float* w, float eps, int rows, int cols,
               int add_one, int dtype, hipStream_t stream);
int ia_add_rmsnorm(void* out, void* x, const void* delta, const float* w, float eps, int rows,
                   int cols, int add_one, int dtype, hipStream_t stream);
int ia_add_inplace(void* x, const void* delta, long long n, int dtype, hipStream_t stream);
int ia_fill_normal(void* out, long long n, unsigned long long seed, double mean, double std,
                   int dtype, hipStream_t stream);
int ia_widen_bf16(float* out, const void* x, long long n, hipStream_t stream);
// rows of [gate | up] -> act(gate) * up; act: 1 SiLU, 2 GELU in its tanh form (the same numbers name the activation
// in the `dual` argument of the products below, where 0 means a plain product)
int ia_gate_mul(void* out, const void* gu, int rows, int inter, int act, int dtype, hipStream_t stream);
// x[row][c] += bias[c] in place (x and bias in the same precision)
int ia_add_bias(void* x, const void* bias, int rows, int cols, int dtype, hipStream_t stream);
// A pure streaming read of `bytes` bytes by `blocks` blocks (one word of `out` a block): the measurement script's
// measured memory roof.  Nothing of the engine calls it.
int ia_stream_read(unsigned* out, const void* x, long long bytes, int blocks, hipStream_t stream);
int ia_rope_table(float* cos_out, float* sin_out, const int* positions, const float* inv_freq,
                  int n, int half, hipStream_t stream);

int ia_qk_rope_kv(void* q_out, void* k_cache, void* v_cache, const void* qkv,
                  const float* q_norm_w, const float* k_norm_w, const float* cos_t,
                  const float* sin_t, const int* slots, int n, int nq, int nkv, int d, int rot,
                  int interleaved, int page_size, float eps, int add_one, int dtype,
                  hipStream_t stream);

// workspace: null, or ia_attention_generic_workspace(...) floats when that is not 0 (steps of few tokens: a wave a
// segment of keys and a merge kernel, the same bits as without); max_kv_len: an upper bound of positions + 1
int ia_attention_generic(void* out, const void* q, const void* k_cache, const void* v_cache,
                         const int* positions, const int* token_seq, const int* block_table,
                         int n, int max_pages, int nq, int nkv, int d, int page_size, int window,
                         float scale, int dtype, float* workspace, int max_kv_len, hipStream_t stream);
long long ia_attention_generic_workspace(int n, int nq, int nkv, int d, int max_kv_len);

int ia_gemm_tiled(void* out, const void* x, const void* w, int M, int N, int K, int in_dtype,
                  int out_dtype, hipStream_t stream);
// bias: bfloat16 [N] ([2 N] with dual), or null
// (ia_gemm_tiled at up to 64 rows: the shape of its kernel for few rows, 100 * output features + staged rows a wave:
// 816, 808, 416 or 1608; 0: the kernel's own rule)
int ia_gemm_rows_tune(int shape);
int ia_gemm_skinny_bf16(void* out, const void* x, const void* w, const void* bias, int M, int N, int K,
                        int out_dtype, int dual, hipStream_t stream);
// Large bfloat16 products through the vendor's library, hipBLASLt, called directly (vendor_gemm.hip).  ia_vendor_gemm_init
// opens the library at `path` (the copy the process already holds) once; ia_vendor_gemm_bf16: out [M, N] = x [M, K] . w [N, K]^T,
// contiguous, with `workspace_bytes` of device memory for kernels that want some.
#define IA_VENDOR_NO_KERNEL 2     // ia_vendor_gemm_bf16: the library's search names no kernel for this shape
int ia_vendor_gemm_init(const char* path);
int ia_vendor_gemm_ready(void);
int ia_vendor_gemm_bf16(void* out, const void* x, const void* w, int M, int N, int K, void* workspace,
                        long long workspace_bytes, hipStream_t stream);
// Large bfloat16 products in tiles of 256 x 256 (gemm_mfma.hip); K a multiple of 64; with `dual` w is [gate; up]
// and out = act(x . gate^T) * (x . up^T).
int ia_gemm_mfma_bf16(void* out, const void* x, const void* w, int M, int N, int K, int dual, hipStream_t stream);
// Tuning knobs of the skinny product (tests switch the staged variants off with stage = 0); the defaults are
// (2048, 8, 5, 8, 1).
void ia_gemm_skinny_tune(int target_waves, int min_ksteps, int rot_mul, int min_waves, int stage);
// The skinny product with a residual stream around it (decode steps; see gemm.hip): adds itself to `resid`
// and leaves the rows' sums of squares and the rows times the next norm's weight, and / or takes such rows
// and finishes their norm.
// (the sums of squares come block by block: ia_gemm_skinny_blocks(N) blocks of ia_gemm_skinny_block_rows(N)
// neighbouring features each, a choice that depends on N and on the chip's number of compute units)
int ia_gemm_skinny_blocks(int N);
int ia_gemm_skinny_block_rows(int N);
int ia_gemm_skinny_stream(void* out, const void* x, const void* w, const void* bias, int M, int N, int K, int out_dtype,
                          int dual, void* resid, float* sums_out, void* scaled_out, const float* next_w,
                          int add_one, const float* sums_in, int n_sums, float eps, hipStream_t stream);

// Products of 17 to 128 bfloat16 rows (gemm_mid.hip); K a multiple of 128.  out_mode 0: out [M, N] bfloat16; 1: float;
// 2: out [ia_gemm_mid_splits(N, K)][M][N] float, the sums of each split of k, to be added up by the reader
// (ia_sum_partials, ia_add_rmsnorm_partials).  dual: w = [gate; up], out = act(x . gate^T) * (x . up^T), mode 0.
int ia_gemm_mid_splits(int N, int K);
// whether the weight's blocks fill the chip evenly, one a compute unit (dual: [gate; up] of N features each)
int ia_gemm_mid_fills(int N, int K, int dual);
// (a fixed pipeline for measurements and tests: k steps of a chunk, 2 or 4, and stages, 2 to 4; (0, 0): the kernel's own
// rule; no product depends on it bit for bit); anything else is an error and changes nothing
int ia_gemm_mid_tune(int kc, int ns);
// (how a block's waves share its products, for measurements and tests: 0 the kernel's own rule, 1 a tile of weight rows a
// wave over all rows of the step, 2 two tiles a wave over half of the rows wherever the shape allows; the same bits)
int ia_gemm_mid_blocking(int how);
// (a fixed shape of the blocks for measurements and tests: waves a block, 2 to 8 (0: the kernel's own rule), ways k is split
// and stages, 2 or 3 (2: four waves only); the caller's partial sums must have as many splits); a shape that has no
// kernel is an error and changes nothing
int ia_gemm_mid_plan(int waves, int splits, int stages);
int ia_gemm_mid_bf16(void* out, const void* x, const void* w, int M, int N, int K, int out_mode, int dual,
                     hipStream_t stream);
// the same for up to 16 rows that are a norm's input times its weight, with their sums of squares sums_in [M][n_sums]: every sum
// of the product is multiplied by the row's rsqrt(sum of sums_in / K + eps); out_mode 0 or 1
int ia_gemm_mid_bf16_scaled(void* out, const void* x, const void* w, int M, int N, int K, int out_mode, int dual,
                            const float* sums_in, int n_sums, float eps, hipStream_t stream);
int ia_sum_partials(void* out, const float* part, int splits, int M, int N, hipStream_t stream);
// x += (sum of the splits, rounded to bfloat16) in place, out = rmsnorm(x) * w; bfloat16 rows of up to 8192 features.
int ia_add_rmsnorm_partials(void* out, void* x, const float* part, int splits, const float* w, float eps,
                            int rows, int cols, int add_one, hipStream_t stream);

long long ia_argmax_workspace(int rows, int vocab);
int ia_argmax(int* out, const float* logits, void* workspace, int rows, int vocab, hipStream_t stream);
// The arg max without any allocation.  It has no counterpart in the reference; it is for callers that cannot
// allocate device memory: code under HIP graph capture, tight serving loops, harnesses that forbid it.  The
// two-step kernels' candidates go to an array of ia_argmax_static_capacity() 32-bit words (64 KiB) that the
// library holds in each GPU's memory until the process ends, instead of a workspace of the caller's; sizes for
// which ia_argmax_workspace(rows, vocab) exceeds that are refused with an error (about 430 rows at a
// vocabulary of 152 k).  No hipMalloc, hipFree or allocating library call happens inside.  All calls on one GPU
// share that GPU's array: calls that overlap on one GPU (two streams, two threads) race; calls on one stream do not.
long long ia_argmax_static_capacity(void);
int ia_argmax_static(int* out, const float* logits, int rows, int vocab, hipStream_t stream);
int ia_penalize(float* logits, int rows, int vocab, const int* window, int w, const float* rep,
                const float* freq, const float* pres, const int* bias_ids, const float* bias_vals,
                int nb, hipStream_t stream);
int ia_window_push(int* window, int rows, int w, const int* caps, const int* tokens, hipStream_t stream);
long long ia_sample_workspace(int rows, int vocab);
int ia_sample_max_top(void);
// n_top, lp_out [rows, 1 + max_top], lp_ids [rows, max_top]: all null, or the log-probabilities asked for per row
int ia_sample(int* out, const float* logits, void* workspace, int rows, int vocab,
              const float* temperature, const int* top_k, const float* top_p, const float* min_p,
              const float* u, const int* n_top, float* lp_out, int* lp_ids, hipStream_t stream);

// Built per head size (-DIA_HEAD_DIM) into a library of its own.
int ia_attention_mfma_head_dim(void);
long long ia_attention_mfma_workspace(int n, int nq, int splits);
int ia_attention_mfma(void* out, float* workspace, const void* q, const void* k_cache,
                      const void* v_cache, const int* block_table, const int* cu_tokens,
                      const int* positions, int n, int seq_begin, int n_seqs, int token_begin,
                      int n_tokens, int max_q_len, int max_kv_len, int max_pages,
                      int nq, int nkv, int d, int page_size, int window, float scale,
                      int splits, int chunk, hipStream_t stream);
// Decode steps (one token a request, head sizes in steps of 64): per-head norm, rotation, cache write, attention
// and the merge of the key splits in one kernel.  `workspace` holds ia_attention_decode_workspace() floats;
// `counters` holds at least ia_attention_decode_counters() 32-bit words that are zero before the call and zero
// again after it (calls that share them must not overlap).
int ia_attention_mfma_has_fused(void);
long long ia_attention_decode_workspace(int n, int nq, int nkv, int splits);
long long ia_attention_decode_counters(int n, int nq, int nkv, int splits);
int ia_attention_mfma_decode_fused(void* out, float* workspace, const void* qkv, void* k_cache,
                                   void* v_cache, const int* block_table, const int* cu_tokens,
                                   const int* positions, const int* slots, const float* q_norm_w,
                                   const float* k_norm_w, const float* cos_t, const float* sin_t,
                                   float eps, int add_one, int n, int seq_begin, int n_seqs,
                                   int token_begin, int n_tokens, int max_kv_len, int max_pages,
                                   int nq, int nkv, int d, int page_size, int window, float scale,
                                   int splits, int chunk, int* counters, int n_counters, hipStream_t stream);

#ifdef __cplusplus
}
#endif
