// C interface of the kernel library (libpsamd_kernels.so). Every function launches on the
// given HIP stream, takes raw device pointers, returns 0 on success and otherwise leaves a
// message for psamd_last_error(). dtype codes: 0 = float32, 1 = bfloat16. Shapes are checked
// on the host before a launch; a shape a kernel does not take is an error, never a wrong
// result.
#pragma once

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* psamd_last_error(void);

// out[t, :] = float(table[ids[t], :]); table is [vocab, hidden]; an id outside [0, vocab) reads the nearest row.
int psamd_embed(void* stream, const int32_t* ids, const void* table, int table_dtype, float* out, int64_t tokens,
                int hidden, int vocab);

// x = residual + delta, where delta is [rows, hidden] (delta_dtype) or n_partials float32 slices of that
// shape, partial_stride elements apart (the partial sums of a K-split product).
// rows == NULL: residual[r] = x[r], out[r] = weight * rmsnorm(x[r]) for r < out_rows.
// rows != NULL: out[i] = weight * rmsnorm(x[rows[i]]); residual untouched.
int psamd_add_rmsnorm(void* stream, float* residual, const void* delta, int delta_dtype, int n_partials,
                      int64_t partial_stride, const int32_t* rows, const void* weight, int weight_dtype, float eps,
                      void* out, int act_dtype, int64_t out_rows, int hidden);

// out[t, c] = silu(gate_up[t, c]) * gate_up[t, inter + c]
int psamd_swiglu(void* stream, const void* gate_up, void* out, int act_dtype, int64_t tokens, int inter);

// Rotates the q and k heads of qkv[t] in place by table[positions[t]] (NULL table: no rotation) and, if kv
// is given, writes k and v of token t to page slot write_slot[t] (= page * 16 + offset).
int psamd_rope_kv_append(void* stream, void* qkv, int act_dtype, int64_t tokens, int hq, int hkv, int head_dim,
                         const int32_t* positions, const float* table, void* kv, const int32_t* write_slot);

// out[M, N] = x[M, K] * w[N, K]^T with float accumulation (LDS-tiled FMA; exact path and fallback).
int psamd_linear(void* stream, const void* x, int x_dtype, const void* w, int w_dtype, void* out, int out_dtype,
                 int64_t M, int N, int K);

// Library product (hipBLASLt, looked up at run time) for large bfloat16 steps, with the
// descriptors and the chosen algorithm kept per shape. psamd_gemm_lt_available(): 1 if the
// library is ready on the current device; its first call per device allocates the workspace.
// use_workspace = 0: only algorithms that need none (for calls under stream capture).
// psamd_gemm_lt returns 2, not an error, if the library has no algorithm for the shape.
int psamd_gemm_lt_available();
int psamd_gemm_lt(void* stream, const void* x, const void* w, void* out, int out_dtype, int64_t M, int N, int K,
                  int use_workspace, int accumulate);


// bfloat16 product for M <= 64 on the matrix cores. epilogue 1: w = [gate; up], out = silu(gate) * up.
// ksplit > 1: out receives ksplit float32 partial sums [ksplit][M, n_out] (plain epilogue only).
int psamd_linear_skinny_ksplit(int M, int n_out, int K);
int psamd_linear_skinny(void* stream, const void* x, const void* w, void* out, int out_dtype, int M, int n_out, int K,
                        int epilogue, int ksplit);

// The q/k/v projection of a step of at most 64 tokens fused with the rotation of q and k and the write of k
// and v into their cache pages (see psamd_rope_kv_append for the meaning of table, kv and write_slot).
int psamd_qkv_rope_append(void* stream, const void* x, const void* w, void* qkv_out, int M, int K, int hq, int hkv,
                          int head_dim, const int32_t* positions, const float* table, void* kv,
                          const int32_t* write_slot);

// Small steps without a norm kernel and without partial slices to add up (bfloat16, M <= 16):
// the products that feed the residual stream add into it (psamd_linear_skinny_add: float atomics,
// K split over workgroups; the order of the additions differs from run to run), and the products
// that read the normalized stream (q/k/v, gate/up, the output matrix) take rows of the float32
// residual and apply the RMS norm themselves (weight norm_w, bfloat16 or float32; statistics in
// 32-bit, eps inside the root). psamd_normed_supports: whether they take M tokens of width K.
int psamd_normed_supports(int M, int K);
int psamd_linear_skinny_add(void* stream, const void* x, const void* w, float* out, int M, int n_out, int K);
int psamd_linear_normed(void* stream, const float* resid, const int32_t* rows, const void* norm_w, int norm_w_dtype,
                        float eps, const void* w, void* out, int out_dtype, int M, int n_out, int K, int epilogue);
int psamd_qkv_rope_append_normed(void* stream, const float* resid, const void* norm_w, int norm_w_dtype, float eps,
                                 const void* w, void* qkv_out, int M, int K, int hq, int hkv, int head_dim,
                                 const int32_t* positions, const float* table, void* kv, const int32_t* write_slot);

int psamd_attention_generic(void* stream, const void* qkv, int q_stride, void* out, const void* kv, int act_dtype,
                            int64_t tokens, const int32_t* positions, const int32_t* tok_item,
                            const int32_t* table_off, const int32_t* block_ids, int hq, int hkv, int head_dim,
                            float scale, int window);

int psamd_attention_mfma_supports(int hq, int hkv, int head_dim);

// Few query tiles on long contexts: their keys are cut into nsplit runs (what
// psamd_attention_prefill_nsplit allows for the step's sizes, or fewer; 1: no cut) that
// part_o [32 * n_tiles * hq * nsplit * head_dim] and part_ml [32 * n_tiles * hq * nsplit * 2] carry
// to a merge kernel.
int psamd_attention_prefill_nsplit(int n_tiles, int max_kv_len, int hq, int hkv, int head_dim);
// pf_tiles: (item, first query) of every tile of 32 queries; pf_blocks: the first tile of every run
// of up to four consecutive tiles of one item, in the order of the tiles (n_blocks = 0: no such
// list; steps with one or two query heads per kv head then run a slower form).
// The most rows (32 * n_tiles * nsplit) of part_o / part_ml any step of this shape needs.
int psamd_attention_prefill_part_rows(int hq, int hkv, int head_dim);
int psamd_attention_prefill(void* stream, const void* qkv, int q_stride, void* out, const void* kv,
                            const int32_t* pf_tiles, int n_tiles, const int32_t* pf_blocks, int n_blocks, int max_kv_len,
                            const int32_t* item_start, const int32_t* item_pos0,
                            const int32_t* table_off, const int32_t* block_ids, int hq, int hkv, int head_dim,
                            float scale, int window, float* part_o, float* part_ml, int nsplit);

// The plan for a decode step's keys: whether its context lengths count as skewed (one far longer
// than the rest), into how many runs of at least how many keys each request's keys are cut, and
// the most (requests x runs) any plan gives (part_o: that many x hq x head_dim floats).
int psamd_attention_decode_skewed(int n_dec, int longest, int64_t total);
int psamd_attention_decode_plan(int n_dec, int kv_len, int skewed, int hkv, int window, int* nsplit, int* min_run);
int psamd_attention_decode_max_parts(int max_requests);

int psamd_attention_decode(void* stream, const void* qkv, int q_stride, void* out, const void* kv, float* part_o,
                           float* part_ml, const int32_t* dec_items, int n_dec, const int32_t* item_start,
                           const int32_t* item_end, const int32_t* table_off, const int32_t* block_ids, int hq,
                           int hkv, int head_dim, int nsplit, float scale, int window, int min_split_keys);

// out[r] = argmax (temperature[r] <= 0) or the inverse-CDF draw with uniform[r] in [0, 1).
int64_t psamd_sample_scratch_floats(int rows);
int psamd_sample(void* stream, const float* logits, const float* temperature, const float* uniform, int32_t* out,
                 float* scratch, int rows, int vocab);

// psamd_sample for callers that cannot allocate or bring a scratch buffer (code under HIP graph
// capture, serving loops and harnesses that forbid hipMalloc). It has no counterpart in the
// reference. The run statistics live in a 128 KiB array inside the library that every GPU holds
// until the process ends, so rows is limited to psamd_sample_static_max_rows() (256); more is an
// error. The call allocates nothing and calls no library routine that does; the caller passes
// inputs and outputs as for psamd_sample, with the stream's device current. All calls on one GPU
// share the array: two calls that overlap there (different streams, or two threads) race, and
// the caller has to order them. Same kernels and the same result as psamd_sample. The first
// call on a device asks the runtime for the array's address there (hipGetSymbolAddress, under
// a mutex): make it once at set-up, outside any graph capture; later calls only launch.
int psamd_sample_static_max_rows(void);
int psamd_sample_static(void* stream, const float* logits, const float* temperature, const float* uniform,
                        int32_t* out, int rows, int vocab);

#ifdef __cplusplus
}
#endif
