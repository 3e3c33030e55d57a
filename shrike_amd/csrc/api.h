// C entry points of libshrike_hip: thin host launchers around the gfx950
// kernels.  Every pointer is device memory unless said otherwise; `dtype` is
// 0 for float32 and 1 for bfloat16; `stream` is a hipStream_t.  A call returns
// 0 on success; otherwise shk_last_error() describes what was refused and
// nothing was launched.  Shapes are checked on the host before any launch.
#pragma once

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* shk_last_error(void);
int shk_version(void);

// dst[i] = src[i] for i < n, except dst[patch_at + j] = patch[j] for j < patch_n (patch
// may be null with patch_n 0).  src and dst may be device memory or page-locked host
// memory: small index arrays and tokens travel by this kernel, not by the copy engine.
int shk_copy_words(const int32_t* src, int32_t* dst, int n, const int32_t* patch, int patch_at,
                   int patch_n, void* stream);

// dst[r, :] = src[index[r], :] for r < rows: rows of `width` 32-bit words, src rows
// `ld` words apart; the caller promises 0 <= index[r] < src_rows.  index may be
// page-locked host memory.
int shk_gather_rows(const int32_t* src, long long ld, int src_rows, const int32_t* index, int32_t* dst,
                    int rows, int width, void* stream);

// Zeroes `bytes` bytes from dst, which must be 4-byte aligned (a fill kernel:
// it may be recorded into a HIP graph).
int shk_zero_bytes(void* dst, long long bytes, void* stream);

// out[i, :] = float(table[ids[i], :]); ids must lie in [0, vocab).
int shk_embed(const void* table, int dtype, const int32_t* ids, float* out, int n, int hidden,
              int vocab, void* stream);

// Residual add fused with RMSNorm.  For each of n rows r (row index rows[r]
// when `rows` is given, else r):  x = resid[row] (+ delta[row]);  if
// write_resid the sum is stored back into resid;  out[r] = x * rsqrt(mean(x^2)
// + eps) * weight.  resid is float32, delta and out have `dtype`, weight is
// float32.  delta_splits > 0: delta is float32 [delta_splits][resid rows][hidden],
// partial sums of a product split along k, added in order.
int shk_add_rmsnorm(float* resid, const void* delta, const float* weight, float eps, void* out,
                    int dtype, const int32_t* rows, int n, int hidden, int write_resid,
                    int delta_splits, int resid_rows, void* stream);

// out[i, j] = act(gu[i, j]) * gu[i, inter + j] for j < inter; gu is [n, 2*inter].
// act 1: SiLU; act 2: GELU in its tanh form.
int shk_act_mul(const void* gu, void* out, int dtype, int n, int inter, int act, void* stream);

// out[n, m] (+)= a[n, k] @ w[m, k]^T + bias[m].  a and w have in_dtype, out has
// out_dtype, bias is float32 or null.  lda/ldo are row strides in elements.
// With `accumulate` the product is added to what out holds (out_dtype float32
// only).  The reduction order over k is the same for every row and column, so
// a row's result does not depend on which other rows are in the call.
int shk_gemm(const void* a, const void* w, const float* bias, void* out, int n, int m, int k,
             int lda, int ldo, int in_dtype, int out_dtype, int accumulate, void* stream);

// wt = the tiled layout of the row-major bfloat16 matrix w[m, k] (see
// gemm_bf16.hip): ceil(m/16) * ceil(k/32) tiles of 1 KiB.
int shk_retile_weight(const void* w, int m, int k, void* wt, void* stream);

// wt = the tiled layouts of a gated feed-forward's gate and up matrices ([m, k]
// each, given tiled) interleaved by blocks of 16 rows.
int shk_interleave_gate_up(const void* gate_t, const void* up_t, int m, int k, void* wt,
                           void* stream);

// out[n, m] (+)= a[n, k] @ w^T + bias with w given in the tiled layout; a is
// bfloat16 row-major with row stride lda; out is bfloat16 or float32.
// gated != 0: wt is an interleaved gate/up pair and out[n, m] = act(a @ gate^T) *
// (a @ up^T), without bias or accumulation; gated is the activation, 1 for SiLU,
// 2 for GELU in its tanh form.
// ksplit > 1 (at most 64 rows, float32 output, no bias): the k range is shared
// by ksplit workgroups per block of weight rows and out is [ksplit][n][m], the
// partial sums, which the kernel that reads the product adds up in order
// (shk_add_rmsnorm, shk_rope_kv_store).  shk_gemm_bf16_splits says how many
// shares fill the chip for a shape (1: do not split).
int shk_gemm_bf16_tiled_weight(const void* a, const void* wt, const float* bias, void* out, int n,
                               int m, int k, int lda, int ldo, int out_dtype, int accumulate,
                               int gated, int ksplit, void* stream);
int shk_gemm_bf16_splits(int n, int m, int k);
// 2 where a product of many tokens runs as two (the weight rows whose tiles make whole
// rounds of the compute units, then the rest with tiles of its own), else 1.
int shk_gemm_bf16_parts(int n, int m, int k, int gated);

// The matrix instruction alone, for measuring its rate on operands of a given kind:
// workgroups x 4 wavefronts each multiply, iters times, a 64 x 64 x 32 block
// (2 * 64 * 64 * 32 flop) from `operands` (64 KiB of bfloat16), kept in registers.
// out: workgroups * 256 floats.
int shk_mfma_alone(const void* operands, float* out, int workgroups, int iters, void* stream);

// Position encoding and cache write for the n tokens of a step.  qkv is
// [n, (heads + 2*kv_heads) * head_dim]: queries, keys, values.  Queries and
// keys are rotated by position (pairs (i, i + rot_dim/2), angle position *
// inv_freq[i]); queries are rewritten in place; keys and values go to their
// page slots: page = tables[token_seq[t] * table_stride + position / page_size].
// The key pool holds each page's keys in slabs of 32 elements, [num_pages,
// kv_heads, head_dim / 32, page_size, 32] (one slab of head_dim elements where
// head_dim is no multiple of 32); the value pool is stored transposed,
// [num_pages, kv_heads, head_dim, page_size].  rot_dim 0 rotates nothing;
// write_kv 0 leaves the pools alone.
// splits > 0: the projections come as float32 partial sums `parts`
// [splits][n][width] of a product split along k; they are added in order, `bias`
// (float32 [width] or null) is added, and the rotated queries are written to
// qkv's query columns (qkv is then output only).
int shk_rope_kv_store(void* qkv, int dtype, int n, int heads, int kv_heads, int head_dim,
                      int rot_dim, const float* inv_freq, const int32_t* positions,
                      const int32_t* token_seq, const int32_t* tables, int table_stride,
                      void* k_pool, void* v_pool, int page_size, int num_pages, int write_kv,
                      const float* parts, int splits, const float* bias, void* stream);

// Causal attention of n query tokens over their sequences' paged caches.
// Token t (position p, sequence s) reads keys j in (p - window, p] (all j <= p
// when window <= 0) through tables[s].  q has row stride q_stride elements,
// out is [n, heads * head_dim].  Softmax and accumulation are float32.
int shk_attention(const void* q, int q_stride, void* out, int dtype, int n, int heads,
                  int kv_heads, int head_dim, const int32_t* positions, const int32_t* token_seq,
                  const int32_t* tables, int table_stride, int num_seqs, const void* k_pool,
                  const void* v_pool, int page_size, int num_pages, int window, float scale,
                  void* stream);

// 1 if the MFMA attention kernels take these shapes (head_dim a multiple of 32
// up to 256, page_size a multiple of 16, at most 16 query heads per key/value
// head, q rows 16-byte aligned); otherwise shk_attention serves them.
int shk_attention_supports_mfma(int heads, int kv_heads, int head_dim, int page_size, int q_stride);

// bfloat16 decode attention: sequence s has one query token, row s of q, at
// positions[s].  Its keys are split over nsplit wavefronts per key/value head;
// `partial` is float32 scratch of num_seqs * heads * nsplit * (head_dim + 2).
// streaming != 0: keys and values are fetched with non-temporal loads (faster when a
// launch reads tens of megabytes of them, slightly slower below; the result is the same).
int shk_attention_decode_bf16(const void* q, int q_stride, void* out, int num_seqs, int heads,
                              int kv_heads, int head_dim, const int32_t* positions,
                              const int32_t* tables, int table_stride, const void* k_pool,
                              const void* v_pool, int page_size, int window, float scale,
                              float* partial, int nsplit, int streaming, void* stream);

// bfloat16 attention for prompt portions, in tiles of 16 queries: tile i covers
// queries tile_q0[i] .. +16 of sequence tile_seq[i]'s portion.  cu_q[s] is the
// first token row of sequence s in q/out, ctx_lens[s] its length after the step.
int shk_attention_prefill_bf16(const void* q, int q_stride, void* out, int num_tiles, int heads,
                               int kv_heads, int head_dim, const int32_t* cu_q,
                               const int32_t* ctx_lens, const int32_t* tile_seq,
                               const int32_t* tile_q0, const int32_t* tables, int table_stride,
                               const void* k_pool, const void* v_pool, int page_size, int window,
                               float scale, void* stream);

// The same for all query heads of a key/value head at once: a workgroup serves
// `tiles` = shk_attention_prefill_shared_tiles(...) consecutive 16-query tiles of
// one sequence (wg_seq, wg_q0 in steps of 16 * tiles) and stages each chunk of
// keys once in LDS.  small != 0: workgroups of 8 wavefronts instead of 16, with
// half as many tiles each, for portions that would otherwise make too few
// workgroups for the chip.  tiles == 0: the shape is not served (more query
// heads per key/value head than a workgroup has wavefronts, head_dim > 128).
// Entries are launched in the order of the list.  nsplit > 1 shares every entry's
// keys among nsplit workgroups (for a few queries far into a sequence, which alone
// would leave most of the chip idle); their results go through `partial`
// (prompt_tokens * heads * nsplit * (head_dim + 2) floats) and are merged into out.
// first_token: the index of the step's first prompt token (prompt tokens follow
// the single tokens); prompt_tokens: how many there are.
int shk_attention_prefill_shared_tiles(int heads, int kv_heads, int head_dim, int small);
int shk_attention_prefill_shared_bf16(const void* q, int q_stride, void* out, int num_wgs,
                                      int heads, int kv_heads, int head_dim, const int32_t* cu_q,
                                      const int32_t* ctx_lens, const int32_t* wg_seq,
                                      const int32_t* wg_q0, const int32_t* tables,
                                      int table_stride, const void* k_pool, const void* v_pool,
                                      int page_size, int window, float scale, int small,
                                      float* partial, int nsplit, int first_token,
                                      int prompt_tokens, void* stream);

// out[r] = lowest index of the largest value of logits[r, :vocab].  Rows wider
// than 4096 are searched in chunks; scratch then holds
// shk_argmax_scratch_floats(rows, vocab) floats (0: not needed).
int shk_argmax(const float* logits, int32_t* out, int rows, int vocab, int ld, float* scratch,
               void* stream);
int shk_argmax_scratch_floats(int rows, int vocab);

// shk_argmax for callers that cannot allocate device memory or bring a workspace
// (code recorded into a HIP graph, tight serving loops, harnesses that forbid
// hipMalloc).  It has no counterpart in the reference.  The chunk results live
// in an array of shk_argmax_static_max_floats() floats (256 KiB) that the library
// holds on every GPU it runs on until the process ends; a call whose
// shk_argmax_scratch_floats(rows, vocab) exceeds that is refused.  No call
// allocates or frees anything.  All calls on one GPU share that GPU's array:
// calls that overlap there (two streams, two threads) race; calls in stream order
// do not, and nothing an earlier call left in the array is read.
int shk_argmax_static(const float* logits, int32_t* out, int rows, int vocab, int ld, void* stream);
int shk_argmax_static_max_floats(void);

// Temperature / top-p sampling of one token per row (see sampling.hip).
// temperature[r] == 0 takes the argmax.  uniforms[r] in [0, 1) is the draw.
// `scratch` holds scratch_floats >= shk_sample_scratch_floats(rows, vocab) floats,
// 16-byte aligned.  nucleus == 0 promises that every row's top_p is 1 or more
// (the passes that find the nucleus are then left out; top_p is not read).
int shk_sample(const float* logits, int32_t* out, const float* temperature, const float* top_p,
               const float* uniforms, float* scratch, long long scratch_floats, int rows, int vocab,
               int ld, int nucleus, void* stream);
long long shk_sample_scratch_floats(int rows, int vocab);

// A list of launches run by one call.  A shk_call names a launcher of this header that
// takes a stream (shk_call_id gives its number by name, -1 for others) and holds its
// arguments in order, one per slot: pointers and integers as they are, a float's bits
// in the low 32 bits; the slot of the launcher's own stream argument is ignored and
// `stream` is passed instead.  The calls run in order on `stream`; the first that
// refuses its arguments ends the run with its status and message (those before it
// have been launched).
#define SHK_CALL_MAX_ARGS 26
typedef struct shk_call {
  int32_t launcher;
  int32_t reserved;
  int64_t args[SHK_CALL_MAX_ARGS];
} shk_call;
int shk_call_id(const char* name);
int shk_run_calls(const shk_call* calls, int n, void* stream);

#ifdef __cplusplus
}
#endif
