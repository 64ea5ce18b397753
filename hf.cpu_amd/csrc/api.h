// The C interface of the kernel library. Pointers are device pointers unless named
// host; sizes are in elements; `dtype` is HFA_F32 (0) or HFA_BF16 (1). Every function
// returns 0 on success; otherwise hfa_last_error() describes what was refused.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* hfa_last_error(void);
int hfa_version(void);

// x[t, :] = table[tokens[t], :] as fp32.  (reference: src/model.c:566-571)
int hfa_embed(const void* table, int table_dtype, const int* tokens, float* x, int n_tokens, int width,
              int vocab, hipStream_t stream);

// out[r, :] = x[rows ? rows[r] : r, :] * rsqrt(mean(x^2) + eps) * w.  (src/mathx.c:65-75)
// With splits > 0 (and no rows): first x[r, :] += sum_s partial[s][r][:] + partial_bias, written
// back: the residual sum of a matrix product that hfa_gemm deferred (src/model.c:609, 623).
int hfa_rmsnorm(float* x, const float* w, void* out, int out_dtype, const int* rows, int n_rows, int width,
                float eps, const float* partial, int splits, const float* partial_bias, hipStream_t stream);

// out[m, n] (+)= sum_k a[m, k] * w[n, k] + bias[n].  a: [M, K] row stride lda; w: [N, K] row
// stride ldw; out row stride ldo. `accumulate` adds into fp32 `out` (the residual sum).
// bf16 operands with K and the row strides multiples of 8 run on the matrix cores (K split over
// `workspace` for small M); everything else, and everything when `force_plain`, runs the plain
// fp32 multiply-add kernel. `epilogue` 1 (matrix cores only): the columns of w come in blocks of
// 32 gate rows, 32 up rows, and out[m, f] = silu(gate) * up has N / 2 columns (src/model.c:537).
// `defer`: if K was split, leave the partial sums ([splits][M][N] fp32 at the start of the
// workspace) for the caller's next kernel and report the number of splits in *pending_splits.
// (src/model.c:408-424)
int hfa_gemm(const void* a, int a_dtype, int lda, const void* w, int w_dtype, int ldw, const float* bias,
             void* out, int out_dtype, int ldo, int accumulate, int epilogue, int M, int N, int K,
             void* workspace, size_t workspace_bytes, int defer, int* pending_splits, int force_plain,
             hipStream_t stream);
int hfa_gemm_finish(const void* partial, int splits, const float* bias, void* out, int out_dtype, int ldo,
                    int accumulate, int epilogue, int M, int N, hipStream_t stream);

// The product for up to 32 rows in which every block owns a range of outputs and finishes them itself (bf16
// operands, K a multiple of 128; see gemm_rows.hip), with what follows a product in a decode step in its last lines:
//   HFA_ROWS_OUT     out[m, n] = r[m] * sum + bias[n], fp32 or bf16 (out_dtype)
//   HFA_ROWS_RESID   x[m, n] += sum + bias[n] (fp32, in place); ssq_out[b][m] = block b's share of sum_n x[m, n]^2
//                    ([hfa_gemm_rows_parts()][16] floats, [..][32] from 17 rows up: give room for 32); xg[m, n] = bf16(x[m, n] * g[n]) if xg is given
//   HFA_ROWS_SWIGLU  act[m, f] = bf16(silu(r[m] * sum_gate) * (r[m] * sum_up)), N features, w's 2 N rows in blocks of
//                    32 gate rows, 32 up rows (src/model.c:537)
// r[m] = rsqrt(sum over the parts_in shares ssq_in[.][m] * inv_width + eps), or 1 without ssq_in: the RMS norm of the
// tensor whose product with the norm's weight is `a` (src/mathx.c:65-75), applied to the sums instead of the operand.
// hfa_gemm_rows_supports says whether a shape is taken (1 to 32 rows, K a multiple of 128, strides multiples of 8).
// ssq_in has the layout that a HFA_ROWS_RESID product of the same number of rows left.
#define HFA_ROWS_OUT 0
#define HFA_ROWS_RESID 1
#define HFA_ROWS_SWIGLU 2
int hfa_gemm_rows_parts(void);
int hfa_gemm_rows_supports(int mode, int M, int N, int K, int lda, int ldw);
int hfa_gemm_rows(int mode, const void* a, int lda, const void* w, int ldw, int M, int N, int K, const float* bias,
                  const float* ssq_in, int parts_in, float inv_width, float eps, void* out, int ldo, int out_dtype,
                  float* x, int ldx, float* ssq_out, const float* g, void* xg, int ldxg, void* act, int ldact,
                  hipStream_t stream);

// Rotary position encoding on the q (and k) heads inside qkv rows [q | k | v], split-half
// pairing, and the store of k (rotated) and v into cache rows slot_map[t] (src/model.c:468-493,
// 587-600). rot_dim 0: no rotation. n_kv_heads 0: the rows hold q only, nothing is stored.
// Query and key heads have head_dim values, value heads v_head_dim (the same in most models; a
// prompt-sized bf16 call with equal sizes takes a kernel of its own).
// Cache layout: row r = page * page_tokens + offset. Keys: k_cache[r * width + c], width =
// n_kv_heads * head_dim. Values (width n_kv_heads * v_head_dim) lie transposed inside their page, so that
// the keys of one value column are contiguous: v_cache[page * page_tokens * width + c * page_tokens + offset].
// With splits > 0 the input is not qkv but the partial sums of a deferred hfa_gemm
// ([splits][n_tokens][(n_heads + 2 n_kv_heads) * head_dim] fp32) plus partial_bias; the rotated
// queries are written into qkv.
int hfa_rope_store(void* qkv, int dtype, int ld, const int* positions, const float* inv_freq, int rot_dim,
                   int n_heads, int n_kv_heads, int head_dim, int v_head_dim, void* k_cache, void* v_cache,
                   const int* slot_map, int page_tokens, int n_tokens, const float* partial, int splits,
                   const float* partial_bias, hipStream_t stream);

// `run` (a request's tokens in one call) from which hfa_paged_attention takes the kernel for prompt
// portions for the whole call; see the launcher in attention_mfma.hip.
int hfa_attention_prompt_rows(void);

// Softmax attention of each token's query heads over its request's cached keys and values
// (src/model.c:499-528). Key j of the request in slot s lies in cache row
// block_table[s, j / page_tokens] * page_tokens + j % page_tokens. A key is visible to the
// query at position p iff j <= p and (window == 0 or p - j < window). q_start[n_seqs + 1] gives
// each request's run of tokens (consecutive positions of one slot); max_q_len and max_seq_len
// bound the runs and the positions. Key rows are kv_width wide with head_dim values a head, value rows
// v_width with v_head_dim a head; out has v_head_dim values per query head. bf16 with one head size for
// both that is a multiple of 32, page_tokens a power of two from 4
// and at most 32 query heads per key/value head runs on the matrix cores, the key range
// split over `workspace` when there are few queries; everything else, and everything when
// `force_plain`, runs the plain kernel. `slopes` (one fp32 per query head, or null) is the hook for a position
// encoding that enters the scores rather than the queries and keys: the score of key j for the query at p
// becomes dot * scale + slopes[h] * (j - p); with slopes the plain kernel runs.
int hfa_paged_attention(const void* q, int dtype, int ldq, const void* k_cache, const void* v_cache,
                        int kv_width, int v_width, const int* block_table, int max_blocks, const int* token_slot,
                        const int* positions, const int* q_start, int n_seqs, int max_q_len, int max_seq_len,
                        void* out, int ldo, int n_tokens, int n_heads, int n_kv_heads, int head_dim, int v_head_dim,
                        int page_tokens, int window, float scale, const float* slopes, void* workspace,
                        size_t workspace_bytes, int force_plain, hipStream_t stream);

// Decoded tokens (one a request) whose queries, new keys and new values are still the 32-bit rows [q | k | v] that
// the product left (`raw`, bias added): rotation of queries and keys (cos_sin: hfa_rope_table's output for the step's
// tokens, [token][head_dim / 2 cosines, head_dim / 2 sines]; null: none), the store of the new key and value into
// cache rows slot_map[t], and attention over the cache, in one kernel (plus the merge of key chunks): what
// hfa_rope_store and hfa_paged_attention give one after the other. bf16 cache, matrix cores only: ask
// hfa_decode_attention_supports first.
int hfa_rope_table(const int* positions, const float* inv_freq, int half, float* out, int n_tokens, hipStream_t stream);
int hfa_decode_attention_supports(int n_heads, int n_kv_heads, int head_dim, int rot_dim, int page_tokens, int kv_width,
                                  int ld_raw, int ldo);
int hfa_decode_attention(const float* raw, int ld_raw, const float* cos_sin, void* k_cache, void* v_cache, int kv_width,
                         const int* slot_map, const int* block_table, int max_blocks, const int* token_slot,
                         const int* positions, const int* q_start, int n_seqs, int max_seq_len, void* out, int ldo,
                         int n_heads, int n_kv_heads, int head_dim, int page_tokens, int window, float scale,
                         void* workspace, size_t workspace_bytes, hipStream_t stream);

// out[t, i] = silu(gate_up[t, i]) * gate_up[t, width + i].  (src/model.c:532-538)
int hfa_swiglu(const void* gate_up, void* out, int dtype, int n_tokens, int width, hipStream_t stream);

// dst[idx[i]] = val[i]
int hfa_scatter_i32(int* dst, const int* idx, const int* val, int n, hipStream_t stream);

// dst[dst_idx[i]] = src[src_idx[i]] (tokens sampled on the device go into the next step's inputs)
int hfa_move_i32(int* dst, const int* dst_idx, const int* src, const int* src_idx, int n, hipStream_t stream);

// out[r] = first index of the maximum of logits[r, :].  (src/sample.c:72-77)
// `workspace` holds the candidates of the first of its two stages (n_rows * 64 * 8 bytes).
int hfa_argmax(const float* logits, int ld, int* out, int n_rows, int vocab, void* workspace,
               size_t workspace_bytes, hipStream_t stream);

// hfa_argmax for callers that cannot allocate or bring a workspace: code under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc. It has no counterpart in the reference. The
// candidates of the first stage lie in a device array that the library holds itself (128 KiB on every
// GPU it runs on, until the process ends), so the call allocates nothing; the caller still passes
// logits and out. At most HFA_ARGMAX_STATIC_ROWS rows; more are refused. Calls that overlap on one
// GPU share that array and race; nothing needs clearing between calls that follow each other.
// The first call on a device asks the runtime for the array's address there, which is no stream
// operation: it must be an eager call (one made while the stream is being captured is refused with
// a message that says so); every later call on that device may be captured.
#define HFA_ARGMAX_STATIC_ROWS 256
int hfa_argmax_static(const float* logits, int ld, int* out, int n_rows, int vocab, hipStream_t stream);

// All candidates of the chosen rows (rows[i], or row i if rows is null) in the order (logit
// descending, id ascending), as the reference's sort leaves them when top-k is off
// (src/sample.c:59-64, 93-98): ids and vals are [n_rows, vocab]. `scratch` needs
// hfa_order_rows_scratch(n_rows, vocab) bytes, 8-byte aligned.
size_t hfa_order_rows_scratch(int n_rows, int vocab);
int hfa_order_rows(const float* logits, int ld, const int* rows, int* ids, float* vals, int n_rows, int vocab,
                   void* scratch, size_t scratch_bytes, hipStream_t stream);

// The draw over ordered rows (src/sample.c:99-114): vals/ids [n_rows, vocab] as hfa_order_rows leaves them,
// params[r] = {temp, top_p, min_p, u} with u the request's uniform number in [0, 1), cuts[r] = candidates
// left by top-k (1..vocab). tokens[r] = the drawn id. vals is overwritten with the probabilities.
int hfa_draw_rows(float* vals, const int* ids, int n_rows, int vocab, const float* params, const int* cuts,
                  int* tokens, hipStream_t stream);

// The k best of each row in the order (logit descending, id ascending) (src/sample.c:59-64),
// and stats[r] = {max, log(sum(exp(l - max)))} (src/sample.c:25-33). k <= 1024.
int hfa_topk(const float* logits, int ld, int* ids, float* vals, float* stats, int n_rows, int vocab, int k,
             hipStream_t stream);

// Random weights on the device: element e of the tensor with `key` by the counter-based rule that
// weights/random_init.py states (the host's writer computes the same bits). dtype HFA_F32 or HFA_BF16
// with rule 0 (N(0, std): scale = std / sqrt(8 (65536^2 - 1) / 12)) or 1 (1 + that); dtype 2 (int32)
// with rule 2 (uniform below `bound`). The reference's one generator for model and oracle:
// tools/mkmodel.pl:104-127.
int hfa_random_fill(void* out, int dtype, size_t n, uint64_t key, float scale, int rule, int bound,
                    hipStream_t stream);

// The device's own peaks (the reference's read_sum and fma_burn, src/kern.h:17-23): a streaming read
// of `bytes` (16-byte aligned; `sink` is 16 bytes that are almost never written) by `blocks_per_cu`
// blocks of 256 threads a CU, a copy, and a burn of
// the matrix cores on register operands (`zeros`: all-zero operands, else small pseudo-random ones):
// `out` takes one float per thread of the launch, hfa_probe_mfma_threads() of them; *flops is what it
// computed. The caller times them.
int hfa_probe_read(const void* src, size_t bytes, void* sink, int blocks_per_cu, hipStream_t stream);
int hfa_probe_copy(const void* src, void* dst, size_t bytes, hipStream_t stream);
int hfa_probe_mfma_threads(void);
int hfa_probe_mfma(float* out, int iters, int zeros, double* flops, hipStream_t stream);

#ifdef __cplusplus
}
#endif
