/*
 * paged_attn.h — C ABI of libpaged_attn.so: paged flash attention for AMD
 * Instinct MI355X (gfx950), hand-written HIP kernels.
 *
 * Role relative to the reference (aws-neuron/nkipy): these entry points stand
 * where the reference runs its attention math on the device, i.e. the body of
 *   examples/models/qwen3/kernels/attention.py:108-144   (repeat_kv, QK^T/sqrt(d),
 *   causal mask, softmax, PV), its multi-token-at-offset variant
 *   examples/models/gpt_oss/kernels/attention.py:102-150, and the execute call
 *   that launches it, spike/src/spike/spike_model.py:248-288 -> spike/src/model.cpp:90-110
 *   (NrtModel::execute).  The reference has no paged/block-table form; the
 *   block-table gather is the np.take form of nkipy/src/nkipy/core/tensor.py:575-640
 *   applied to a pool laid out [num_blocks, block_size, Hkv, D].
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller (the reference's
 *     ownership rule: caller allocates inputs and outputs,
 *     nkipy/src/nkipy/runtime/device_tensor.py:51-74); nothing is allocated,
 *     freed or retained by the library;
 *   - calls are asynchronous on `stream` (a hipStream_t passed as void*; NULL is
 *     the default stream) and never synchronise;
 *   - return 0 = launched; negative = argument error found on the host before
 *     any launch (pa_last_error() holds the text); positive = hipError_t;
 *   - thread-safe and re-entrant: no mutable global state except the debug and
 *     profiling switches below, which are meant for tests and benchmarks;
 *   - dtype codes: PA_F32 = 0, PA_BF16 = 1, PA_FP8_E4M3FN = 2 (OCP e4m3fn,
 *     KV cache only, with one float scale per (block, kv head)).
 *
 * Tensor layouts (row-major, contiguous)
 *   q, out (decode)      [B, Hq, D]
 *   q, out (prefill)     [B, T, Hq, D]; rows t >= query_lens[b] are padding
 *   k_cache, v_cache     [num_blocks, block_size, Hkv, D]
 *   k_scale, v_scale     [num_blocks, Hkv] float (fp8 KV only, else NULL)
 *   block_tables         [B, max_blocks_per_seq] int32, logical -> physical block
 *   seq_lens             [B] int32, keys visible to the last query token
 *   query_lens           [B] int32, new tokens of each sequence (<= T, <= seq_lens[b])
 * q head h reads kv head h / (Hq / Hkv)   (attention.py:15-22 repeat_kv).
 */
#ifndef PAGED_ATTN_H_
#define PAGED_ATTN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { PA_F32 = 0, PA_BF16 = 1, PA_FP8_E4M3FN = 2 };

/* Library version: major * 10000 + minor * 100 + patch (a minor step marks a changed or added signature). */
int pa_version(void);

/* Text of the calling thread's most recent error ("" if none).  Mirrors the
 * status strings of spike/src/include/error.h:23-43. */
const char* pa_last_error(void);

/* Optional last step of the reference's pre-attention code, done by the attention kernels
 * themselves as they load the Q rows: QK RMSNorm of Q (examples/models/qwen3/kernels/rmsnorm.py:4-21,
 * applied at qwen3/kernels/attention.py:78-80) and RoPE at the row's absolute position
 * (rope.py:23-48; attention.py:83-97), the position being seq_lens[b] - query_lens[b] + t
 * (seq_lens[b] - 1 for pa_decode).  Results are bit for bit those of pa_qk_norm_rope_kv_write's
 * Q pass followed by the attention call, without that pass's read and rewrite of Q.
 * Tables as for pa_qk_norm_rope_kv_write; norm_weight NULL = rotation only. */
typedef struct pa_q_transform {
  const void* norm_weight;   /* [D] bf16 or NULL */
  const void* rope_cos;      /* [rope_max_pos, D/2] bf16 */
  const void* rope_sin;
  int rope_max_pos;
  float norm_eps;
} pa_q_transform;

/* Bytes of scratch that is enough for pa_decode whichever kernel it picks: split-K
 * partials of D floats of normalised output plus (max, sum) each — one per
 * (sequence, q head, partition) for the fixed-partition kernels, one per
 * (q head, sequence + chunk) for the balanced MFMA schedule. */
size_t pa_decode_workspace_bytes(int B, int Hq, int D, int max_seq_len, int partition_size);

/* The same for a known shape and dtype pair: exactly what the kernel pa_decode picks for it
 * needs (the balanced schedule's [Hq][B + chunks][D + 2] floats for bf16 / fp8 pools at head
 * dim 64 or 128 and a power-of-two block size >= 16, whatever max_seq_len is; the fixed
 * partitions' B x Hq x ceil(max_seq_len / partition_size) slots otherwise, and where the bound
 * makes the call small enough for the fixed-partition matrix-core kernel).  max_seq_len is the
 * positive bound the pa_decode call will pass, already clamped to the table capacity; with
 * max_seq_len <= 0 (pa_decode then uses the capacity, which this function is not told) the
 * answer covers every matrix-core kernel that call can pick — the balanced schedule or up to
 * four fixed partitions — and is 0 for shapes that take the scalar kernel, whose callers must
 * give the bound.  With a positive bound never more than pa_decode_workspace_bytes.  Sizing helper next to the output allocation of
 * nkipy/src/nkipy/runtime/device_tensor.py:51-74. */
size_t pa_decode_workspace_bytes_for(int B, int Hq, int Hkv, int D, int block_size, int max_seq_len,
                                     int partition_size, int q_dtype, int kv_dtype);

/*
 * Paged decode attention: one query token per sequence.
 *   out[b, h, :] = softmax(q[b, h, :] . K_b^T * scale) V_b,  K_b/V_b = the first
 *   seq_lens[b] rows gathered through block_tables[b]   (the decode branch of
 *   examples/models/qwen3/kernels/attention.py:103-144, start_pos = seq_len - 1).
 * Long contexts are split (split-K); partial results go through `workspace` and
 * are merged by a second kernel.  The scalar-ALU kernel (fp32, odd shapes) and
 * the fixed-partition MFMA kernel cut every context into partition_size-token
 * partitions; the default MFMA kernel for bf16 / fp8 KV instead cuts the
 * flattened stream of all sequences' 32-token tiles into equal chunks, one per
 * resident wavefront group, so its partition length follows the batch and the
 * device, not partition_size.  Small calls (by max_seq_len, or by what a sliding window
 * reaches if that is less: at most eight partitions per sequence, at most 256 (sequence,
 * kv head) pairs -- 320 at head dim 64, 1 024 when a sequence is one partition's worth
 * (a bound of at most 768 tokens, or a sliding window that fits a partition) --
 * and at most 160 MiB of K and V) take the fixed-partition MFMA kernel,
 * whose fixed cost is lower: on partitions of 256 tokens when those of partition_size
 * would give the device fewer than about 64 workgroups (a single sequence), and on
 * partitions sized to give one workgroup per CU (256-1 152 tokens) when those of
 * partition_size would give it more workgroups than it has CUs; under a
 * window the partitions count from the first 32-token tile the window reaches.  At head
 * dim 64 and on fp8 pools, whose tokens are half the bytes, a call that would exceed eight
 * partitions is counted on partitions of twice partition_size (not an fp8 pool of head dim
 * 64), a single sequence that would exceed twelve of the finer partitions takes them at 512
 * tokens, and the sized ones may be 2 304 long.
 * The result does not depend on the split beyond the order of float32 sums.
 * max_seq_len: upper bound of seq_lens (sizes the grid and picks the kernel; 0 =
 * max_blocks_per_seq * block_size).  seq_lens[b] == 0 yields zeros.
 * q_dtype / kv_dtype: (F32, F32), (BF16, BF16) or (BF16, FP8_E4M3FN).
 * sinks: NULL, or [Hq] float32 per-head logits that join every softmax as one more column and
 *   are dropped afterwards (examples/models/gpt_oss/kernels/attention.py:137-148): they only
 *   enlarge the denominator.  sliding_window: 0, or W >= 1: the query at position p sees the W
 *   keys (p - W, p] (attention.py:118-125).  Both need the MFMA kernel's shapes (bf16 q, bf16 or
 *   fp8 KV, D in {64, 128}, block_size a power of two >= 16); tiles wholly outside the window are
 *   not read.
 * q_transform: NULL, or the norm and rotation to apply to the Q rows on load (same shapes).
 *   pa_verify and pa_prefill (tiled kernel with asynchronous copies) take it too.
 */
int pa_decode(const void* q, const void* k_cache, const void* v_cache,
              const float* k_scale, const float* v_scale,
              const int32_t* block_tables, const int32_t* seq_lens,
              void* out, void* workspace, size_t workspace_bytes,
              int B, int Hq, int Hkv, int D, int block_size,
              int max_blocks_per_seq, int num_blocks, int max_seq_len,
              float scale, int partition_size, int q_dtype, int kv_dtype,
              const float* sinks, int sliding_window, const pa_q_transform* q_transform, void* stream);

/*
 * pa_decode for callers that cannot allocate device memory or bring a workspace: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the
 * reference (its runtime allocates every tensor up front, nkipy/src/nkipy/runtime/device_tensor.py:51-74).
 * Arguments, validation, kernels and results are pa_decode's (bit for bit); the split-K partials go
 * to a static array of PA_DECODE_NOALLOC_SCRATCH_BYTES inside the library's device code, one copy per
 * GPU, held until the process ends.  A call whose partials need more (see
 * pa_decode_workspace_bytes_for) fails with an argument error before any launch.  The call itself
 * allocates and frees nothing.  All calls on one GPU share that GPU's array: calls that overlap in
 * time on one GPU (different streams, or threads) race; calls on one stream are ordered.
 */
#define PA_DECODE_NOALLOC_SCRATCH_BYTES (32u << 20)
int pa_decode_noalloc(const void* q, const void* k_cache, const void* v_cache,
                      const float* k_scale, const float* v_scale,
                      const int32_t* block_tables, const int32_t* seq_lens, void* out,
                      int B, int Hq, int Hkv, int D, int block_size,
                      int max_blocks_per_seq, int num_blocks, int max_seq_len,
                      float scale, int partition_size, int q_dtype, int kv_dtype,
                      const float* sinks, int sliding_window, const pa_q_transform* q_transform, void* stream);

/*
 * Speculative verify: a few query tokens per sequence against the paged context, causal among
 * themselves -- the non-prefill branch of examples/models/gpt_oss/kernels/attention.py:80-100,
 * 127-135 with seq_len = K+1 ("query at start_pos+i attends to keys <= start_pos+i"), driven by
 * examples/models/gpt_oss/peagle/speculate.py:137-202.  Same result as pa_prefill on the same
 * arguments, and fp8 pools are accepted; built for small T: the (token, head) pairs of a kv group
 * ride along as extra rows of the decode kernel's 16-row query operand, so the context is streamed
 * from HBM once per kv head however many tokens are verified, at decode's bandwidth.
 *   q, out       [B, T, Hq, D] bf16; rows t >= query_lens[b] are padding, zero in out
 *   seq_lens[b]  context length including the query tokens, whose K/V are already in the pool
 *   kv_dtype     PA_BF16 or PA_FP8_E4M3FN (then k_scale / v_scale [num_blocks, Hkv] f32)
 *   workspace    pa_verify_workspace_bytes(B, T, Hq, D) bytes, 16-byte aligned
 *   sinks, sliding_window   as for pa_decode (the window counts back from each query token's own position)
 *   max_seq_len  0, or a host-known upper bound of seq_lens (longer contexts are read up to the bound).  The table
 *                capacity says nothing about the size of a call; with a bound, a small call -- at most eight
 *                512-token partitions per sequence, few sequences and little K and V in all (pa_decode's rule): the
 *                reference's own use, one sequence and a handful of draft tokens -- runs on fixed partitions
 *                as a small pa_decode call does, without the balanced schedule's fixed cost.  Same workspace.
 * D in {64, 128}; block_size a power of two >= 16; T <= PA_VERIFY_MAX_TOKENS.
 */
#define PA_VERIFY_MAX_TOKENS 64
size_t pa_verify_workspace_bytes(int B, int T, int Hq, int D);
int pa_verify(const void* q, const void* k_cache, const void* v_cache,
              const float* k_scale, const float* v_scale,
              const int32_t* block_tables, const int32_t* seq_lens, const int32_t* query_lens,
              void* out, void* workspace, size_t workspace_bytes,
              int B, int T, int Hq, int Hkv, int D, int block_size,
              int max_blocks_per_seq, int num_blocks, int max_seq_len,
              float scale, int kv_dtype, const float* sinks, int sliding_window,
              const pa_q_transform* q_transform, void* stream);

/*
 * Paged chunked prefill with a cached prefix, causal: query token i of sequence
 * b (i < query_lens[b]) sees keys j <= seq_lens[b] - query_lens[b] + i
 * (examples/models/gpt_oss/kernels/attention.py:85,127-135: "query at
 * start_pos+i attends to keys <= start_pos+i").  The new tokens' K/V are
 * already in the pool.  dtype: BF16 for q and out; kv_dtype PA_BF16, or PA_FP8_E4M3FN with
 * k_scale / v_scale [num_blocks, Hkv] (NULL otherwise): the codes are copied into LDS as they are
 * and expanded there, times their block's scale, to bf16.  sinks / sliding_window as for pa_decode, the
 * window counted back from each query token's own position; key tiles outside every row's
 * window are skipped.
 * D = 128 runs the tiled matrix-core kernel (any block_size; the sliding window, the split and
 * q_transform need a power of two >= 16).  D = 64 needs block_size a power of two >= 16 and the
 * workspace: an even Hkv and T > 64 run the same tiled kernel (two adjacent kv
 * heads share its 256-byte rows), anything else launches of pa_verify's kernel over 64 query
 * tokens each.
 * workspace: NULL, or pa_prefill_workspace_bytes(...) bytes (16-byte aligned; 0 = none needed).  With
 * it, a call with too few query tiles to fill the device (one long-context request prefilled in
 * chunks) splits the key tiles of each query tile over up to 16 workgroups and merges their partial
 * results in a second kernel; the result does not depend on the split.
 * max_seq_len: 0, or a host-known upper bound of seq_lens (a hint for the split: a prompt with little or
 * nothing cached in front of it -- bound below 3 T -- is bound by its causal diagonal, whose light query
 * tiles leave the device room anyway, and runs faster unsplit; the table capacity says nothing about
 * that).  Contexts are not clamped to it by the tiled kernel.
 */
size_t pa_prefill_workspace_bytes(int B, int T, int Hq, int Hkv, int D, int block_size, int max_blocks_per_seq);
int pa_prefill(const void* q, const void* k_cache, const void* v_cache,
               const float* k_scale, const float* v_scale,
               const int32_t* block_tables, const int32_t* seq_lens,
               const int32_t* query_lens, void* out,
               int B, int T, int Hq, int Hkv, int D, int block_size,
               int max_blocks_per_seq, int num_blocks, int max_seq_len,
               float scale, int dtype, int kv_dtype, const float* sinks, int sliding_window,
               void* workspace, size_t workspace_bytes, const pa_q_transform* q_transform, void* stream);

/*
 * Block-sparse causal prefill over dense q [B, S, Hq, D], k/v [B, S, Hkv, D]:
 * q block i attends k block j iff j <= i and (i - j < local_blocks or
 * (j + h % vert_stride) % vert_stride == 0), token-causal inside a block.
 * Equals the dense causal prefill of attention.py:112-144 under that mask.
 * `block` must be 64.  dtype: BF16.
 */
int pa_blocksparse_prefill(const void* q, const void* k, const void* v, void* out,
                           int B, int S, int Hq, int Hkv, int D,
                           int block, int local_blocks, int vert_stride,
                           float scale, int dtype, void* stream);

/*
 * Post-attention output projection, the step behind the attention call:
 *   out[m, :] = x[m, :] @ w (+ bias)
 * `output_to_be_reduced = np.matmul(output, o_weight)` of examples/models/qwen3/kernels/attention.py:143-147
 * and, with the bias, examples/models/gpt_oss/kernels/attention.py:155-163 (`+ o_bias`, which the
 * reference adds on rank 0 only; the all-reduce behind it, attention.py:150-154, is the caller's).
 *   x    [M, K] bf16: the attention output [B, T, Hq, D] (or [B, Hq, D]) viewed as [tokens, Hq * D],
 *        padding rows included (they project to bias)
 *   w    [K, N] bf16 row-major, i.e. o_proj.weight transposed as the reference stores it
 *        (examples/models/qwen3/tensor_preparation.py:148-156); a tensor-parallel rank passes its K rows
 *   bias [N] bf16 or NULL;  out [M, N] bf16
 * Products and sums in float32 on the matrix cores, one rounding to bf16 on the way out.
 * K a multiple of 64, N a multiple of 8; dtype PA_BF16.
 */
int pa_o_proj(const void* x, const void* w, const void* bias, void* out, int M, int K, int N, int dtype, void* stream);

/*
 * The same product with scratch memory for calls of few rows (a decode or verify step: M <= 128).  Such a call
 * is bound by streaming `w` once, and one workgroup per 64 output columns leaves most of the device idle; with a
 * workspace, up to four workgroups per column slab take equal ranges of K, leave float32 partial products there,
 * and a second kernel adds them in the order of the ranges, then the bias, and rounds once (results are the same
 * from call to call; they can differ from pa_o_proj's in the last bf16 bit, the sums being taken in another order).
 *   workspace  device memory of pa_o_proj_workspace_bytes(M, K, N) bytes (0: the shape would not use one),
 *              16-byte aligned, owned by the caller, free again when the call's work on `stream` is done;
 *              NULL or too small for two ranges: the call runs as pa_o_proj does.
 * No counterpart in the reference (np.matmul, examples/models/qwen3/kernels/attention.py:147, has no scratch argument).
 */
size_t pa_o_proj_workspace_bytes(int M, int K, int N);
int pa_o_proj_ws(const void* x, const void* w, const void* bias, void* out, void* workspace, size_t workspace_bytes,
                 int M, int K, int N, int dtype, void* stream);

/*
 * One decode step of an attention layer in one call: the cache update, the attention and (optionally) the output
 * projection -- the decode branch of the reference's attention_kernel as a whole
 * (examples/models/qwen3/kernels/attention.py:78-147: QK norm and RoPE, `cache_k[:, query_pos] = xk`, scores,
 * softmax, P V, `np.matmul(output, o_weight)`; with sinks, window and bias the gpt-oss form,
 * examples/models/gpt_oss/kernels/attention.py:85-163), called once per layer and step by the decode loop of
 * examples/models/qwen3/qwen3.py:310-336,372-396.  The result is, bit for bit, that of
 *     pa_qk_norm_rope_kv_write(NULL, xk, xv, NULL, ...)   (pa_kv_write without q_transform)
 *     pa_decode(q, ..., q_transform)
 *     pa_o_proj_ws(attention output, o_weight, o_bias, out, ...)
 * on the same arguments; what the one call adds is that a small step (the fixed-partition decode kernels, bf16 pool)
 * runs as three launches instead of five: the kernel that reaches a sequence's newest token takes its K / V rows
 * from xk / xv (K transformed on the way) and stores them in the pool itself, and the projection merges the
 * sequence's split-K partials while it forms its rows (with sinks or a window the merge stays a launch of its own;
 * a window that fits one partition needs none).  Calls that those kernels do not take (fp8 or fp32 pools, large
 * batches or long contexts) run the separate launches inside.
 *   new_kv    the step's new token per sequence: xk, xv [B, Hkv, D] of the pool's source type (bf16; float32 for
 *             an fp32 pool); query_lens [B]: 1 for a sequence that takes a token this step, 0 for one that does
 *             not (its row of xk / xv is ignored); seq_lens counts the new token, as for pa_kv_write;
 *             k_norm_weight [D] bf16 or NULL: K's RMSNorm weight, used with q_transform's tables and eps (K is
 *             normed and rotated exactly when Q is: q_transform NULL = both go in as given)
 *   k_cache, v_cache, k_scale, v_scale   as for pa_kv_write: updated in place
 *   attn_out  [B, Hq, D] like q, or NULL when out_proj is given and the attention output itself is not wanted
 *   out_proj  NULL (attention only), or o_weight [Hq * D, N] bf16 row-major, o_bias [N] bf16 or NULL, out [B, N]
 *             bf16, N a multiple of 8 (pa_o_proj's conventions)
 *   workspace pa_decode_step_workspace_bytes(...) bytes, 16-byte aligned; the other arguments as for pa_decode
 */
typedef struct pa_new_kv {
  const void* xk;
  const void* xv;
  const void* k_norm_weight;
  const int32_t* query_lens;
} pa_new_kv;
typedef struct pa_out_proj {
  const void* o_weight;
  const void* o_bias;
  void* out;
  int N;
} pa_out_proj;
size_t pa_decode_step_workspace_bytes(int B, int Hq, int Hkv, int D, int block_size, int max_seq_len, int partition_size,
                                      int N, int q_dtype, int kv_dtype);
/*
 * The same for a step of up to PA_VERIFY_MAX_TOKENS tokens per sequence: a speculative verify step of a layer
 * (examples/models/gpt_oss/kernels/attention.py:80-163 with seq_len = K + 1, called from peagle/speculate.py:137-202)
 * in one call, bit for bit pa_qk_norm_rope_kv_write (pa_kv_write without q_transform) + pa_verify + pa_o_proj_ws.
 *   q [B, T, Hq, D] bf16; new_kv: xk, xv [B, T, Hkv, D], query_lens [B] (0 .. T new tokens per sequence; rows
 *   t >= query_lens[b] are padding), k_norm_weight as for pa_decode_step; attn_out [B, T, Hq, D] or NULL;
 *   out_proj->out [B, T, N]; workspace pa_verify_step_workspace_bytes(B, T, Hq, D, N) bytes; max_seq_len as for
 *   pa_verify (with a bound, a small call merges its split-K partials on the projection's load: four launches
 *   instead of five).
 */
size_t pa_verify_step_workspace_bytes(int B, int T, int Hq, int D, int N);
int pa_verify_step(const void* q, const pa_new_kv* new_kv, void* k_cache, void* v_cache, float* k_scale, float* v_scale,
                   const int32_t* block_tables, const int32_t* seq_lens, void* attn_out, const pa_out_proj* out_proj,
                   void* workspace, size_t workspace_bytes,
                   int B, int T, int Hq, int Hkv, int D, int block_size, int max_blocks_per_seq, int num_blocks,
                   int max_seq_len, float scale, int kv_dtype,
                   const float* sinks, int sliding_window, const pa_q_transform* q_transform, void* stream);
int pa_decode_step(const void* q, const pa_new_kv* new_kv, void* k_cache, void* v_cache, float* k_scale, float* v_scale,
                   const int32_t* block_tables, const int32_t* seq_lens, void* attn_out, const pa_out_proj* out_proj,
                   void* workspace, size_t workspace_bytes,
                   int B, int Hq, int Hkv, int D, int block_size, int max_blocks_per_seq, int num_blocks, int max_seq_len,
                   float scale, int partition_size, int q_dtype, int kv_dtype,
                   const float* sinks, int sliding_window, const pa_q_transform* q_transform, void* stream);

/*
 * Test hook: materialise the block-table gather.  out [B, max_seq_len, Hkv, D]
 * (elem_bytes per element, bits copied verbatim); rows >= seq_lens[b] are zero.
 * Bit-exact counterpart of np.take(pool, table, axis=0)
 * (nkipy/src/nkipy/core/tensor.py:575-640).
 */
int pa_gather_kv(const void* cache, const int32_t* block_tables, const int32_t* seq_lens,
                 void* out, int B, int Hkv, int D, int block_size,
                 int max_blocks_per_seq, int num_blocks, int max_seq_len,
                 int elem_bytes, void* stream);

/* Paged KV-cache write, to be run before the attention call of the same step: token
 * t < query_lens[b] of sequence b sits at position seq_lens[b] - query_lens[b] + t and its
 * K/V rows go to pool row (block_tables[b, pos / block_size], pos % block_size).  Replaces
 * the reference's dense cache update `cache_k[:, query_pos] = xk` with query_pos =
 * start_pos + arange(seq_len) (examples/models/gpt_oss/kernels/attention.py:85,92-100;
 * examples/models/qwen3/kernels/attention.py:100-106); the pool is updated in place like the
 * reference's aliased cache tensors (examples/models/qwen3/qwen3.py:289-301).
 *   k_new, v_new  [B, T, Hkv, D], bf16 (float32 when kv_dtype is PA_F32); rows t >= query_lens[b] are padding
 *   k/v_cache     [num_blocks, block_size, Hkv, D] of kv_dtype
 *   k/v_scale     [num_blocks, Hkv] float32, PA_FP8_E4M3FN only (NULL otherwise): kept as the running
 *                 maximum of absmax / 448 over the tokens a block holds; when a write raises it the
 *                 block's earlier rows are re-encoded; a block whose first row is written is fresh.
 *                 The fp8 part has no counterpart in the reference.
 * Blocks being written must belong to one sequence only (shared prefix blocks are read-only).
 * Sequences with query_lens[b] <= 0 or seq_lens[b] < query_lens[b], and table entries outside
 * the pool, write nothing. */
int pa_kv_write(const void* k_new, const void* v_new, void* k_cache, void* v_cache,
                float* k_scale, float* v_scale,
                const int32_t* block_tables, const int32_t* seq_lens, const int32_t* query_lens,
                int B, int T, int Hkv, int D, int block_size, int max_blocks_per_seq, int num_blocks,
                int kv_dtype, void* stream);

/* The reference's pre-attention step fused with the KV write: QK RMSNorm
 * (examples/models/qwen3/kernels/rmsnorm.py:4-21, applied at qwen3/kernels/attention.py:78-80),
 * RoPE at the tokens' absolute positions start_pos + t, start_pos = seq_lens[b] -
 * query_lens[b] (rope.py:23-48; attention.py:83-97; gpt_oss/kernels/attention.py:85-90), then
 * pa_kv_write of the rotated K and of V.  Two launches: Q rows, then the K/V scatter; with xq
 * and q_out both NULL only the second (for callers that hand the Q part to the attention call
 * as a pa_q_transform).
 *   xq [B, T, Hq, D], xk, xv [B, T, Hkv, D]  bf16; q_out [B, T, Hq, D] bf16 (may be xq); rows
 *                 t >= query_lens[b] of q_out are zero
 *   q_norm_weight, k_norm_weight [D] bf16, or NULL for no norm on that tensor
 *   rope_cos, rope_sin [rope_max_pos, D/2] bf16 (rope.py:4-20 cast to bf16); positions past the
 *                 table are clamped to its last row
 * Arithmetic as the reference's bf16 tensors give it: the norm in float32 rounded once to bf16,
 * every product and sum of the rotation rounded to bf16.  D in {64, 128, 256};
 * kv_dtype PA_BF16 or PA_FP8_E4M3FN (then scales as in pa_kv_write). */
int pa_qk_norm_rope_kv_write(const void* xq, const void* xk, const void* xv, void* q_out,
                             const void* q_norm_weight, const void* k_norm_weight, float norm_eps,
                             const void* rope_cos, const void* rope_sin, int rope_max_pos,
                             void* k_cache, void* v_cache, float* k_scale, float* v_scale,
                             const int32_t* block_tables, const int32_t* seq_lens, const int32_t* query_lens,
                             int B, int T, int Hq, int Hkv, int D, int block_size, int max_blocks_per_seq,
                             int num_blocks, int kv_dtype, void* stream);

/* Debug switches (process-wide; tests only).  They work only when PA_ENABLE_DEBUG=1 was in the
 * environment at the library's first use; otherwise every call is refused with an argument error
 * and changes nothing, so a server that links the library cannot have its kernels rerouted.  key 0: decode kernel choice
 * (0 = automatic, 1 = scalar-ALU kernel, 2 = MFMA kernel with fixed partitions,
 * 3 = MFMA kernel with the balanced schedule); key 1: waves per workgroup of the
 * fixed-partition MFMA kernel (0 = default); key 2: its grid order (1 = kv head
 * fastest, the default; 0 = partition fastest); key 3: prefill kernel choice (0 =
 * automatic, 1 = register-staged kernel, 4 / 8 = asynchronous-copy kernel with that
 * many wavefronts per workgroup and one q head per workgroup, 5 = the same with the rows of a
 * workgroup packed over the q heads of a kv head, which is what short chunks get by default); key 4:
 * per-tile barrier that keeps the kv-head wavefronts of a balanced decode workgroup on
 * the same tile (1 = automatic, the default: on for bf16 pools, off for fp8 pools; 0 = never; 2 = always); key 5: query rows per wavefront of pa_verify (0 =
 * automatic, 16 or 32 = forced); key 6: split form of pa_prefill (1 = when useful, the default; 0 = never; 2-16 = that many shares);
 * key 7: query tokens from which pa_prefill at head dim 64 takes the tiled kernel (0 = the default, 65);
 * key 3 value 6: one q head per wave at head dim 64; key 8: pa_o_proj takes 256 x 256 tiles
 * also where it would take 128 x 128 ones (1 = on); key 9: the longest length bound (tokens) up to which a small
 * pa_decode call runs as one partition per sequence on eight wavefronts (default 1024; 0 = never); key 10: what
 * pa_decode_step lets ride on its decode and projection launches (0 = the new row and the merge, the default; 1 = neither:
 * the separate launches; 2 = the new row only; 3 = the merge only); key 11: tokens per partition that the smallest
 * fixed-partition decode calls take instead of the caller's larger ones (default 256; 0 = the caller's always);
 * key 12: the most (sequence, kv head) pairs a small call may have (0 = the rule described at pa_decode).
 * key 13: 0 = partitions of small calls counted in tokens at head dim 64 and on fp8 pools too (1, the default: see pa_decode). */
int pa_debug_set(int key, int value);

/* Kernel timing for benchmarks: when enabled, every launch of the main kernel
 * of pa_decode / pa_prefill / pa_blocksparse_prefill / pa_o_proj is bracketed by HIP events
 * on its own stream.  pa_profile_collect synchronises those events, writes up
 * to `cap` durations (milliseconds, oldest first) and clears the list; returns
 * the number written.  The counterpart of the reference's device-side timing,
 * spike/src/spike/spike_model.py:290-363. */
int pa_profile_enable(int on);
int pa_profile_collect(float* ms, int cap);
/* Launches a kernel that does nothing on `stream`, bracketed like the main kernels when timing is enabled: what
 * pa_profile_collect then reports for it is the part of every such figure that is not kernel time (the events
 * are stamped around the dispatch; a kernel trace reports first wave to last). */
int pa_profile_empty_launch(void* stream);

#ifdef __cplusplus
}
#endif
#endif /* PAGED_ATTN_H_ */
