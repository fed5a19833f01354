/*
 * muxserve_attn.h - C ABI of the device half of the hot path (libmuxattn.so,
 * HIP, gfx950): KV-cache write, paged decode attention and causal prefill
 * attention over the unified head-granular KV block pool, plus CU-masked
 * stream creation for prefill/decode colocation.
 *
 * What these replace.  In the reference the attention layer is constructed at
 * muxserve/flexserver/models/llama.py:138-147 and invoked at
 * muxserve/flexserver/models/llama.py:159-161 as
 *     attn(positions, q, k, v, k_cache, v_cache, input_metadata, cache_event)
 * with k_cache/v_cache the WHOLE pool (models/llama.py:276-288,
 * pipeworker.py:93-106) and the index tensors built at
 * muxserve/flexserver/llm_runtime.py:300-334.  The arithmetic behind that call
 * lives in the external MuxServe-vLLM fork (cache_ops.reshape_and_cache,
 * attention_ops.paged_attention, the prefill attention); the entry points
 * below are what a binding for that call would link instead.
 *
 * Pool layout (muxserve/flexstore/manager.py:456-468, 485-492), one entry per
 * (token block, layer, head) - "head-block":
 *     K pool  [num_blocks, D/x, block_size, x]   x = 16 / sizeof(elem) = 8
 *     V pool  [num_blocks, D,   block_size]
 * D (head size) is 128 (manager.py:337).  A slot is block_id*block_size+offset
 * (csrc/batch_scheduler.h:50-53).
 *
 * Conventions: every pointer is a DEVICE pointer owned by the caller unless
 * noted; nothing is retained past the call; all work is enqueued on `stream`
 * (a hipStream_t passed as void*; NULL = the default stream) and the call
 * returns without synchronising.  Return value: 0 on success, a negative
 * MUXA_E* code on a rejected argument; no exceptions cross the boundary.
 * Shapes are validated on the host before any launch.  A call with nothing to
 * do (no tokens, sequences, prompts or rows) returns MUXA_OK without a launch,
 * and the data pointers of such a call may be NULL.
 */
#ifndef MUXSERVE_ATTN_H
#define MUXSERVE_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MUXA_OK 0
#define MUXA_EINVAL (-1)      /* null pointer / negative size / bad stride     */
#define MUXA_EUNSUPPORTED (-2)/* head size != 128, block size not 8/16/32 ...  */
#define MUXA_EWORKSPACE (-3)  /* workspace missing or too small                */
#define MUXA_EHIP (-4)        /* a HIP runtime call failed (see mux_last_hip_error) */
#define MUXA_ESCRATCH_LIMIT (-5) /* the call needs more scratch than the library's fixed
                                    static array holds (mux_multi_decode_noalloc only)  */

#define MUXA_DTYPE_F16 0
#define MUXA_DTYPE_BF16 1

#define MUXA_MAX_DECODE_ITEMS 8
/* Leading region of a decode workspace: int32 arrival counters, one per
 * (sequence, group of query heads sharing a wave) over all items of a call. */
#define MUXA_DECODE_COUNTER_BYTES (1u << 20)

/* Library version (major*10000 + minor*100 + patch). */
int32_t mux_attn_version(void);
/* hipError_t of the last failing HIP call made by this library on the calling
 * thread (0 if none). */
int32_t mux_last_hip_error(void);

/* ---- KV-cache write ------------------------------------------------------
 * Stands in for cache_ops.reshape_and_cache as called by the attention layer
 * behind models/llama.py:159-161: for token t, kv-head h, dim d
 *     slot = slot_mapping[t, layer, h]; b = slot / block_size; o = slot % block_size
 *     K_pool[b, d/8, o, d%8] = k[t, h, d];   V_pool[b, d, o] = v[t, h, d]
 * k, v: [num_tokens, Hkv*D] with row stride kv_row_stride (elements; q,k,v are
 * column slices of one qkv row, models/llama.py:157-158).  slot_mapping: int64
 * [num_tokens, L, Hkv] as built at llm_runtime.py:301-302.  Slots < 0 are
 * skipped.  Bit-exact byte movement; no arithmetic. */
int32_t mux_reshape_and_cache(const void *k, const void *v, int64_t kv_row_stride,
                              void *k_pool, void *v_pool, int64_t num_pool_blocks,
                              const int64_t *slot_mapping, int32_t layer, int32_t num_layers,
                              int32_t num_tokens, int32_t num_kv_heads, int32_t head_size,
                              int32_t block_size, int32_t dtype, void *stream);

/* ---- Paged decode attention ---------------------------------------------
 * One model's decode step for one layer; stands in for
 * attention_ops.paged_attention behind models/llama.py:159-161.  For sequence
 * s and query head hq (kv head hk = hq / (Hq/Hkv)):
 *     out[s,hq,:] = softmax(scale * q[s,hq,:] . K[0:ctx_s]) . V[0:ctx_s]
 * with K/V gathered block by block through block_tables[layer, s, hk, :].
 * fp16/bf16 storage, fp32 accumulation.
 *
 * q, out: [>=num_seqs, Hq*D], row strides in elements.
 * block_tables: int32 [L, num_seqs, Hkv, max_blocks] (llm_runtime.py:327);
 * only the first ceil(ctx/block_size) entries of a row are read.
 * context_lens: int32 [num_seqs].  max_context_len: host-side upper bound on
 * context_lens (InputMetadata.max_context_len, pipeworker.py:81-90); it sizes
 * the grid, device values above it are clamped.
 * total_context_len: optional host-side upper bound on the sum of
 * context_lens (the serving loop has them on the host before the copy,
 * llm_runtime.py:311-326); it only tightens the grid of a launch whose units
 * are enumerated on the device, 0 = unknown.  A bound that turns out too small
 * costs time, not results: the units it leaves without a workgroup of their own
 * are run, one after the other, by the workgroups of the last unit that has
 * one, so every output is still written and the workspace's arrival counters
 * still return to zero.  With context_lens_host the enumeration is exact and
 * this field is not used.
 * context_lens_host: optional HOST copy of context_lens [num_seqs] (same
 * place in the serving loop, llm_runtime.py:311-326: the lengths are a host
 * list before they become a tensor).  When every model of a launch comes with
 * one and the batch is small (at most 384 (sequence, partition) pairs), the
 * work list is enumerated on the host and travels in the kernel argument, so a
 * workgroup reaches its K/V loads one dependent memory latency sooner.  The
 * launch then follows the HOST values (clamped to max_context_len) and does not
 * read the device tensor: they must be equal.  The values are fixed when the
 * call is made, so leave this NULL for launches recorded into a HIP graph that
 * is replayed with changed lengths.  NULL = enumerate on the device.
 * partition_size: tokens per split of a context (multiple of 64), 0 = choose:
 * 256, or 1024 for a large launch (at least 1.5 M tokens x head groups over
 * its models, by total_context_len or by num_seqs * max_context_len / 2 without
 * it), or 512 when contexts exceed 4096 tokens; when every model of the launch
 * has four or more query heads per kv head: that sum / 768 (a workgroup slot's
 * share of the launch), rounded up to a multiple of 256.  The workspace size
 * reported for 0 covers every choice, so it may differ from launch to launch.
 * workspace: scratch for the partial results of split contexts and, for
 * batches of more than 256 sequences, the table that maps workgroups to
 * (sequence, unit) pairs (written by a small kernel launched ahead of
 * the attention kernel on the same stream; a row for every pair the shapes
 * allow, num_seqs * ceil(max_context_len / partition)); at least
 * mux_paged_decode_workspace_bytes(...) bytes, 16-byte aligned; may be NULL
 * when that is 0.  Its first MUXA_DECODE_COUNTER_BYTES bytes are arrival
 * counters that must be ZERO when a launch begins: zero them once with
 * mux_paged_decode_workspace_init (or any fill) before first use; every
 * completed launch leaves them zero again.  Launches that share a workspace
 * must not overlap. */
typedef struct MuxDecodeItem {
  void *out;
  const void *q;
  int64_t out_row_stride;
  int64_t q_row_stride;
  const int32_t *block_tables;   /* base of the [L, B, Hkv, max_blocks] tensor */
  const int32_t *context_lens;
  int64_t total_context_len;     /* host-side upper bound on sum(context_lens); 0 = unknown */
  int32_t layer;
  int32_t num_layers;
  int32_t num_seqs;
  int32_t num_q_heads;
  int32_t num_kv_heads;
  int32_t max_blocks;
  int32_t max_context_len;
  float scale;
  const int32_t *context_lens_host; /* optional HOST copy of context_lens, or NULL (see above) */
} MuxDecodeItem;

size_t mux_paged_decode_workspace_bytes(const MuxDecodeItem *items, int32_t n_items,
                                        int32_t partition_size);

/* How many (sequence, unit) pairs a mux_multi_decode call with these items
 * would enumerate on the host and carry in the kernel argument (its first
 * launch group); 0: the units of that call are enumerated on the device (no
 * context_lens_host, or more pairs than the argument holds).  Host arithmetic
 * only, no device needed.  No reference counterpart. */
int32_t mux_paged_decode_host_pairs(const MuxDecodeItem *items, int32_t n_items, int32_t partition_size);

/* Zero-fills the counter region of a decode workspace (a fill kernel on
 * `stream`, safe to capture). */
int32_t mux_paged_decode_workspace_init(void *workspace, size_t workspace_bytes, void *stream);

/* Fused launch over up to MUXA_MAX_DECODE_ITEMS models that share the pool,
 * head size, block size and dtype ("mixed multi-LLM decode": one grid covers
 * every model's (sequence, head, partition) work).  `items` is a HOST array. */
int32_t mux_multi_decode(const MuxDecodeItem *items, int32_t n_items,
                         const void *k_pool, const void *v_pool, int64_t num_pool_blocks,
                         int32_t head_size, int32_t block_size, int32_t dtype,
                         int32_t partition_size, void *workspace, size_t workspace_bytes,
                         void *stream);

/* mux_multi_decode for callers that cannot allocate.  No counterpart in the
 * reference: it exists for callers that must not call hipMalloc or any
 * allocating routine - code under HIP graph capture, tight serving loops,
 * harnesses that forbid it - and that have no workspace of their own to pass.
 * Same arguments, results and kernels as mux_multi_decode, except that the
 * scratch (arrival counters, partial results of split contexts, the pair table
 * of large batches) is a static device array of MUXA_STATIC_SCRATCH_BYTES inside
 * the library: one copy per GPU the library runs on, held until the process
 * ends.  The call allocates and frees nothing, records no memset (its arrival
 * counters are cleared by a small fill kernel on `stream` ahead of the
 * attention kernel) and never synchronises.  A call whose scratch need
 * (mux_paged_decode_workspace_bytes) exceeds MUXA_STATIC_SCRATCH_BYTES is
 * refused with MUXA_ESCRATCH_LIMIT before anything is launched.  Every call on
 * a GPU shares that GPU's array: calls that overlap in time on one GPU (two
 * streams, two threads) race on it and must be serialised by the caller. */
#define MUXA_STATIC_SCRATCH_BYTES (32u << 20)
size_t mux_multi_decode_noalloc_max_bytes(void);
int32_t mux_multi_decode_noalloc(const MuxDecodeItem *items, int32_t n_items,
                                 const void *k_pool, const void *v_pool, int64_t num_pool_blocks,
                                 int32_t head_size, int32_t block_size, int32_t dtype,
                                 int32_t partition_size, void *stream);

/* Single-model convenience wrapper around mux_multi_decode. */
int32_t mux_paged_decode(void *out, int64_t out_row_stride, const void *q, int64_t q_row_stride,
                         const void *k_pool, const void *v_pool, int64_t num_pool_blocks,
                         const int32_t *block_tables, const int32_t *context_lens,
                         int32_t layer, int32_t num_layers, int32_t num_seqs,
                         int32_t num_q_heads, int32_t num_kv_heads, int32_t head_size,
                         int32_t block_size, int32_t max_blocks, int32_t max_context_len,
                         float scale, int32_t dtype, int32_t partition_size,
                         void *workspace, size_t workspace_bytes, void *stream);

/* ---- Causal prefill attention -------------------------------------------
 * Stands in for the prompt branch of the attention layer behind
 * models/llama.py:159-161: per prompt p (tokens cu_seqlens[p]..cu_seqlens[p+1])
 *     out[t,hq,:] = softmax(scale * q[t,hq,:] . k[<=t,hk,:]) . v[<=t,hk,:]
 * on the fresh q,k,v (the pool is not read).  cu_seqlens: DEVICE int32
 * [num_prompts+1] prefix sums of InputMetadata.prompt_lens; max_prompt_len is
 * a host-side upper bound that sizes the grid.  prompt_order: optional DEVICE
 * int32 [num_prompts], a permutation of the prompts - the order in which their
 * workgroups are started (the caller knows the lengths on the host; longest
 * first keeps the longest prompt off the end of the launch); NULL: as packed.
 * prompt_lens_host: optional HOST int32 [num_prompts], the prompt lengths the
 * caller holds on the host anyway (InputMetadata.prompt_lens,
 * pipeworker.py:81-90; each <= max_prompt_len).  With them the launch holds
 * only the query tiles that exist, the heaviest of the whole batch first, and
 * prompt_order is not used; batches of more than 768 query tiles of 128 rows
 * fall back to the grid sized by max_prompt_len.  The device-side cu_seqlens
 * stay authoritative for addresses and lengths (a host length shorter than the
 * device's only leaves that prompt's further query tiles unstarted).  With
 * consistent lengths the results depend on neither. */
int32_t mux_prefill_causal(void *out, int64_t out_row_stride,
                           const void *q, int64_t q_row_stride,
                           const void *k, const void *v, int64_t kv_row_stride,
                           const int32_t *cu_seqlens, const int32_t *prompt_order,
                           const int32_t *prompt_lens_host, int32_t num_prompts,
                           int32_t max_prompt_len, int32_t num_q_heads, int32_t num_kv_heads,
                           int32_t head_size, float scale, int32_t dtype, void *stream);

/* Causal prefill attention of up to MUXA_MAX_DECODE_ITEMS colocated models in
 * ONE launch (the prompt-side counterpart of mux_multi_decode; the reference
 * runs one attention call per model, models/llama.py:159-161): models of the
 * same dtype whose prompts are prefilled in the same step share the grid, the
 * heaviest query tiles of all of them first, so that the short prompts of one
 * model fill the compute units that the long prompts of another leave idle at
 * the end of its launch.  Field meanings are those of mux_prefill_causal.  The
 * shared grid needs prompt_lens_host for every item and at most 768 query tiles
 * of 128 rows in all; otherwise the call falls back to one launch per model.
 * Results are bit-identical to the per-model calls.  `items` is a HOST array. */
typedef struct MuxPrefillItem {
  void *out;
  int64_t out_row_stride;
  const void *q;
  int64_t q_row_stride;
  const void *k;
  const void *v;
  int64_t kv_row_stride;
  const int32_t *cu_seqlens;         /* DEVICE int32 [num_prompts + 1] */
  const int32_t *prompt_lens_host;   /* HOST int32 [num_prompts] */
  int32_t num_prompts;
  int32_t max_prompt_len;
  int32_t num_q_heads;
  int32_t num_kv_heads;
  float scale;
} MuxPrefillItem;

int32_t mux_multi_prefill_causal(const MuxPrefillItem *items, int32_t n_items, int32_t head_size,
                                 int32_t dtype, void *stream);

/* ---- Rotary position embedding --------------------------------------------
 * The attention layer of the reference is PagedAttentionWithRoPE constructed
 * with rotary_dim = head_dim and base = rope_theta
 * (muxserve/flexserver/models/llama.py:138-147): NeoX-style rotation of q and k
 * in place, before the cache write.  positions: int64 [>= num_tokens]
 * (llm_runtime.py:325).  cos_sin: DEVICE fp32 [max_position, rotary_dim], row p
 * = [cos(p*f_0..f_{r/2-1}) | sin(...)], f_i = base^(-2i/rotary_dim).  fp32
 * arithmetic, one rounding to the storage type. */
int32_t mux_rotary_neox(const int64_t *positions, void *q, int64_t q_row_stride, void *k,
                        int64_t k_row_stride, const float *cos_sin, int32_t max_position,
                        int32_t rotary_dim, int32_t num_tokens, int32_t num_q_heads,
                        int32_t num_kv_heads, int32_t head_size, int32_t dtype, void *stream);

/* The same rotation fused with the cache write (the two steps that open the
 * attention layer's forward, models/llama.py:159-161): q and k of the first
 * num_tokens rows are rotated in place and the rotated k, with v, is scattered
 * through slot_mapping as by mux_reshape_and_cache - one launch and one pass
 * over k.  Rows without a slot (< 0) are still rotated.  rotary_dim must be
 * head_size (128), q/k/v 16-byte aligned with row strides that are multiples
 * of 8; q may be NULL (k only). */
int32_t mux_rope_reshape_and_cache(const int64_t *positions, void *q, int64_t q_row_stride, void *k,
                                   const void *v, int64_t kv_row_stride, const float *cos_sin,
                                   int32_t max_position, int32_t rotary_dim, void *k_pool, void *v_pool,
                                   int64_t num_pool_blocks, const int64_t *slot_mapping, int32_t layer,
                                   int32_t num_layers, int32_t num_tokens, int32_t num_q_heads,
                                   int32_t num_kv_heads, int32_t head_size, int32_t block_size,
                                   int32_t dtype, void *stream);

/* The cache writes of one step of up to MUXA_MAX_DECODE_ITEMS colocated models
 * in ONE launch (the write-side counterpart of mux_multi_decode): the reference
 * issues one reshape_and_cache per model and layer (models/llama.py:159-161);
 * models that share the pool, block size and dtype and run the same step can
 * share the grid, which removes the per-launch latency that dominates a decode
 * step's write of a few dozen tokens.  Field meanings are those of
 * mux_rope_reshape_and_cache / mux_reshape_and_cache; either every item rotates
 * (positions != NULL: q and k rotated in place, rotated k scattered) or none
 * does (positions == NULL: plain scatter; q, cos_sin, rotary fields unused).
 * Result: bit-identical to the per-model calls.  `items` is a HOST array. */
typedef struct MuxCacheWriteItem {
  const int64_t *positions;      /* [num_tokens] or NULL (no rotation) */
  void *q;                       /* rotated in place; may be NULL */
  int64_t q_row_stride;
  void *k;                       /* rotated in place when positions != NULL */
  const void *v;
  int64_t kv_row_stride;
  const float *cos_sin;          /* [max_position, rotary_dim] = [cos | sin] */
  const int64_t *slot_mapping;   /* base of the int64 [num_tokens, L, Hkv] tensor */
  int32_t max_position;
  int32_t rotary_dim;
  int32_t layer;
  int32_t num_layers;
  int32_t num_tokens;
  int32_t num_q_heads;
  int32_t num_kv_heads;
} MuxCacheWriteItem;

int32_t mux_multi_rope_reshape_and_cache(const MuxCacheWriteItem *items, int32_t n_items, void *k_pool,
                                         void *v_pool, int64_t num_pool_blocks, int32_t head_size,
                                         int32_t block_size, int32_t dtype, void *stream);

/* ---- Operators of the model step around the attention layer ---------------
 * The reference's LLaMA layer takes RMSNorm and SiluAndMul from its vLLM fork
 * (muxserve/flexserver/models/llama.py:35-36; used at :79-81, 200-203, 217-232,
 * 257, 283) and samples with its own GreedySampler
 * (muxserve/flexserver/sampler.py:9-35).  Device pointers, row strides in
 * elements; rows and weights 16-byte aligned, sizes multiples of 8.
 *
 * mux_rms_norm: out[t,:] = T(x[t,:] * rsqrt(mean(x[t,:]^2) + eps)) * weight,
 * statistics in fp32, the product with the weight taken in the storage type T. */
int32_t mux_rms_norm(void *out, int64_t out_row_stride, const void *x, int64_t x_row_stride,
                     const void *weight, float eps, int32_t num_tokens, int32_t hidden_size,
                     int32_t dtype, void *stream);

/* mux_silu_and_mul: x [num_tokens, 2 d] = [gate | up] ->
 * out[t,:] = T(gate / (1 + exp(-gate))) * up, the product taken in T. */
int32_t mux_silu_and_mul(void *out, int64_t out_row_stride, const void *x, int64_t x_row_stride,
                         int32_t num_tokens, int32_t d, int32_t dtype, void *stream);

/* mux_greedy_sample: GreedySampler.forward (sampler.py:15-35) without
 * materialising the logits.  For sampled row r < num_rows:
 *     h = hidden_states[row_index ? row_index[r] : r]     (entries clamped to num_hidden_rows - 1)
 *     next_tokens[r] = argmax_{v < vocab_size} T(h . embedding[v,:])
 * (fp32 accumulation, each logit rounded to T before the comparison as the
 * reference's fp16 logits are; ties go to the lowest id).  On a prompt step
 * row_index holds cumsum(prompt_lens) - 1 (sampler.py:18-24), on a decode step
 * it is NULL.  embedding: [embedding_rows >= vocab_size, hidden_size], the
 * lm_head weight (models/llama.py:317-323); hidden_size a multiple of 256.
 * next_tokens: DEVICE int64 [num_rows].  workspace: DEVICE,
 * mux_greedy_sample_workspace_bytes(vocab_size) bytes, 16-byte aligned, its
 * first 256 bytes (an arrival counter) zeroed once before the first use
 * (mux_greedy_sample_workspace_init, or any zero fill); every call leaves them
 * zeroed again.  Calls that share a workspace must
 * not overlap.  Nothing is allocated and no memset is recorded, so a call can
 * be captured into a HIP graph. */
size_t mux_greedy_sample_workspace_bytes(int32_t vocab_size);
int32_t mux_greedy_sample_workspace_init(void *workspace, size_t workspace_bytes, void *stream);
int32_t mux_greedy_sample(int64_t *next_tokens, const void *hidden_states, int64_t hidden_row_stride,
                          int32_t num_hidden_rows, const int32_t *row_index, int32_t num_rows,
                          const void *embedding,
                          int64_t embedding_row_stride, int32_t embedding_rows, int32_t vocab_size,
                          int32_t hidden_size, int32_t dtype, void *workspace, size_t workspace_bytes,
                          void *stream);

/* ---- Step inputs built on the device ---------------------------------------
 * No reference counterpart (the reference builds slot_mapping and the block
 * table on the host, csrc/batch_scheduler.cpp:131-169, and uploads them,
 * muxserve/flexserver/llm_runtime.py:301-327).  Companion of
 * mux_sched_get_batch_compact (muxserve_host.h): mirror is a DEVICE int32
 * [max_rows, max_blocks_per_seq, L, H] array the caller allocates once and
 * only this call writes; desc (DEVICE int32 [num_seqs, 8]) and block_info
 * (DEVICE copy of the allocator's reply, n_block_info ints) are the step's
 * upload.  In stream order: the reply's ids are appended to the mirror rows,
 * slot_mapping int64 [num_tokens, L, H] is written, and, when
 * max_blocks_out > 0 (decode step), block_tables int32
 * [L, num_seqs, H, max_blocks_out] - both bit-identical to what
 * mux_sched_get_batch + permute(2,0,3,1) give on the entries the reference
 * defines (others 0).  max_new_blocks: host-side upper bound of desc[.][3]
 * (sizes the copy grid).  Descriptors that do not fit the mirror or the reply
 * are skipped. */
int32_t mux_build_step_inputs(int32_t *mirror, int32_t max_rows, int32_t max_blocks_per_seq,
                              int32_t num_layers, int32_t num_heads, int32_t block_size,
                              const int32_t *desc, int32_t num_seqs, const int32_t *block_info,
                              int64_t n_block_info, int32_t max_new_blocks, int32_t num_tokens,
                              int64_t *slot_mapping, int32_t *block_tables, int32_t max_blocks_out,
                              void *stream);

/* ---- CU-masked streams ---------------------------------------------------
 * Replacement for the reference's per-process MPS share
 * (CUDA_MPS_ACTIVE_THREAD_PERCENTAGE, muxserve/muxsched/launcher.py:54-61):
 * a stream whose kernels run only on the compute units selected by bits
 * [lo_percent*N/100, hi_percent*N/100) of the device's N-bit CU mask.  The
 * kernel driver deals consecutive mask bits round-robin over XCDs and shader
 * engines, so a contiguous bit range is a share spread evenly over the chip,
 * and two disjoint ranges never share a CU.  *stream_out receives a
 * hipStream_t; *num_cus_out (optional) the number of CUs enabled. */
int32_t mux_stream_create_cu_range(void **stream_out, int32_t lo_percent, int32_t hi_percent,
                                   int32_t *num_cus_out);
/* The same for a SET of tenths of the GPU: the reference's scheduler hands out
 * compute in 10 parts (SMResource, muxserve/muxsched/resource.py:35-81) and a
 * job holds whichever parts were free - not a contiguous range.  Bit p of
 * part_mask (p = 0..9) enables mask bits [N*p/10, N*(p+1)/10) of the device's N
 * compute units.  Consecutive mask bits go round-robin over the accelerator
 * dies first and the shader engines next (measured on MI355X with a kernel that
 * records XCC_ID / HW_ID per workgroup), so every part takes 3 or 4 compute
 * units from each of the 8 dies, two part sets without a common part never share
 * a compute unit, and no die is left without one (the driver refuses such
 * masks).  mux_cu_parts_mask builds the mask words on the host without a GPU
 * (words: n_words >= ceil(num_cus / 32) uint32) and returns the number of
 * compute units enabled, or a negative code. */
#define MUXA_CU_PARTS 10
int32_t mux_cu_parts_mask(uint32_t part_mask, int32_t num_cus, uint32_t *words, int32_t n_words);
int32_t mux_stream_create_cu_parts(void **stream_out, uint32_t part_mask, int32_t *num_cus_out);
int32_t mux_stream_destroy(void *stream);
/* Device facts used by the mask builder: out = [num_cus, num_xcds]. */
int32_t mux_device_cu_info(int32_t out[2]);

#ifdef __cplusplus
}
#endif
#endif /* MUXSERVE_ATTN_H */
