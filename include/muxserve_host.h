/*
 * muxserve_host.h - C ABI of the host-side half of the hot path: the
 * head-granular KV block allocator and the per-step block-table / slot-mapping
 * builder.  Pure host code (libmuxhost.so has no HIP dependency), so the
 * allocator can live in a process that never touches the GPU.
 *
 * Every entry point replaces one method of the reference's two pybind11
 * modules; the citation on each names the reference lines it stands in for.
 * Conventions: all pointers are host pointers owned by the caller, nothing is
 * retained past the call, functions return >= 0 on success and a negative
 * MUX_E* code on a rejected argument (where the reference would assert, read
 * out of bounds or dereference a null request).  Objects are not thread-safe,
 * like the reference's (one serving loop per object).
 */
#ifndef MUXSERVE_HOST_H
#define MUXSERVE_HOST_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MUX_OK 0
#define MUX_EINVAL (-1)   /* malformed argument (null pointer, negative size) */
#define MUX_ENOSPC (-2)   /* caller buffer too small / pool exhausted         */
#define MUX_ENOENT (-3)   /* unknown request id                              */
#define MUX_ESTATE (-4)   /* call sequence violates the step protocol        */

typedef struct MuxKVStorage MuxKVStorage;
typedef struct MuxBatchScheduler MuxBatchScheduler;

/* ---- KVStorage: csrc/memory_manager.h:8-28 ------------------------------ */

/* KVStorage::KVStorage(int numBlocks), csrc/memory_manager.cpp:4-10.
 * Free list starts as 0..num_blocks-1.  Returns NULL if num_blocks < 0. */
MuxKVStorage *mux_kvstorage_create(int32_t num_blocks);
void mux_kvstorage_destroy(MuxKVStorage *s);

/* KVStorage::allocate, csrc/memory_manager.cpp:12-23: pops `size` ids from
 * the back of the free list into out[0..size).  MUX_ENOSPC if fewer are free
 * (the reference pops an empty vector). Returns size. */
int32_t mux_kvstorage_allocate(MuxKVStorage *s, int32_t size, int32_t *out);

/* Upper bound on the length of an allocate_batch reply for this request
 * vector: 1 + sum(info[3i+1]) * num_layers * num_heads. */
int64_t mux_kvstorage_allocate_batch_bound(const int32_t *info, int32_t n_info,
                                           int32_t num_layers, int32_t num_heads);

/* KVStorage::allocateBatch, csrc/memory_manager.cpp:25-142.  info is
 * int32[n_info] = rows (request id, token blocks wanted, prompt-allocated
 * flag).  Writes [preemptIdx, ids...] to out and returns its length
 * (1 when preemptIdx <= 0).  MUX_ENOSPC if out_cap is too small.  The blocks
 * are keyed by request id alone, whatever the (num_layers, num_heads) of the
 * call: callers that share one KVStorage - the models of a FlexStore - must
 * hand out ids that are unique among them.  A row that asks for fewer blocks
 * than its id already holds (the sign of two callers using one id) returns
 * MUX_ESTATE where the reference asserts or copies from before the list. */
int64_t mux_kvstorage_allocate_batch(MuxKVStorage *s, const int32_t *info, int32_t n_info,
                                     int32_t num_layers, int32_t num_heads,
                                     int32_t *out, int64_t out_cap);

/* KVStorage::freeBatch, csrc/memory_manager.cpp:144-157.  Returns the number
 * of head-blocks returned to the free list. */
int64_t mux_kvstorage_free_batch(MuxKVStorage *s, const int32_t *request_ids, int32_t n);

/* KVStorage::newBlocksAllocated, csrc/memory_manager.h:17. */
int32_t mux_kvstorage_new_blocks_allocated(const MuxKVStorage *s);

/* Introspection with no reference counterpart (the reference exposes the
 * members freeBlocks_/allocatedBlocks_ only to C++): used by invariants tests. */
int64_t mux_kvstorage_num_free(const MuxKVStorage *s);
int64_t mux_kvstorage_num_held(const MuxKVStorage *s, int32_t request_id);

/* ---- BatchScheduler: csrc/batch_scheduler.h:70-106 ---------------------- */

/* BatchScheduler::BatchScheduler, csrc/batch_scheduler.cpp:4-10. */
MuxBatchScheduler *mux_sched_create(int32_t num_layers, int32_t num_heads,
                                    int32_t max_seq_len, int32_t block_size);
void mux_sched_destroy(MuxBatchScheduler *s);

/* BatchScheduler::addRequest, csrc/batch_scheduler.cpp:12-19 (+ Request ctor,
 * csrc/batch_scheduler.h:22-29). */
int32_t mux_sched_add_request(MuxBatchScheduler *s, const int32_t *prompt, int32_t prompt_len,
                              int32_t req_id, int32_t max_tokens);

/* BatchScheduler::tryBatch, csrc/batch_scheduler.cpp:21-48.  Decode step iff
 * n_last > 0 (then n_last must equal n).  out is int32[3n+1].  MUX_ENOENT on
 * an unknown id (the reference dereferences a null request). Returns 3n+1. */
int32_t mux_sched_try_batch(MuxBatchScheduler *s, const int32_t *request_ids, int32_t n,
                            const int32_t *last_tokens, int32_t n_last, int32_t *out);

/* BatchScheduler::getBatchInfo, csrc/batch_scheduler.cpp:50-97.  req is the
 * int32[3R] request vector (try_batch output minus its last element),
 * block_info the allocator reply.  Writes [numTokens, numContexts,
 * maxContextLen, maxNumBlocksPerSeq, L, H, promptLens...] and returns its
 * length. */
int32_t mux_sched_get_batch_info(MuxBatchScheduler *s, const int32_t *req, int32_t n_req,
                                 const int32_t *block_info, int64_t n_block_info,
                                 int32_t *out, int32_t out_cap);

/* BatchScheduler::getBatch, csrc/batch_scheduler.cpp:99-193 (+ getPromptSlots
 * / getLastEmptySlot, csrc/batch_scheduler.h:42-67).  Fills the caller's CPU
 * buffers: tokens/positions int32[n_tok_padded] (zero padded), context_lens
 * int32, block_tables int32 [numTokens, maxBlk, L, H], slot_mapping int64
 * [numTokens, L, H].  *_cap are element capacities; unlike the reference the
 * sizes are checked (MUX_ENOSPC).  Table entries past a request's physical
 * blocks are left as the caller supplied them.  Returns numTokens. */
int64_t mux_sched_get_batch(MuxBatchScheduler *s, const int32_t *req, int32_t n_req,
                            const int32_t *block_info, int64_t n_block_info,
                            int32_t *tokens, int32_t *positions, int64_t n_tok_padded,
                            int32_t *context_lens, int64_t context_lens_cap,
                            int32_t *block_tables, int64_t block_tables_cap,
                            int64_t *slot_mapping, int64_t slot_mapping_cap);

/* No reference counterpart: the same fill as mux_sched_get_batch but the
 * block table is emitted directly in the layout the attention layer consumes,
 * int32 [L, numContexts, H, max_blocks] - what the reference produces with
 * block_tables.permute(2,0,3,1).contiguous() on the device
 * (muxserve/flexserver/llm_runtime.py:327).  max_blocks is the caller's row
 * length (>= maxNumBlocksPerSeq). */
int64_t mux_sched_get_batch_permuted(MuxBatchScheduler *s, const int32_t *req, int32_t n_req,
                                     const int32_t *block_info, int64_t n_block_info,
                                     int32_t *tokens, int32_t *positions, int64_t n_tok_padded,
                                     int32_t *context_lens, int64_t context_lens_cap,
                                     int32_t *block_tables_lbhm, int64_t block_tables_cap,
                                     int32_t max_blocks,
                                     int64_t *slot_mapping, int64_t slot_mapping_cap);

/* No reference counterpart: the step without the O(tokens x L x H) host work.
 * The reference rebuilds the whole block table and a slot per (token, layer,
 * head) on the host every step and uploads both (csrc/batch_scheduler.cpp:
 * 131-169, muxserve/flexserver/llm_runtime.py:301-327: 16 MB of table per
 * decode step of a 7B model, 130 MB of slots per prefill step of a 30B model).
 * Here the device keeps a mirror of every request's id run
 * [row][token block][L][H]; a step uploads only the allocator's reply and
 * MUX_STEP_DESC_INTS ints per sequence, and mux_build_step_inputs
 * (muxserve_attn.h) derives slot_mapping and the step's block table on the
 * device, bit-identical to what mux_sched_get_batch writes.
 *
 * mux_sched_enable_device_rows: once, before the first compact step; max_rows =
 * rows of the device mirror (>= requests alive at a time).
 * mux_sched_get_batch_compact: same step protocol and side effects as
 * mux_sched_get_batch (preempted requests forgotten, prompt_info / batch_reqs
 * refreshed, tokens / positions / context_lens filled); instead of tables and
 * slots it writes one descriptor per batch entry i < block_info[0]:
 *   desc[i] = { row, numPhysicalBlocks, first token block brought by this
 *               reply, token blocks brought, offset of their ids in block_info,
 *               contextLen (decode) or promptLen, first token of the entry in
 *               the batch, 1 if decoding }
 * MUX_ENOSPC when no row is free.  Returns numTokens. */
#define MUX_STEP_DESC_INTS 8
int32_t mux_sched_enable_device_rows(MuxBatchScheduler *s, int32_t max_rows);
int64_t mux_sched_get_batch_compact(MuxBatchScheduler *s, const int32_t *req, int32_t n_req,
                                    const int32_t *block_info, int64_t n_block_info,
                                    int32_t *tokens, int32_t *positions, int64_t n_tok_padded,
                                    int32_t *context_lens, int64_t context_lens_cap,
                                    int32_t *desc, int64_t desc_cap);

/* BatchScheduler::releaseRequests, csrc/batch_scheduler.cpp:195-199. */
int32_t mux_sched_release_requests(MuxBatchScheduler *s, const int32_t *request_ids, int32_t n);

/* getPreemptRequests / getPromptInfo / getBatchReqs,
 * csrc/batch_scheduler.h:90-94.  Each copies up to cap ints and returns the
 * full length; batch_reqs is flattened (id, maxTokens) pairs. */
int32_t mux_sched_get_preempt_requests(const MuxBatchScheduler *s, int32_t *out, int32_t cap);
int32_t mux_sched_get_prompt_info(const MuxBatchScheduler *s, int32_t *out, int32_t cap);
int32_t mux_sched_get_batch_reqs(const MuxBatchScheduler *s, int32_t *out, int32_t cap);

/* Introspection (tests): fields of one request, MUX_ENOENT if unknown.
 * out = [contextLen, numPhysicalBlocks, logicalBlockIdx, logicalBlockOffset,
 *        promptLen, numOutputs]. */
int32_t mux_sched_request_state(const MuxBatchScheduler *s, int32_t req_id, int32_t out[6]);
int32_t mux_sched_num_requests(const MuxBatchScheduler *s);

#ifdef __cplusplus
}
#endif
#endif /* MUXSERVE_HOST_H */
