// Per-step block-table / slot-mapping builder behind the C ABI in
// include/muxserve_host.h.
//
// Behavioural contract: the same step protocol and bit-identical index
// tensors as the reference builder (csrc/batch_scheduler.{h,cpp}):
//   try_batch -> (allocator) -> get_batch_info -> get_batch.
// Structure is this library's own: each sequence keeps a growable run of
// head-block ids ordered [token block][layer][head] (the reference reserves
// maxBlocksPerSeq*L*H ints per request up front), slots are written straight
// into the caller's tensor instead of through a temporary vector, and the
// block table can be emitted directly in the [L, B, H, maxBlk] layout the
// attention kernels read.
#include "muxserve_host.h"

#include <algorithm>
#include <cstring>
#include <memory>
#include <unordered_map>
#include <vector>

namespace {

struct Sequence {
  int32_t id = 0;
  int32_t max_tokens = 0;
  int32_t context_len = 0;
  int32_t physical_blocks = 0;   // token blocks whose ids have been received
  int32_t logical_block = 0;     // index of the token block the last token lives in
  int32_t logical_offset = 0;    // its offset inside that block
  std::vector<int32_t> prompt;
  std::vector<int32_t> outputs;
  std::vector<int32_t> ids;      // [physical_blocks][L][H]
  int32_t row = -1;              // row of the device-resident table mirror, once assigned

  bool decoding() const { return !outputs.empty(); }
};

}  // namespace

struct MuxBatchScheduler {
  int32_t L = 0, H = 0, max_seq_len = 0, block_size = 0, max_blocks_per_seq = 0;
  std::unordered_map<int32_t, std::unique_ptr<Sequence>> seqs;
  std::vector<int32_t> preempted, prompt_info, batch_reqs;
  std::vector<int32_t> free_rows;            // device-table rows not in use (empty: feature off)
  int32_t max_rows = 0;

  Sequence *find(int32_t id) const {
    auto it = seqs.find(id);
    return it == seqs.end() ? nullptr : it->second.get();
  }
  // Forget a request; its device-table row goes back to the free list.
  int32_t drop(int32_t id) {
    auto it = seqs.find(id);
    if (it == seqs.end()) return 0;
    if (it->second->row >= 0) free_rows.push_back(it->second->row);
    seqs.erase(it);
    return 1;
  }
};

namespace {

int32_t copy_out(const std::vector<int32_t> &v, int32_t *out, int32_t cap) {
  const int32_t n = static_cast<int32_t>(v.size());
  if (out && cap > 0) std::memcpy(out, v.data(), sizeof(int32_t) * static_cast<size_t>(std::min(n, cap)));
  return n;
}

// Shared body of get_batch / get_batch_permuted.  `permuted` selects the
// block-table layout: false = [numTokens, maxBlk, L, H] (row length taken from
// the batch), true = [L, numContexts, H, max_blocks_arg].
int64_t fill_batch(MuxBatchScheduler *s, const int32_t *req, int32_t n_req,
                   const int32_t *block_info, int64_t n_block_info,
                   int32_t *tokens, int32_t *positions, int64_t n_tok_padded,
                   int32_t *context_lens, int64_t context_lens_cap,
                   int32_t *block_tables, int64_t block_tables_cap,
                   bool permuted, int32_t max_blocks_arg,
                   int64_t *slot_mapping, int64_t slot_mapping_cap) {
  if (!s || !req || !block_info || n_req < 0 || n_block_info < 1 || n_tok_padded < 0) return MUX_EINVAL;
  const int32_t rows = n_req / 3;
  const int32_t cut = block_info[0];
  const int64_t per = static_cast<int64_t>(s->L) * s->H;
  const int32_t bs = s->block_size;

  // Pass 1 (read-only): sizes, so every capacity is checked before any write
  // or any request is dropped.
  int64_t n_tokens = 0, n_ctx = 0, n_slots = 0;
  int32_t max_blocks = 0;
  for (int32_t i = 0; i < rows && i < cut; ++i) {
    const Sequence *q = s->find(req[3 * i]);
    if (!q) return MUX_ENOENT;
    if (q->decoding()) {
      if (q->physical_blocks < 1) return MUX_ESTATE;
      max_blocks = std::max(max_blocks, q->physical_blocks);
      n_tokens += 1;
      n_ctx += 1;
      n_slots += per;
    } else {
      const int64_t p = static_cast<int64_t>(q->prompt.size());
      if ((p + bs - 1) / bs > q->physical_blocks) return MUX_ESTATE;
      n_tokens += p;
      n_slots += p * per;
    }
  }
  if (n_tokens > n_tok_padded || n_ctx > context_lens_cap || n_slots > slot_mapping_cap) return MUX_ENOSPC;
  if ((n_tokens > 0 && (!tokens || !positions)) || (n_ctx > 0 && !context_lens) || (n_slots > 0 && !slot_mapping))
    return MUX_EINVAL;
  const int32_t row_blocks = permuted ? max_blocks_arg : max_blocks;
  if (max_blocks > 0) {
    if (!block_tables) return MUX_EINVAL;
    if (permuted && max_blocks_arg < max_blocks) return MUX_ENOSPC;
    const int64_t need = permuted ? per * n_ctx * row_blocks
                                  : n_tokens * static_cast<int64_t>(row_blocks) * per;
    if (need > block_tables_cap) return MUX_ENOSPC;
  }

  // Pass 2: fill.
  s->preempted.clear();
  s->prompt_info.clear();
  s->batch_reqs.clear();
  int64_t t = 0;        // token cursor
  int64_t c = 0;        // context (decode sequence) cursor
  int64_t w = 0;        // slot cursor
  int32_t max_ctx = 0;
  for (int32_t i = 0; i < rows; ++i) {
    const int32_t id = req[3 * i];
    if (i >= cut) {     // preempted by the allocator: forget the request
      s->preempted.push_back(id);
      s->drop(id);
      continue;
    }
    Sequence *q = s->find(id);
    if (q->decoding()) {
      tokens[t] = q->outputs.back();
      positions[t] = q->context_len - 1;
      context_lens[c] = q->context_len;
      max_ctx = std::max(max_ctx, q->context_len);
      // One new token: it lands in the last physical token block at the
      // running in-block offset, once per (layer, head).
      const int32_t *last = q->ids.data() + static_cast<int64_t>(q->physical_blocks - 1) * per;
      for (int64_t j = 0; j < per; ++j)
        slot_mapping[w + j] = static_cast<int64_t>(last[j]) * bs + q->logical_offset;
      w += per;
      if (max_blocks > 0) {
        if (!permuted) {
          // Row index is the batch position i (decode batches hold one token
          // per request, so this equals the token cursor).
          std::memcpy(block_tables + static_cast<int64_t>(i) * row_blocks * per, q->ids.data(),
                      sizeof(int32_t) * static_cast<size_t>(q->physical_blocks * per));
        } else {
          // [L, n_ctx, H, row_blocks]  <-  ids[tb][l][h]: a transpose of the
          // request's [blocks][L*H] matrix, 16 token blocks at a time so that
          // every write is one 64-byte run and the 16 source rows are each read
          // front to back.
          for (int32_t tb0 = 0; tb0 < q->physical_blocks; tb0 += 16) {
            const int32_t kmax = std::min(16, q->physical_blocks - tb0);
            const int32_t *src = q->ids.data() + static_cast<int64_t>(tb0) * per;
            for (int32_t l = 0; l < s->L; ++l) {
              int32_t *dst = block_tables + ((static_cast<int64_t>(l) * n_ctx + c) * s->H) * row_blocks + tb0;
              const int32_t *sl = src + static_cast<int64_t>(l) * s->H;
              for (int32_t h = 0; h < s->H; ++h, dst += row_blocks)
                for (int32_t k = 0; k < kmax; ++k) dst[k] = sl[static_cast<int64_t>(k) * per + h];
            }
          }
        }
      }
      t += 1;
      c += 1;
    } else {
      const int64_t p = static_cast<int64_t>(q->prompt.size());
      std::memcpy(tokens + t, q->prompt.data(), sizeof(int32_t) * static_cast<size_t>(p));
      for (int64_t k = 0; k < p; ++k) positions[t + k] = static_cast<int32_t>(k);
      s->prompt_info.push_back(static_cast<int32_t>(p));
      // Prompt token k lives in token block k / bs at offset k % bs.
      for (int64_t k = 0; k < p; ++k) {
        const int32_t *blk = q->ids.data() + (k / bs) * per;
        const int64_t off = k % bs;
        int64_t *dst = slot_mapping + w + k * per;
        for (int64_t j = 0; j < per; ++j) dst[j] = static_cast<int64_t>(blk[j]) * bs + off;
      }
      w += p * per;
      t += p;
      if (max_blocks > 0 && !permuted) {
        // Mixed batches are not produced by the serving loop; keep the
        // reference's behaviour of copying the run into row i regardless.
        if (static_cast<int64_t>(i + 1) * row_blocks * per <= block_tables_cap &&
            q->physical_blocks <= row_blocks)
          std::memcpy(block_tables + static_cast<int64_t>(i) * row_blocks * per, q->ids.data(),
                      sizeof(int32_t) * static_cast<size_t>(q->physical_blocks * per));
      }
    }
    s->batch_reqs.push_back(id);
    s->batch_reqs.push_back(q->max_tokens);
  }
  s->prompt_info.push_back(max_ctx);
  for (int64_t k = t; k < n_tok_padded; ++k) {
    tokens[k] = 0;
    positions[k] = 0;
  }
  return n_tokens;
}

}  // namespace

extern "C" {

MuxBatchScheduler *mux_sched_create(int32_t num_layers, int32_t num_heads,
                                    int32_t max_seq_len, int32_t block_size) {
  if (num_layers <= 0 || num_heads <= 0 || max_seq_len <= 0 || block_size <= 0) return nullptr;
  auto *s = new MuxBatchScheduler();
  s->L = num_layers;
  s->H = num_heads;
  s->max_seq_len = max_seq_len;
  s->block_size = block_size;
  s->max_blocks_per_seq = (max_seq_len + block_size - 1) / block_size;
  return s;
}

void mux_sched_destroy(MuxBatchScheduler *s) { delete s; }

int32_t mux_sched_add_request(MuxBatchScheduler *s, const int32_t *prompt, int32_t prompt_len,
                              int32_t req_id, int32_t max_tokens) {
  if (!s || prompt_len < 0 || (prompt_len > 0 && !prompt)) return MUX_EINVAL;
  auto q = std::make_unique<Sequence>();
  q->id = req_id;
  q->max_tokens = max_tokens;
  q->prompt.assign(prompt, prompt + prompt_len);
  q->context_len = prompt_len;
  // Position of the last prompt token: block ceil(P/bs)-1, offset (P-1) % bs
  // (C++ truncating division, so an empty prompt gives block -1, offset -1).
  q->logical_block = (prompt_len + s->block_size - 1) / s->block_size - 1;
  q->logical_offset = (prompt_len - 1) % s->block_size;
  s->drop(req_id);                  // re-adding an id replaces the old request
  s->seqs[req_id] = std::move(q);
  return MUX_OK;
}

int32_t mux_sched_try_batch(MuxBatchScheduler *s, const int32_t *request_ids, int32_t n,
                            const int32_t *last_tokens, int32_t n_last, int32_t *out) {
  if (!s || n < 0 || n_last < 0 || !out || (n > 0 && !request_ids)) return MUX_EINVAL;
  const bool decoding = n_last > 0;
  if (decoding && (n_last < n || !last_tokens)) return MUX_EINVAL;
  for (int32_t i = 0; i < n; ++i)
    if (!s->find(request_ids[i])) return MUX_ENOENT;   // checked before any state changes
  int64_t total = 0;
  for (int32_t i = 0; i < n; ++i) {
    Sequence *q = s->find(request_ids[i]);
    int32_t need = q->logical_block + 1;               // prefill: every prompt token block
    if (decoding) {
      // The sampled token joins the sequence; a new token block is needed
      // only when it opens one.
      q->outputs.push_back(last_tokens[i]);
      q->context_len += 1;
      if (++q->logical_offset == s->block_size) {
        q->logical_offset = 0;
        q->logical_block += 1;
      }
      need = q->logical_block + 1 - q->physical_blocks;
    }
    out[3 * i] = q->id;
    out[3 * i + 1] = need;
    out[3 * i + 2] = std::min(q->physical_blocks, 1);
    total += need;
  }
  out[3 * n] = static_cast<int32_t>(total);
  return 3 * n + 1;
}

int32_t mux_sched_get_batch_info(MuxBatchScheduler *s, const int32_t *req, int32_t n_req,
                                 const int32_t *block_info, int64_t n_block_info,
                                 int32_t *out, int32_t out_cap) {
  if (!s || !req || !block_info || !out || n_req < 0 || n_block_info < 1) return MUX_EINVAL;
  const int32_t rows = n_req / 3;
  const int32_t cut = block_info[0];
  if (cut > rows) return MUX_EINVAL;
  const int64_t per = static_cast<int64_t>(s->L) * s->H;

  // Validate before mutating: ids known, reply long enough, output fits.
  int64_t reply = 1;
  int32_t prompts = 0;
  for (int32_t i = 0; i < cut; ++i) {
    const Sequence *q = s->find(req[3 * i]);
    if (!q) return MUX_ENOENT;
    if (req[3 * i + 1] > 0) reply += static_cast<int64_t>(req[3 * i + 1]) * per;
    if (!q->decoding()) ++prompts;
  }
  if (reply > n_block_info) return MUX_EINVAL;
  if (6 + prompts > out_cap) return MUX_ENOSPC;

  int32_t n_tokens = 0, n_ctx = 0, max_ctx = 0, max_blocks = 0, n_prompts = 0;
  int64_t cursor = 1;
  for (int32_t i = 0; i < cut; ++i) {
    Sequence *q = s->find(req[3 * i]);
    const int32_t granted = req[3 * i + 1];
    if (granted > 0) {
      const int64_t cnt = static_cast<int64_t>(granted) * per;
      q->ids.resize(static_cast<size_t>(q->physical_blocks * per));
      q->ids.insert(q->ids.end(), block_info + cursor, block_info + cursor + cnt);
      cursor += cnt;
      q->physical_blocks += granted;
    }
    if (q->decoding()) {
      max_blocks = std::max(max_blocks, q->physical_blocks);
      max_ctx = std::max(max_ctx, q->context_len);
      n_ctx += 1;
      n_tokens += 1;
    } else {
      out[6 + n_prompts++] = static_cast<int32_t>(q->prompt.size());
      n_tokens += static_cast<int32_t>(q->prompt.size());
    }
  }
  out[0] = n_tokens;
  out[1] = n_ctx;
  out[2] = max_ctx;
  out[3] = max_blocks;
  out[4] = s->L;
  out[5] = s->H;
  return 6 + n_prompts;
}

int64_t mux_sched_get_batch(MuxBatchScheduler *s, const int32_t *req, int32_t n_req,
                            const int32_t *block_info, int64_t n_block_info,
                            int32_t *tokens, int32_t *positions, int64_t n_tok_padded,
                            int32_t *context_lens, int64_t context_lens_cap,
                            int32_t *block_tables, int64_t block_tables_cap,
                            int64_t *slot_mapping, int64_t slot_mapping_cap) {
  return fill_batch(s, req, n_req, block_info, n_block_info, tokens, positions, n_tok_padded,
                    context_lens, context_lens_cap, block_tables, block_tables_cap,
                    /*permuted=*/false, 0, slot_mapping, slot_mapping_cap);
}

int64_t mux_sched_get_batch_permuted(MuxBatchScheduler *s, const int32_t *req, int32_t n_req,
                                     const int32_t *block_info, int64_t n_block_info,
                                     int32_t *tokens, int32_t *positions, int64_t n_tok_padded,
                                     int32_t *context_lens, int64_t context_lens_cap,
                                     int32_t *block_tables_lbhm, int64_t block_tables_cap,
                                     int32_t max_blocks,
                                     int64_t *slot_mapping, int64_t slot_mapping_cap) {
  return fill_batch(s, req, n_req, block_info, n_block_info, tokens, positions, n_tok_padded,
                    context_lens, context_lens_cap, block_tables_lbhm, block_tables_cap,
                    /*permuted=*/true, max_blocks, slot_mapping, slot_mapping_cap);
}

int32_t mux_sched_enable_device_rows(MuxBatchScheduler *s, int32_t max_rows) {
  if (!s || max_rows <= 0) return MUX_EINVAL;
  if (s->max_rows != 0) return MUX_ESTATE;
  s->max_rows = max_rows;
  s->free_rows.resize(static_cast<size_t>(max_rows));
  for (int32_t r = 0; r < max_rows; ++r) s->free_rows[static_cast<size_t>(r)] = max_rows - 1 - r;   // row 0 first
  return MUX_OK;
}

int64_t mux_sched_get_batch_compact(MuxBatchScheduler *s, const int32_t *req, int32_t n_req,
                                    const int32_t *block_info, int64_t n_block_info,
                                    int32_t *tokens, int32_t *positions, int64_t n_tok_padded,
                                    int32_t *context_lens, int64_t context_lens_cap,
                                    int32_t *desc, int64_t desc_cap) {
  if (!s || !req || !block_info || n_req < 0 || n_block_info < 1 || n_tok_padded < 0) return MUX_EINVAL;
  if (s->max_rows == 0) return MUX_ESTATE;
  const int32_t rows = n_req / 3;
  const int32_t cut = block_info[0];
  const int64_t per = static_cast<int64_t>(s->L) * s->H;
  const int32_t bs = s->block_size;

  // Pass 1 (read-only): sizes and row demand, checked before any write or drop.
  int64_t n_tokens = 0, n_ctx = 0, n_live = 0, new_rows = 0, freed_rows = 0;
  for (int32_t i = 0; i < rows; ++i) {
    const Sequence *q = s->find(req[3 * i]);
    if (i >= cut) {
      if (q && q->row >= 0) ++freed_rows;
      continue;
    }
    if (!q) return MUX_ENOENT;
    if (q->physical_blocks > s->max_blocks_per_seq) return MUX_ENOSPC;
    if (q->decoding()) {
      if (q->physical_blocks < 1) return MUX_ESTATE;
      n_tokens += 1;
      n_ctx += 1;
    } else {
      const int64_t p = static_cast<int64_t>(q->prompt.size());
      if ((p + bs - 1) / bs > q->physical_blocks) return MUX_ESTATE;
      n_tokens += p;
    }
    if (q->row < 0) ++new_rows;
    ++n_live;
  }
  if (n_tokens > n_tok_padded || n_ctx > context_lens_cap || n_live * MUX_STEP_DESC_INTS > desc_cap) return MUX_ENOSPC;
  if (new_rows > static_cast<int64_t>(s->free_rows.size()) + freed_rows) return MUX_ENOSPC;
  if ((n_tokens > 0 && (!tokens || !positions)) || (n_ctx > 0 && !context_lens) || (n_live > 0 && !desc))
    return MUX_EINVAL;

  // Pass 2: requests the allocator preempted go first (their rows become free).
  s->preempted.clear();
  s->prompt_info.clear();
  s->batch_reqs.clear();
  for (int32_t i = std::max(cut, 0); i < rows; ++i) {
    s->preempted.push_back(req[3 * i]);
    s->drop(req[3 * i]);
  }
  int64_t t = 0, c = 0, cursor = 1;
  int32_t max_ctx = 0;
  for (int32_t i = 0; i < rows && i < cut; ++i) {
    Sequence *q = s->find(req[3 * i]);
    if (q->row < 0) {
      q->row = s->free_rows.back();
      s->free_rows.pop_back();
    }
    const int32_t granted = std::max(req[3 * i + 1], 0);
    int32_t *d = desc + static_cast<int64_t>(i) * MUX_STEP_DESC_INTS;
    d[0] = q->row;
    d[1] = q->physical_blocks;
    d[2] = q->physical_blocks - granted;          // first token block the reply brought
    d[3] = granted;
    d[4] = static_cast<int32_t>(cursor);           // where its ids start in block_info
    d[6] = static_cast<int32_t>(t);
    cursor += static_cast<int64_t>(granted) * per;
    if (q->decoding()) {
      tokens[t] = q->outputs.back();
      positions[t] = q->context_len - 1;
      context_lens[c] = q->context_len;
      max_ctx = std::max(max_ctx, q->context_len);
      d[5] = q->context_len;
      d[7] = 1;
      t += 1;
      c += 1;
    } else {
      const int64_t p = static_cast<int64_t>(q->prompt.size());
      std::memcpy(tokens + t, q->prompt.data(), sizeof(int32_t) * static_cast<size_t>(p));
      for (int64_t k = 0; k < p; ++k) positions[t + k] = static_cast<int32_t>(k);
      s->prompt_info.push_back(static_cast<int32_t>(p));
      d[5] = static_cast<int32_t>(p);
      d[7] = 0;
      t += p;
    }
    s->batch_reqs.push_back(q->id);
    s->batch_reqs.push_back(q->max_tokens);
  }
  s->prompt_info.push_back(max_ctx);
  for (int64_t k = t; k < n_tok_padded; ++k) {
    tokens[k] = 0;
    positions[k] = 0;
  }
  return n_tokens;
}

int32_t mux_sched_release_requests(MuxBatchScheduler *s, const int32_t *request_ids, int32_t n) {
  if (!s || n < 0 || (n > 0 && !request_ids)) return MUX_EINVAL;
  int32_t erased = 0;
  for (int32_t i = 0; i < n; ++i) erased += s->drop(request_ids[i]);
  return erased;
}

int32_t mux_sched_get_preempt_requests(const MuxBatchScheduler *s, int32_t *out, int32_t cap) {
  return s ? copy_out(s->preempted, out, cap) : MUX_EINVAL;
}

int32_t mux_sched_get_prompt_info(const MuxBatchScheduler *s, int32_t *out, int32_t cap) {
  return s ? copy_out(s->prompt_info, out, cap) : MUX_EINVAL;
}

int32_t mux_sched_get_batch_reqs(const MuxBatchScheduler *s, int32_t *out, int32_t cap) {
  return s ? copy_out(s->batch_reqs, out, cap) : MUX_EINVAL;
}

int32_t mux_sched_request_state(const MuxBatchScheduler *s, int32_t req_id, int32_t out[6]) {
  if (!s || !out) return MUX_EINVAL;
  const Sequence *q = s->find(req_id);
  if (!q) return MUX_ENOENT;
  out[0] = q->context_len;
  out[1] = q->physical_blocks;
  out[2] = q->logical_block;
  out[3] = q->logical_offset;
  out[4] = static_cast<int32_t>(q->prompt.size());
  out[5] = static_cast<int32_t>(q->outputs.size());
  return MUX_OK;
}

int32_t mux_sched_num_requests(const MuxBatchScheduler *s) {
  return s ? static_cast<int32_t>(s->seqs.size()) : MUX_EINVAL;
}

}  // extern "C"
