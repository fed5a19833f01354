// Head-granular KV block allocator behind the C ABI in include/muxserve_host.h.
//
// Behavioural contract: identical id sequences to the reference allocator
// (csrc/memory_manager.cpp:4-157) for every call sequence the reference
// survives, including tail preemption inside allocate_batch.  The structure is
// this library's own: one flat LIFO vector for the free list, a hash map of
// per-request runs, and a single planning pass that decides the preemption
// cut before any state is touched.
#include "muxserve_host.h"

#include <algorithm>
#include <cstring>
#include <unordered_map>
#include <vector>

struct MuxKVStorage {
  std::vector<int32_t> free_list;                              // back = next id handed out
  std::unordered_map<int32_t, std::vector<int32_t>> held;      // request id -> ids in grant order
  int64_t blocks_allocated = 0;
  int32_t last_delta = 0;                                      // what get_new_blocks_allocated reports
};

namespace {

struct RowPlan {
  int32_t request_id;
  int64_t wanted;      // head-blocks the reply must carry for this row
  int64_t fresh;       // head-blocks that must come off the free list
  int64_t held_before; // head-blocks the request owns on entry
  bool decode_row;     // third column: request already owns its prompt blocks
};

}  // namespace

extern "C" {

MuxKVStorage *mux_kvstorage_create(int32_t num_blocks) {
  if (num_blocks < 0) return nullptr;
  auto *s = new MuxKVStorage();
  s->free_list.resize(static_cast<size_t>(num_blocks));
  for (int32_t i = 0; i < num_blocks; ++i) s->free_list[static_cast<size_t>(i)] = i;
  return s;
}

void mux_kvstorage_destroy(MuxKVStorage *s) { delete s; }

int32_t mux_kvstorage_allocate(MuxKVStorage *s, int32_t size, int32_t *out) {
  if (!s || size < 0 || (size > 0 && !out)) return MUX_EINVAL;
  if (static_cast<size_t>(size) > s->free_list.size()) return MUX_ENOSPC;
  // Ids leave from the back one by one, so the caller sees them descending on
  // a fresh pool.
  for (int32_t i = 0; i < size; ++i) {
    out[i] = s->free_list.back();
    s->free_list.pop_back();
  }
  return size;
}

int64_t mux_kvstorage_allocate_batch_bound(const int32_t *info, int32_t n_info,
                                           int32_t num_layers, int32_t num_heads) {
  if (!info || n_info < 0) return MUX_EINVAL;
  int64_t per = static_cast<int64_t>(num_layers) * num_heads;
  int64_t total = 1;
  for (int32_t i = 0; i + 2 < n_info; i += 3) total += std::max<int64_t>(info[i + 1], 0) * per;
  return total;
}

int64_t mux_kvstorage_allocate_batch(MuxKVStorage *s, const int32_t *info, int32_t n_info,
                                     int32_t num_layers, int32_t num_heads,
                                     int32_t *out, int64_t out_cap) {
  if (!s || !info || !out || n_info < 0 || out_cap < 1 || num_layers < 0 || num_heads < 0)
    return MUX_EINVAL;
  const int32_t rows = n_info / 3;
  const int64_t per = static_cast<int64_t>(num_layers) * num_heads;

  // Pass 1: what every row wants and what it already owns.  A prefill row
  // (flag 0) for a request that owns blocks only needs the difference; a
  // decode row (flag 1) always needs its full count fresh.
  std::vector<RowPlan> plan(static_cast<size_t>(rows));
  std::vector<int64_t> fresh_prefix(static_cast<size_t>(rows) + 1, 0);
  std::vector<int64_t> wanted_prefix(static_cast<size_t>(rows) + 1, 0);
  for (int32_t i = 0; i < rows; ++i) {
    RowPlan &r = plan[static_cast<size_t>(i)];
    r.request_id = info[3 * i];
    r.wanted = static_cast<int64_t>(info[3 * i + 1]) * per;
    r.decode_row = info[3 * i + 2] != 0;
    auto it = s->held.find(r.request_id);
    r.held_before = it == s->held.end() ? 0 : static_cast<int64_t>(it->second.size());
    r.fresh = r.decode_row ? r.wanted : r.wanted - r.held_before;
    fresh_prefix[static_cast<size_t>(i) + 1] = fresh_prefix[static_cast<size_t>(i)] + r.fresh;
    wanted_prefix[static_cast<size_t>(i) + 1] = wanted_prefix[static_cast<size_t>(i)] + r.wanted;
  }

  // Pass 2: the cut.  Keep the longest prefix of rows whose fresh demand fits
  // in the free list once every row behind the cut has given its blocks back.
  int32_t cut = rows;
  {
    std::vector<int64_t> held_suffix(static_cast<size_t>(rows) + 1, 0);
    for (int32_t i = rows - 1; i >= 0; --i)
      held_suffix[static_cast<size_t>(i)] =
          held_suffix[static_cast<size_t>(i) + 1] + plan[static_cast<size_t>(i)].held_before;
    const int64_t free_now = static_cast<int64_t>(s->free_list.size());
    while (cut > 0 &&
           fresh_prefix[static_cast<size_t>(cut)] > free_now + held_suffix[static_cast<size_t>(cut)])
      --cut;
  }

  // Pass 3: rows behind the cut lose their blocks (appended to the free list
  // in row order, each run in its grant order).
  int64_t reclaimed = 0;
  for (int32_t i = cut; i < rows; ++i) {
    const RowPlan &r = plan[static_cast<size_t>(i)];
    if (r.held_before <= 0) continue;
    auto it = s->held.find(r.request_id);
    if (it == s->held.end()) continue;   // same id listed twice behind the cut
    reclaimed += static_cast<int64_t>(it->second.size());
    s->free_list.insert(s->free_list.end(), it->second.begin(), it->second.end());
    s->held.erase(it);
  }
  s->blocks_allocated -= reclaimed;
  s->last_delta = static_cast<int32_t>(-reclaimed);

  out[0] = cut;
  if (cut <= 0) return 1;

  const int64_t take = fresh_prefix[static_cast<size_t>(cut)];
  const int64_t reply_len = 1 + wanted_prefix[static_cast<size_t>(cut)];
  if (reply_len > out_cap) return MUX_ENOSPC;
  if (take < 0 || take > static_cast<int64_t>(s->free_list.size())) return MUX_ESTATE;

  // Pass 4: grant.  The `take` ids at the tail of the free list are dealt out
  // front to back in row order; each row's reply is the last `wanted` ids of
  // its (now extended) run.
  const int32_t *grant = s->free_list.data() + (s->free_list.size() - static_cast<size_t>(take));
  int64_t dealt = 0;
  int64_t w = 1;
  for (int32_t i = 0; i < cut; ++i) {
    const RowPlan &r = plan[static_cast<size_t>(i)];
    if (r.fresh > 0) {
      if (dealt + r.fresh > take) return MUX_ESTATE;   // a row asked for fewer blocks than it holds
      auto &run = s->held[r.request_id];
      run.insert(run.end(), grant + dealt, grant + dealt + r.fresh);
      dealt += r.fresh;
    }
    if (r.wanted > 0) {
      auto &run = s->held[r.request_id];
      if (static_cast<int64_t>(run.size()) < r.wanted) return MUX_ESTATE;
      std::memcpy(out + w, run.data() + (run.size() - static_cast<size_t>(r.wanted)),
                  static_cast<size_t>(r.wanted) * sizeof(int32_t));
      w += r.wanted;
    }
  }
  s->last_delta += static_cast<int32_t>(take);
  s->blocks_allocated += s->last_delta;
  s->free_list.resize(s->free_list.size() - static_cast<size_t>(take));
  return reply_len;
}

int64_t mux_kvstorage_free_batch(MuxKVStorage *s, const int32_t *request_ids, int32_t n) {
  if (!s || n < 0 || (n > 0 && !request_ids)) return MUX_EINVAL;
  int64_t freed = 0;
  for (int32_t i = 0; i < n; ++i) {
    auto it = s->held.find(request_ids[i]);
    if (it == s->held.end()) continue;
    freed += static_cast<int64_t>(it->second.size());
    s->free_list.insert(s->free_list.end(), it->second.begin(), it->second.end());
    s->held.erase(it);
  }
  s->blocks_allocated -= freed;
  return freed;
}

int32_t mux_kvstorage_new_blocks_allocated(const MuxKVStorage *s) {
  return s ? s->last_delta : MUX_EINVAL;
}

int64_t mux_kvstorage_num_free(const MuxKVStorage *s) {
  return s ? static_cast<int64_t>(s->free_list.size()) : MUX_EINVAL;
}

int64_t mux_kvstorage_num_held(const MuxKVStorage *s, int32_t request_id) {
  if (!s) return MUX_EINVAL;
  auto it = s->held.find(request_id);
  return it == s->held.end() ? 0 : static_cast<int64_t>(it->second.size());
}

}  // extern "C"
