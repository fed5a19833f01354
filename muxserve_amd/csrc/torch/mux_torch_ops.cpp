// Thin PyTorch-ROCm operator library over the C ABI of libmuxattn.so
// (include/muxserve_attn.h): at::Tensor arguments are checked (device, dtype,
// shape, unit inner stride), raw pointers and torch's current HIP stream are
// passed on, a negative return code becomes a c10::Error.  No arithmetic and no
// kernels live here; everything below is what a binding of the attention layer
// called at muxserve/flexserver/models/llama.py:159-161 needs on the torch side.
//
//     torch.ops.load_library(".../libmuxtorch.so")
//     torch.ops.muxserve_amd.paged_decode(out, q, k_pool, v_pool, block_tables,
//                                         context_lens, max_ctx, scale, layer, 0, 0, workspace)
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include <algorithm>
#include <vector>

#include "muxserve_attn.h"

namespace {

constexpr int64_t kHead = 128;   // muxserve/flexstore/manager.py:337

void *stream_of(const at::Tensor &t) {
  return static_cast<void *>(c10::hip::getCurrentHIPStream(t.device().index()).stream());
}

int32_t dtype_code(const at::Tensor &t) {
  if (t.scalar_type() == at::kHalf) return MUXA_DTYPE_F16;
  if (t.scalar_type() == at::kBFloat16) return MUXA_DTYPE_BF16;
  TORCH_CHECK(false, "muxserve_amd: expected float16 or bfloat16, got ", t.scalar_type());
}

void need_gpu(std::initializer_list<const at::Tensor *> ts) {
  for (const at::Tensor *t : ts) TORCH_CHECK(t->is_cuda(), "muxserve_amd: tensors must live on the GPU (no CPU path)");
}

int64_t rows(const at::Tensor &t, const char *what) {
  TORCH_CHECK(t.dim() == 2 && (t.size(1) == 0 || t.stride(1) == 1), what, ": expected [rows, width] with contiguous rows");
  return t.stride(0);
}

void check(int32_t rc, const char *what) {
  if (rc == MUXA_OK) return;
  const char *why = rc == MUXA_EINVAL        ? "invalid argument"
                    : rc == MUXA_EUNSUPPORTED ? "unsupported shape or type"
                    : rc == MUXA_EWORKSPACE   ? "workspace missing or too small"
                                              : "HIP runtime error";
  TORCH_CHECK(false, what, ": ", why, " (code ", rc, rc == MUXA_EHIP ? ", hipError " : "",
              rc == MUXA_EHIP ? std::to_string(mux_last_hip_error()) : std::string(), ")");
}

// K pool [N, 16, block_size, 8], V pool [N, 128, block_size]; returns block_size.
int64_t check_pools(const at::Tensor &k_pool, const at::Tensor &v_pool) {
  TORCH_CHECK(k_pool.dim() == 4 && k_pool.size(1) == 16 && k_pool.size(3) == 8, "k_pool: expected [N, 16, block_size, 8]");
  const int64_t bs = k_pool.size(2);
  TORCH_CHECK(v_pool.dim() == 3 && v_pool.size(0) == k_pool.size(0) && v_pool.size(1) == kHead && v_pool.size(2) == bs,
              "v_pool: expected [N, 128, block_size]");
  TORCH_CHECK(k_pool.is_contiguous() && v_pool.is_contiguous(), "pools must be contiguous");
  TORCH_CHECK(k_pool.scalar_type() == v_pool.scalar_type(), "k_pool and v_pool dtypes differ");
  return bs;
}

void reshape_and_cache(const at::Tensor &k, const at::Tensor &v, at::Tensor k_pool, at::Tensor v_pool,
                       const at::Tensor &slot_mapping, int64_t layer, int64_t num_tokens) {
  need_gpu({&k, &v, &k_pool, &v_pool, &slot_mapping});
  const int64_t bs = check_pools(k_pool, v_pool);
  TORCH_CHECK(slot_mapping.scalar_type() == at::kLong && slot_mapping.dim() == 3 && slot_mapping.is_contiguous(),
              "slot_mapping: expected contiguous int64 [T, L, Hkv]");
  const int64_t T = num_tokens < 0 ? slot_mapping.size(0) : std::min(num_tokens, slot_mapping.size(0));
  const int64_t L = slot_mapping.size(1), H = slot_mapping.size(2);
  const int64_t stride = rows(k, "k");
  TORCH_CHECK(rows(v, "v") == stride && k.sizes() == v.sizes() && k.scalar_type() == v.scalar_type() &&
                  k.scalar_type() == k_pool.scalar_type(),
              "k and v must have the same shape, strides and dtype as each other and the pool's dtype");
  TORCH_CHECK(k.size(0) >= T && k.size(1) == H * kHead, "k: expected [>=T, Hkv*128]");
  check(mux_reshape_and_cache(k.data_ptr(), v.data_ptr(), stride, k_pool.data_ptr(), v_pool.data_ptr(), k_pool.size(0),
                              slot_mapping.data_ptr<int64_t>(), static_cast<int32_t>(layer), static_cast<int32_t>(L),
                              static_cast<int32_t>(T), static_cast<int32_t>(H), kHead, static_cast<int32_t>(bs),
                              dtype_code(k), stream_of(k)),
        "mux_reshape_and_cache");
}

void rope_reshape_and_cache(const at::Tensor &positions, at::Tensor q, at::Tensor k, const at::Tensor &v,
                            const at::Tensor &cos_sin, at::Tensor k_pool, at::Tensor v_pool,
                            const at::Tensor &slot_mapping, int64_t layer, int64_t num_tokens) {
  need_gpu({&positions, &q, &k, &v, &cos_sin, &k_pool, &v_pool, &slot_mapping});
  const int64_t bs = check_pools(k_pool, v_pool);
  TORCH_CHECK(positions.scalar_type() == at::kLong && positions.dim() == 1 && positions.is_contiguous(),
              "positions: expected contiguous int64 [T]");
  TORCH_CHECK(cos_sin.scalar_type() == at::kFloat && cos_sin.dim() == 2 && cos_sin.is_contiguous(),
              "cos_sin: expected contiguous float32 [max_position, rotary_dim]");
  TORCH_CHECK(slot_mapping.scalar_type() == at::kLong && slot_mapping.dim() == 3 && slot_mapping.is_contiguous(),
              "slot_mapping: expected contiguous int64 [T, L, Hkv]");
  const int64_t T = num_tokens < 0 ? slot_mapping.size(0) : std::min(num_tokens, slot_mapping.size(0));
  const int64_t L = slot_mapping.size(1), H = slot_mapping.size(2);
  const int64_t stride = rows(k, "k");
  TORCH_CHECK(rows(v, "v") == stride && k.sizes() == v.sizes() && k.scalar_type() == v.scalar_type() &&
                  k.scalar_type() == k_pool.scalar_type() && q.scalar_type() == k.scalar_type(),
              "q, k, v must share a dtype with the pool; k and v a shape and strides");
  TORCH_CHECK(k.size(0) >= T && q.size(0) >= T && positions.size(0) >= T && k.size(1) == H * kHead &&
                  q.size(1) % kHead == 0,
              "q [>=T, Hq*128], k/v [>=T, Hkv*128], positions [>=T] expected");
  check(mux_rope_reshape_and_cache(positions.data_ptr<int64_t>(), q.data_ptr(), rows(q, "q"), k.data_ptr(), v.data_ptr(),
                                   stride, cos_sin.data_ptr<float>(), static_cast<int32_t>(cos_sin.size(0)),
                                   static_cast<int32_t>(cos_sin.size(1)), k_pool.data_ptr(), v_pool.data_ptr(),
                                   k_pool.size(0), slot_mapping.data_ptr<int64_t>(), static_cast<int32_t>(layer),
                                   static_cast<int32_t>(L), static_cast<int32_t>(T),
                                   static_cast<int32_t>(q.size(1) / kHead), static_cast<int32_t>(H), kHead,
                                   static_cast<int32_t>(bs), dtype_code(k), stream_of(k)),
        "mux_rope_reshape_and_cache");
}

// The cache writes of several colocated models' step in one launch.  Element i
// of every list describes model i; positions / qs / cos_sins are either all
// empty (plain scatter) or one entry per model (rotary embedding of q and k in
// place first).  num_tokens[i] < 0: all rows of slot_mappings[i].
void multi_reshape_and_cache(at::TensorList ks, at::TensorList vs, at::Tensor k_pool, at::Tensor v_pool,
                             at::TensorList slot_mappings, at::IntArrayRef layers, at::IntArrayRef num_tokens,
                             at::TensorList positions, at::TensorList qs, at::TensorList cos_sins) {
  need_gpu({&k_pool, &v_pool});
  const int64_t bs = check_pools(k_pool, v_pool);
  const size_t n = ks.size();
  const bool rope = !positions.empty();
  TORCH_CHECK(n >= 1 && n <= MUXA_MAX_DECODE_ITEMS && vs.size() == n && slot_mappings.size() == n &&
                  layers.size() == n && num_tokens.size() == n,
              "multi_reshape_and_cache: 1..", MUXA_MAX_DECODE_ITEMS, " models, one entry per model in every list");
  TORCH_CHECK(rope ? (positions.size() == n && qs.size() == n && cos_sins.size() == n)
                   : (qs.empty() && cos_sins.empty()),
              "positions, qs and cos_sins: all empty, or one entry per model");
  MuxCacheWriteItem items[MUXA_MAX_DECODE_ITEMS];
  for (size_t i = 0; i < n; ++i) {
    const at::Tensor &k = ks[i], &v = vs[i], &sm = slot_mappings[i];
    need_gpu({&k, &v, &sm});
    TORCH_CHECK(sm.scalar_type() == at::kLong && sm.dim() == 3 && sm.is_contiguous(),
                "slot_mapping: expected contiguous int64 [T, L, Hkv]");
    const int64_t T = num_tokens[i] < 0 ? sm.size(0) : std::min<int64_t>(num_tokens[i], sm.size(0));
    const int64_t H = sm.size(2);
    const int64_t stride = rows(k, "k");
    TORCH_CHECK(rows(v, "v") == stride && k.sizes() == v.sizes() && k.scalar_type() == v.scalar_type() &&
                    k.scalar_type() == k_pool.scalar_type(),
                "k and v must have the same shape, strides and dtype as each other and the pool's dtype");
    TORCH_CHECK(k.size(0) >= T && k.size(1) == H * kHead, "k: expected [>=T, Hkv*128]");
    MuxCacheWriteItem &it = items[i];
    it = MuxCacheWriteItem{};
    it.k = k.data_ptr();
    it.v = v.data_ptr();
    it.kv_row_stride = stride;
    it.slot_mapping = sm.data_ptr<int64_t>();
    it.layer = static_cast<int32_t>(layers[i]);
    it.num_layers = static_cast<int32_t>(sm.size(1));
    it.num_tokens = static_cast<int32_t>(T);
    it.num_kv_heads = static_cast<int32_t>(H);
    if (rope) {
      const at::Tensor &pos = positions[i], &q = qs[i], &cs = cos_sins[i];
      need_gpu({&pos, &q, &cs});
      TORCH_CHECK(pos.scalar_type() == at::kLong && pos.dim() == 1 && pos.is_contiguous() && pos.size(0) >= T,
                  "positions: expected contiguous int64 [>=T]");
      TORCH_CHECK(cs.scalar_type() == at::kFloat && cs.dim() == 2 && cs.is_contiguous(),
                  "cos_sin: expected contiguous float32 [max_position, rotary_dim]");
      TORCH_CHECK(q.dim() == 2 && q.scalar_type() == k.scalar_type() && q.size(0) >= T && q.size(1) % kHead == 0,
                  "q [>=T, Hq*128] of the dtype of k expected");
      it.positions = pos.data_ptr<int64_t>();
      it.cos_sin = cs.data_ptr<float>();
      it.max_position = static_cast<int32_t>(cs.size(0));
      it.rotary_dim = static_cast<int32_t>(cs.size(1));
      it.q = q.data_ptr();
      it.q_row_stride = rows(q, "q");
      it.num_q_heads = static_cast<int32_t>(q.size(1) / kHead);
    }
  }
  check(mux_multi_rope_reshape_and_cache(items, static_cast<int32_t>(n), k_pool.data_ptr(), v_pool.data_ptr(),
                                         k_pool.size(0), kHead, static_cast<int32_t>(bs), dtype_code(k_pool),
                                         stream_of(k_pool)),
        "mux_multi_rope_reshape_and_cache");
}

MuxDecodeItem decode_item(const at::Tensor &out, const at::Tensor &q, const at::Tensor &block_tables,
                          const at::Tensor &context_lens, int64_t max_context_len, double scale, int64_t layer,
                          int64_t total_context_len, const c10::optional<at::Tensor> &context_lens_host = c10::nullopt) {
  need_gpu({&out, &q, &block_tables, &context_lens});
  TORCH_CHECK(block_tables.scalar_type() == at::kInt && block_tables.dim() == 4 && block_tables.is_contiguous(),
              "block_tables: expected contiguous int32 [L, B, Hkv, max_blocks]");
  TORCH_CHECK(context_lens.scalar_type() == at::kInt && context_lens.dim() == 1 && context_lens.is_contiguous(),
              "context_lens: expected contiguous int32 [B]");
  const int64_t B = block_tables.size(1);
  TORCH_CHECK(context_lens.size(0) == B, "context_lens and block_tables disagree on the number of sequences");
  TORCH_CHECK(q.dim() == 2 && q.size(1) % kHead == 0 && q.size(0) >= B && out.sizes() == q.sizes() &&
                  q.scalar_type() == out.scalar_type(),
              "q/out: expected [>=B, Hq*128] of equal shape and dtype");
  MuxDecodeItem it = {};
  it.out = out.data_ptr();
  it.q = q.data_ptr();
  it.out_row_stride = rows(out, "out");
  it.q_row_stride = rows(q, "q");
  it.block_tables = block_tables.data_ptr<int32_t>();
  it.context_lens = context_lens.data_ptr<int32_t>();
  it.total_context_len = total_context_len;
  it.layer = static_cast<int32_t>(layer);
  it.num_layers = static_cast<int32_t>(block_tables.size(0));
  it.num_seqs = static_cast<int32_t>(B);
  it.num_q_heads = static_cast<int32_t>(q.size(1) / kHead);
  it.num_kv_heads = static_cast<int32_t>(block_tables.size(2));
  it.max_blocks = static_cast<int32_t>(block_tables.size(3));
  it.max_context_len = static_cast<int32_t>(max_context_len);
  it.scale = static_cast<float>(scale);
  it.context_lens_host = nullptr;
  if (context_lens_host.has_value() && context_lens_host->defined() && context_lens_host->numel() > 0) {
    const at::Tensor &h = *context_lens_host;
    TORCH_CHECK(h.is_cpu() && h.scalar_type() == at::kInt && h.dim() == 1 && h.is_contiguous() && h.size(0) == B,
                "context_lens_host: expected a contiguous CPU int32 [B] tensor");
    it.context_lens_host = h.data_ptr<int32_t>();      // read during this call only
  }
  return it;
}

// Bytes of workspace a decode call of these shapes needs (0: none).
int64_t paged_decode_workspace_bytes(const at::Tensor &out, const at::Tensor &q, const at::Tensor &block_tables,
                                     const at::Tensor &context_lens, int64_t max_context_len, int64_t partition_size) {
  const MuxDecodeItem it = decode_item(out, q, block_tables, context_lens, max_context_len, 1.0, 0, 0);
  return static_cast<int64_t>(mux_paged_decode_workspace_bytes(&it, 1, static_cast<int32_t>(partition_size)));
}

// workspace: uint8, at least paged_decode_workspace_bytes(...) bytes, zero-filled
// before its first use (every call leaves its counters zero); may be empty when
// that is 0.
void paged_decode(at::Tensor out, const at::Tensor &q, const at::Tensor &k_pool, const at::Tensor &v_pool,
                  const at::Tensor &block_tables, const at::Tensor &context_lens, int64_t max_context_len,
                  double scale, int64_t layer, int64_t partition_size, int64_t total_context_len,
                  at::Tensor workspace, const c10::optional<at::Tensor> &context_lens_host) {
  need_gpu({&k_pool, &v_pool});
  const int64_t bs = check_pools(k_pool, v_pool);
  TORCH_CHECK(q.scalar_type() == k_pool.scalar_type(), "q dtype must equal the pool dtype");
  const MuxDecodeItem it =
      decode_item(out, q, block_tables, context_lens, max_context_len, scale, layer, total_context_len,
                  context_lens_host);
  void *ws = nullptr;
  size_t ws_bytes = 0;
  if (workspace.defined() && workspace.numel() > 0) {
    TORCH_CHECK(workspace.is_cuda() && workspace.is_contiguous(), "workspace: expected a contiguous GPU tensor");
    ws = workspace.data_ptr();
    ws_bytes = static_cast<size_t>(workspace.numel()) * workspace.element_size();
  }
  check(mux_multi_decode(&it, 1, k_pool.data_ptr(), v_pool.data_ptr(), k_pool.size(0), kHead,
                         static_cast<int32_t>(bs), dtype_code(k_pool), static_cast<int32_t>(partition_size), ws,
                         ws_bytes, stream_of(q)),
        "mux_multi_decode");
}

// Several colocated models (different head counts, tables, q/out tensors) that
// share the pool, in one launch: element i of every list describes model i.
int64_t multi_decode_workspace_bytes(at::TensorList outs, at::TensorList qs, at::TensorList block_tables,
                                     at::TensorList context_lens, at::IntArrayRef max_context_lens,
                                     int64_t partition_size) {
  const size_t n = outs.size();
  TORCH_CHECK(n >= 1 && n <= MUXA_MAX_DECODE_ITEMS && qs.size() == n && block_tables.size() == n &&
                  context_lens.size() == n && max_context_lens.size() == n,
              "multi_decode: 1..", MUXA_MAX_DECODE_ITEMS, " models, one entry per model in every list");
  MuxDecodeItem items[MUXA_MAX_DECODE_ITEMS];
  for (size_t i = 0; i < n; ++i)
    items[i] = decode_item(outs[i], qs[i], block_tables[i], context_lens[i], max_context_lens[i], 1.0, 0, 0);
  return static_cast<int64_t>(
      mux_paged_decode_workspace_bytes(items, static_cast<int32_t>(n), static_cast<int32_t>(partition_size)));
}

void multi_decode(at::TensorList outs, at::TensorList qs, const at::Tensor &k_pool, const at::Tensor &v_pool,
                  at::TensorList block_tables, at::TensorList context_lens, at::IntArrayRef max_context_lens,
                  at::ArrayRef<double> scales, at::IntArrayRef layers, at::IntArrayRef total_context_lens,
                  int64_t partition_size, at::Tensor workspace, at::TensorList context_lens_host) {
  need_gpu({&k_pool, &v_pool});
  const int64_t bs = check_pools(k_pool, v_pool);
  const size_t n = outs.size();
  TORCH_CHECK(n >= 1 && n <= MUXA_MAX_DECODE_ITEMS && qs.size() == n && block_tables.size() == n &&
                  context_lens.size() == n && max_context_lens.size() == n && scales.size() == n &&
                  layers.size() == n && total_context_lens.size() == n &&
                  (context_lens_host.empty() || context_lens_host.size() == n),
              "multi_decode: 1..", MUXA_MAX_DECODE_ITEMS, " models, one entry per model in every list");
  MuxDecodeItem items[MUXA_MAX_DECODE_ITEMS];
  for (size_t i = 0; i < n; ++i) {
    TORCH_CHECK(qs[i].scalar_type() == k_pool.scalar_type(), "q dtype must equal the pool dtype");
    items[i] = decode_item(outs[i], qs[i], block_tables[i], context_lens[i], max_context_lens[i], scales[i],
                           layers[i], total_context_lens[i],
                           context_lens_host.empty() ? c10::nullopt : c10::optional<at::Tensor>(context_lens_host[i]));
  }
  void *ws = nullptr;
  size_t ws_bytes = 0;
  if (workspace.defined() && workspace.numel() > 0) {
    TORCH_CHECK(workspace.is_cuda() && workspace.is_contiguous(), "workspace: expected a contiguous GPU tensor");
    ws = workspace.data_ptr();
    ws_bytes = static_cast<size_t>(workspace.numel()) * workspace.element_size();
  }
  check(mux_multi_decode(items, static_cast<int32_t>(n), k_pool.data_ptr(), v_pool.data_ptr(), k_pool.size(0), kHead,
                         static_cast<int32_t>(bs), dtype_code(k_pool), static_cast<int32_t>(partition_size), ws,
                         ws_bytes, stream_of(k_pool)),
        "mux_multi_decode");
}

void rotary_neox(const at::Tensor &positions, at::Tensor q, at::Tensor k, const at::Tensor &cos_sin,
                 int64_t num_tokens) {
  need_gpu({&positions, &q, &k, &cos_sin});
  TORCH_CHECK(positions.scalar_type() == at::kLong && positions.dim() == 1 && positions.is_contiguous(),
              "positions: expected contiguous int64 [T]");
  TORCH_CHECK(cos_sin.scalar_type() == at::kFloat && cos_sin.dim() == 2 && cos_sin.is_contiguous(),
              "cos_sin: expected contiguous float32 [max_position, rotary_dim]");
  TORCH_CHECK(q.dim() == 2 && k.dim() == 2 && q.scalar_type() == k.scalar_type() && q.size(1) % kHead == 0 &&
                  k.size(1) % kHead == 0,
              "q [T, Hq*128], k [T, Hkv*128] of one dtype expected");
  const int64_t T = num_tokens < 0 ? positions.size(0) : num_tokens;
  TORCH_CHECK(std::min({q.size(0), k.size(0), positions.size(0)}) >= T, "fewer rows than tokens");
  check(mux_rotary_neox(positions.data_ptr<int64_t>(), q.data_ptr(), rows(q, "q"), k.data_ptr(), rows(k, "k"),
                        cos_sin.data_ptr<float>(), static_cast<int32_t>(cos_sin.size(0)),
                        static_cast<int32_t>(cos_sin.size(1)), static_cast<int32_t>(T),
                        static_cast<int32_t>(q.size(1) / kHead), static_cast<int32_t>(k.size(1) / kHead), kHead,
                        dtype_code(q), stream_of(q)),
        "mux_rotary_neox");
}

// GreedySampler.forward (muxserve/flexserver/sampler.py:15-35) without the
// logits: int64 [num_rows].  row_index: int32 rows of hidden_states to sample,
// or an empty tensor for rows 0 .. num_rows-1.  workspace: uint8,
// greedy_sample_workspace_bytes(vocab_size) bytes, zero-filled before its first
// use (every call leaves its counter zero).
int64_t greedy_sample_workspace_bytes(int64_t vocab_size) {
  return static_cast<int64_t>(mux_greedy_sample_workspace_bytes(static_cast<int32_t>(vocab_size)));
}

at::Tensor greedy_sample(const at::Tensor &embedding, const at::Tensor &hidden_states, int64_t vocab_size,
                         int64_t num_rows, const at::Tensor &row_index, at::Tensor workspace) {
  need_gpu({&embedding, &hidden_states, &workspace});
  TORCH_CHECK(embedding.dim() == 2 && hidden_states.dim() == 2 && embedding.size(1) == hidden_states.size(1) &&
                  embedding.scalar_type() == hidden_states.scalar_type(),
              "embedding [V, hidden] and hidden_states [T, hidden] of one dtype expected");
  const int32_t *ri = nullptr;
  if (row_index.defined() && row_index.numel() > 0) {
    TORCH_CHECK(row_index.is_cuda() && row_index.scalar_type() == at::kInt && row_index.dim() == 1 &&
                    row_index.is_contiguous() && row_index.size(0) >= num_rows,
                "row_index: expected contiguous int32 [>= num_rows] on the GPU");
    ri = row_index.data_ptr<int32_t>();
  } else {
    TORCH_CHECK(hidden_states.size(0) >= num_rows, "fewer rows of hidden states than sampled rows");
  }
  TORCH_CHECK(workspace.is_contiguous(), "workspace: expected a contiguous GPU tensor");
  at::Tensor out = at::empty({num_rows}, hidden_states.options().dtype(at::kLong));
  check(mux_greedy_sample(out.data_ptr<int64_t>(), hidden_states.data_ptr(), rows(hidden_states, "hidden_states"),
                          static_cast<int32_t>(hidden_states.size(0)), ri, static_cast<int32_t>(num_rows),
                          embedding.data_ptr(), rows(embedding, "embedding"), static_cast<int32_t>(embedding.size(0)),
                          static_cast<int32_t>(vocab_size), static_cast<int32_t>(hidden_states.size(1)),
                          dtype_code(hidden_states), workspace.data_ptr(),
                          static_cast<size_t>(workspace.numel()) * workspace.element_size(), stream_of(hidden_states)),
        "mux_greedy_sample");
  return out;
}

void prefill_causal(at::Tensor out, const at::Tensor &q, const at::Tensor &k, const at::Tensor &v,
                    const at::Tensor &cu_seqlens, at::IntArrayRef prompt_lens, int64_t max_prompt_len, double scale,
                    int64_t num_kv_heads) {
  need_gpu({&out, &q, &k, &v, &cu_seqlens});
  TORCH_CHECK(cu_seqlens.scalar_type() == at::kInt && cu_seqlens.dim() == 1 && cu_seqlens.is_contiguous() &&
                  cu_seqlens.size(0) >= 1,
              "cu_seqlens: expected contiguous int32 [P+1]");
  const int64_t P = cu_seqlens.size(0) - 1;
  TORCH_CHECK(q.dim() == 2 && q.size(1) % kHead == 0 && k.dim() == 2 && k.size(1) == num_kv_heads * kHead &&
                  k.sizes() == v.sizes(),
              "q [T, Hq*128], k/v [T, Hkv*128] expected");
  TORCH_CHECK(q.scalar_type() == k.scalar_type() && k.scalar_type() == v.scalar_type() &&
                  v.scalar_type() == out.scalar_type(),
              "q, k, v, out dtypes differ");
  const int64_t kv_stride = rows(k, "k");
  TORCH_CHECK(rows(v, "v") == kv_stride, "k and v row strides differ");
  // Host-side lengths (InputMetadata.prompt_lens): empty = not given.
  std::vector<int32_t> lens;
  if (!prompt_lens.empty()) {
    TORCH_CHECK(static_cast<int64_t>(prompt_lens.size()) == P, "prompt_lens: expected one length per prompt");
    lens.assign(prompt_lens.begin(), prompt_lens.end());
  }
  check(mux_prefill_causal(out.data_ptr(), rows(out, "out"), q.data_ptr(), rows(q, "q"), k.data_ptr(), v.data_ptr(),
                           kv_stride, cu_seqlens.data_ptr<int32_t>(), nullptr, lens.empty() ? nullptr : lens.data(),
                           static_cast<int32_t>(P), static_cast<int32_t>(max_prompt_len),
                           static_cast<int32_t>(q.size(1) / kHead), static_cast<int32_t>(num_kv_heads), kHead,
                           static_cast<float>(scale), dtype_code(q), stream_of(q)),
        "mux_prefill_causal");
}

// The prompts of several colocated models in one launch: element i of every
// list describes model i.  prompt_lens_host: CPU int32 [P_i] per model (the
// reference holds them on the host, InputMetadata.prompt_lens), or an empty
// list when none is given.
void multi_prefill_causal(at::TensorList outs, at::TensorList qs, at::TensorList ks, at::TensorList vs,
                          at::TensorList cu_seqlens, at::TensorList prompt_lens_host, at::IntArrayRef max_prompt_lens,
                          at::ArrayRef<double> scales, at::IntArrayRef num_kv_heads) {
  const size_t n = outs.size();
  TORCH_CHECK(n >= 1 && n <= MUXA_MAX_DECODE_ITEMS && qs.size() == n && ks.size() == n && vs.size() == n &&
                  cu_seqlens.size() == n && max_prompt_lens.size() == n && scales.size() == n &&
                  num_kv_heads.size() == n && (prompt_lens_host.empty() || prompt_lens_host.size() == n),
              "multi_prefill_causal: 1..", MUXA_MAX_DECODE_ITEMS, " models, one entry per model in every list");
  MuxPrefillItem items[MUXA_MAX_DECODE_ITEMS];
  for (size_t i = 0; i < n; ++i) {
    const at::Tensor &out = outs[i], &q = qs[i], &k = ks[i], &v = vs[i], &cu = cu_seqlens[i];
    need_gpu({&out, &q, &k, &v, &cu});
    TORCH_CHECK(cu.scalar_type() == at::kInt && cu.dim() == 1 && cu.is_contiguous() && cu.size(0) >= 1,
                "cu_seqlens: expected contiguous int32 [P+1]");
    const int64_t P = cu.size(0) - 1;
    TORCH_CHECK(q.dim() == 2 && q.size(1) % kHead == 0 && k.dim() == 2 && k.size(1) == num_kv_heads[i] * kHead &&
                    k.sizes() == v.sizes(),
                "q [T, Hq*128], k/v [T, Hkv*128] expected");
    TORCH_CHECK(q.scalar_type() == qs[0].scalar_type() && q.scalar_type() == k.scalar_type() &&
                    k.scalar_type() == v.scalar_type() && v.scalar_type() == out.scalar_type(),
                "q, k, v, out of all models must share one dtype");
    const int64_t kv_stride = rows(k, "k");
    TORCH_CHECK(rows(v, "v") == kv_stride, "k and v row strides differ");
    MuxPrefillItem &it = items[i];
    it = MuxPrefillItem{};
    it.out = out.data_ptr();
    it.out_row_stride = rows(out, "out");
    it.q = q.data_ptr();
    it.q_row_stride = rows(q, "q");
    it.k = k.data_ptr();
    it.v = v.data_ptr();
    it.kv_row_stride = kv_stride;
    it.cu_seqlens = cu.data_ptr<int32_t>();
    it.prompt_lens_host = nullptr;
    if (!prompt_lens_host.empty()) {
      const at::Tensor &h = prompt_lens_host[i];
      TORCH_CHECK(h.device().is_cpu() && h.scalar_type() == at::kInt && h.dim() == 1 && h.is_contiguous() &&
                      h.size(0) == P,
                  "prompt_lens_host: expected a contiguous CPU int32 tensor with one length per prompt");
      it.prompt_lens_host = h.data_ptr<int32_t>();
    }
    it.num_prompts = static_cast<int32_t>(P);
    it.max_prompt_len = static_cast<int32_t>(max_prompt_lens[i]);
    it.num_q_heads = static_cast<int32_t>(q.size(1) / kHead);
    it.num_kv_heads = static_cast<int32_t>(num_kv_heads[i]);
    it.scale = static_cast<float>(scales[i]);
  }
  check(mux_multi_prefill_causal(items, static_cast<int32_t>(n), kHead, dtype_code(qs[0]), stream_of(qs[0])),
        "mux_multi_prefill_causal");
}

at::Tensor rms_norm(const at::Tensor &x, const at::Tensor &weight, double eps) {
  need_gpu({&x, &weight});
  TORCH_CHECK(x.dim() == 2 && weight.dim() == 1 && weight.size(0) == x.size(1) &&
                  weight.scalar_type() == x.scalar_type() && weight.is_contiguous(),
              "x [T, hidden] and a contiguous weight [hidden] of the same dtype expected");
  at::Tensor out = at::empty_like(x, x.options(), at::MemoryFormat::Contiguous);
  check(mux_rms_norm(out.data_ptr(), rows(out, "out"), x.data_ptr(), rows(x, "x"), weight.data_ptr(),
                     static_cast<float>(eps), static_cast<int32_t>(x.size(0)), static_cast<int32_t>(x.size(1)),
                     dtype_code(x), stream_of(x)),
        "mux_rms_norm");
  return out;
}

at::Tensor silu_and_mul(const at::Tensor &x) {
  need_gpu({&x});
  TORCH_CHECK(x.dim() == 2 && x.size(1) % 2 == 0, "x: expected [T, 2 d]");
  const int64_t d = x.size(1) / 2;
  at::Tensor out = at::empty({x.size(0), d}, x.options());
  check(mux_silu_and_mul(out.data_ptr(), rows(out, "out"), x.data_ptr(), rows(x, "x"), static_cast<int32_t>(x.size(0)),
                         static_cast<int32_t>(d), dtype_code(x), stream_of(x)),
        "mux_silu_and_mul");
  return out;
}

}  // namespace

TORCH_LIBRARY(muxserve_amd, m) {
  m.def("reshape_and_cache(Tensor k, Tensor v, Tensor(a!) k_pool, Tensor(b!) v_pool, Tensor slot_mapping, "
        "int layer, int num_tokens) -> ()");
  m.def("rope_reshape_and_cache(Tensor positions, Tensor(a!) q, Tensor(b!) k, Tensor v, Tensor cos_sin, "
        "Tensor(c!) k_pool, Tensor(d!) v_pool, Tensor slot_mapping, int layer, int num_tokens) -> ()");
  m.def("multi_reshape_and_cache(Tensor(a!)[] ks, Tensor[] vs, Tensor(b!) k_pool, Tensor(c!) v_pool, "
        "Tensor[] slot_mappings, int[] layers, int[] num_tokens, Tensor[] positions, Tensor(d!)[] qs, "
        "Tensor[] cos_sins) -> ()");
  m.def("paged_decode_workspace_bytes(Tensor out, Tensor q, Tensor block_tables, Tensor context_lens, "
        "int max_context_len, int partition_size) -> int");
  m.def("paged_decode(Tensor(a!) out, Tensor q, Tensor k_pool, Tensor v_pool, Tensor block_tables, "
        "Tensor context_lens, int max_context_len, float scale, int layer, int partition_size, "
        "int total_context_len, Tensor(b!) workspace, Tensor? context_lens_host=None) -> ()");
  m.def("prefill_causal(Tensor(a!) out, Tensor q, Tensor k, Tensor v, Tensor cu_seqlens, int[] prompt_lens, "
        "int max_prompt_len, float scale, int num_kv_heads) -> ()");
  m.def("multi_prefill_causal(Tensor(a!)[] outs, Tensor[] qs, Tensor[] ks, Tensor[] vs, Tensor[] cu_seqlens, "
        "Tensor[] prompt_lens_host, int[] max_prompt_lens, float[] scales, int[] num_kv_heads) -> ()");
  m.def("multi_decode_workspace_bytes(Tensor[] outs, Tensor[] qs, Tensor[] block_tables, Tensor[] context_lens, "
        "int[] max_context_lens, int partition_size) -> int");
  m.def("multi_decode(Tensor(a!)[] outs, Tensor[] qs, Tensor k_pool, Tensor v_pool, Tensor[] block_tables, "
        "Tensor[] context_lens, int[] max_context_lens, float[] scales, int[] layers, int[] total_context_lens, "
        "int partition_size, Tensor(b!) workspace, Tensor[] context_lens_host) -> ()");
  m.def("rotary_neox(Tensor positions, Tensor(a!) q, Tensor(b!) k, Tensor cos_sin, int num_tokens) -> ()");
  m.def("greedy_sample_workspace_bytes(int vocab_size) -> int", &greedy_sample_workspace_bytes);
  m.def("greedy_sample(Tensor embedding, Tensor hidden_states, int vocab_size, int num_rows, Tensor row_index, "
        "Tensor(a!) workspace) -> Tensor");
  m.def("rms_norm(Tensor x, Tensor weight, float eps) -> Tensor");
  m.def("silu_and_mul(Tensor x) -> Tensor");
}

TORCH_LIBRARY_IMPL(muxserve_amd, CUDA, m) {
  m.impl("reshape_and_cache", &reshape_and_cache);
  m.impl("rope_reshape_and_cache", &rope_reshape_and_cache);
  m.impl("multi_reshape_and_cache", &multi_reshape_and_cache);
  m.impl("paged_decode_workspace_bytes", &paged_decode_workspace_bytes);
  m.impl("paged_decode", &paged_decode);
  m.impl("prefill_causal", &prefill_causal);
  m.impl("multi_prefill_causal", &multi_prefill_causal);
  m.impl("multi_decode_workspace_bytes", &multi_decode_workspace_bytes);
  m.impl("multi_decode", &multi_decode);
  m.impl("rotary_neox", &rotary_neox);
  m.impl("greedy_sample", &greedy_sample);
  m.impl("rms_norm", &rms_norm);
  m.impl("silu_and_mul", &silu_and_mul);
}
