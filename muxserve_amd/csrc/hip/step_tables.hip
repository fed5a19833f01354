// Device-side construction of a step's index tensors, gfx950.
//
// The reference builds slot_mapping [tokens, L, H] and the block table on the
// host every step and uploads them (csrc/batch_scheduler.cpp:131-169,
// muxserve/flexserver/llm_runtime.py:301-327).  Here the device keeps a mirror
// of every live request's block-id run in the reference's own order,
//     mirror[row][token block][layer][head]          (csrc/batch_scheduler.h:19,44-52)
// and a step uploads only the allocator's reply plus 8 ints per sequence
// (mux_sched_get_batch_compact).  Three small kernels, all plain coalesced
// integer copies bound by HBM:
//   append   the reply's new ids are copied behind each request's run
//   slots    slot_mapping[t][l][h] = id * block_size + offset, read from the
//            mirror: prompt token k -> block k / bs, offset k % bs; decode token ->
//            last block, offset (ctx - 1) % bs    (csrc/batch_scheduler.h:42-67)
//   table    decode steps: mirror rows transposed through LDS into the layout the
//            attention kernel reads, [L][sequence][H][token block]
// Results are bit-identical to what mux_sched_get_batch writes.
#include "mux_common.h"

namespace mux {

constexpr int kDescInts = 8;   // row, blocks, first new block, new blocks, offset in reply, length, first token, decoding

struct StepParams {
  int32_t *mirror;               // [max_rows][max_blocks_per_seq][per]
  const int32_t *desc;           // [num_seqs][kDescInts]
  const int32_t *block_info;     // the allocator's reply, [n_block_info]
  int64_t *slot_mapping;         // [num_tokens][per]
  int32_t *block_tables;         // [L][num_seqs][H][max_blocks_out]
  int64_t n_block_info;
  int32_t num_seqs, per, H, max_rows, max_blocks_per_seq, block_size, max_blocks_out, num_tokens;
};

// A descriptor that does not fit the mirror or the reply is skipped, never followed.
__device__ __forceinline__ bool desc_ok(const StepParams &P, const int32_t *d) {
  const int64_t count = static_cast<int64_t>(d[3]) * P.per;
  return d[0] >= 0 && d[0] < P.max_rows && d[1] >= 0 && d[1] <= P.max_blocks_per_seq && d[2] >= 0 && d[3] >= 0 &&
         static_cast<int64_t>(d[2]) + d[3] <= d[1] && d[4] >= 1 && d[4] + count <= P.n_block_info && d[5] >= 0 && d[6] >= 0;
}

__global__ __launch_bounds__(256) void step_append_kernel(const StepParams P) {
  const int32_t *d = P.desc + blockIdx.y * kDescInts;
  if (!desc_ok(P, d)) return;
  const int64_t count = static_cast<int64_t>(d[3]) * P.per;
  const int64_t begin = static_cast<int64_t>(blockIdx.x) * 1024;
  const int64_t end = min(count, begin + 1024);
  int32_t *dst = P.mirror + (static_cast<int64_t>(d[0]) * P.max_blocks_per_seq + d[2]) * P.per;
  const int32_t *src = P.block_info + d[4];
  for (int64_t e = begin + threadIdx.x; e < end; e += 256) dst[e] = src[e];
}

__global__ __launch_bounds__(256) void step_slots_kernel(const StepParams P) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63;
  // The batch entry that owns token t: the last one whose first token is <= t.
  int before = 0;
  for (int base = 0; base < P.num_seqs; base += 64) {
    const int i = base + lane;
    const int first = i < P.num_seqs ? P.desc[i * kDescInts + 6] : 0x7fffffff;
    before += __popcll(__builtin_amdgcn_ballot_w64(first <= t));
  }
  if (before == 0) return;
  const int32_t *d = P.desc + (before - 1) * kDescInts;
  if (!desc_ok(P, d)) return;
  int tb, off;
  if (d[7]) {                                 // decoding: the token just appended
    tb = d[1] - 1;
    off = (d[5] - 1) % P.block_size;
    if (t != d[6] || d[5] < 1) return;
  } else {
    const int k = t - d[6];
    if (k >= d[5]) return;
    tb = k / P.block_size;
    off = k % P.block_size;
  }
  if (tb < 0 || tb >= d[1]) return;
  const int32_t *ids = P.mirror + (static_cast<int64_t>(d[0]) * P.max_blocks_per_seq + tb) * P.per;
  int64_t *out = P.slot_mapping + static_cast<int64_t>(t) * P.per;
  for (int j = blockIdx.y * 1024 + threadIdx.x; j < min(P.per, (static_cast<int>(blockIdx.y) + 1) * 1024); j += 256)
    out[j] = static_cast<int64_t>(ids[j]) * P.block_size + off;
}

// One 64 x 64 tile of a sequence's [token block][layer, head] matrix, transposed.
__global__ __launch_bounds__(256) void step_table_kernel(const StepParams P) {
  __shared__ int32_t tile[64][65];
  const int c = blockIdx.z;
  const int32_t *d = P.desc + c * kDescInts;
  const bool ok = desc_ok(P, d) && d[7];
  const int n_blocks = ok ? d[1] : 0;
  const int j0 = blockIdx.x * 64, tb0 = blockIdx.y * 64;
  const int x = threadIdx.x & 63, y = threadIdx.x >> 6;
  if (n_blocks > tb0) {
    const int32_t *src = P.mirror + static_cast<int64_t>(d[0]) * P.max_blocks_per_seq * P.per;
#pragma unroll 4
    for (int r = y; r < 64; r += 4) {
      const int tb = tb0 + r, j = j0 + x;
      tile[r][x] = (tb < n_blocks && j < P.per) ? src[static_cast<int64_t>(tb) * P.per + j] : 0;
    }
  }
  __syncthreads();
#pragma unroll 4
  for (int r = y; r < 64; r += 4) {
    const int j = j0 + r, tb = tb0 + x;
    if (j < P.per && tb < P.max_blocks_out) {
      const int l = j / P.H, h = j - l * P.H;
      // Entries past the sequence's blocks are never read; zero keeps them defined.
      P.block_tables[((static_cast<int64_t>(l) * P.num_seqs + c) * P.H + h) * P.max_blocks_out + tb] =
          tb < n_blocks ? tile[x][r] : 0;
    }
  }
}

}  // namespace mux

extern "C" int32_t mux_build_step_inputs(int32_t *mirror, int32_t max_rows, int32_t max_blocks_per_seq,
                                         int32_t num_layers, int32_t num_heads, int32_t block_size,
                                         const int32_t *desc, int32_t num_seqs, const int32_t *block_info,
                                         int64_t n_block_info, int32_t max_new_blocks, int32_t num_tokens,
                                         int64_t *slot_mapping, int32_t *block_tables, int32_t max_blocks_out,
                                         void *stream) {
  using namespace mux;
  if (!mirror || max_rows <= 0 || max_blocks_per_seq <= 0 || num_layers <= 0 || num_heads <= 0 || block_size <= 0)
    return MUXA_EINVAL;
  if (num_seqs < 0 || num_tokens < 0 || n_block_info < 1 || max_new_blocks < 0 || max_blocks_out < 0) return MUXA_EINVAL;
  if (num_seqs == 0) return MUXA_OK;
  if (!desc || !block_info || (num_tokens > 0 && !slot_mapping) || (max_blocks_out > 0 && !block_tables))
    return MUXA_EINVAL;
  const int64_t per = static_cast<int64_t>(num_layers) * num_heads;
  // Grid limits: y and z dimensions hold at most 65535 workgroups.
  if (per > 65535 * 1024 || num_seqs > 65535 || max_blocks_out > 65535 * 64 ||
      static_cast<int64_t>(max_new_blocks) * per > (int64_t{1} << 40))
    return MUXA_EUNSUPPORTED;
  StepParams P;
  P.mirror = mirror;
  P.desc = desc;
  P.block_info = block_info;
  P.slot_mapping = slot_mapping;
  P.block_tables = block_tables;
  P.n_block_info = n_block_info;
  P.num_seqs = num_seqs;
  P.per = static_cast<int32_t>(per);
  P.H = num_heads;
  P.max_rows = max_rows;
  P.max_blocks_per_seq = max_blocks_per_seq;
  P.block_size = block_size;
  P.max_blocks_out = max_blocks_out;
  P.num_tokens = num_tokens;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (max_new_blocks > 0) {
    const int64_t chunks = (static_cast<int64_t>(max_new_blocks) * per + 1023) / 1024;
    if (chunks > 0x7fffffff) return MUXA_EUNSUPPORTED;
    hipLaunchKernelGGL(step_append_kernel, dim3(static_cast<uint32_t>(chunks), num_seqs), dim3(256), 0, st, P);
  }
  if (num_tokens > 0)
    hipLaunchKernelGGL(step_slots_kernel, dim3(num_tokens, static_cast<uint32_t>((per + 1023) / 1024)), dim3(256), 0,
                       st, P);
  if (max_blocks_out > 0)
    hipLaunchKernelGGL(step_table_kernel,
                       dim3(static_cast<uint32_t>((per + 63) / 64), (max_blocks_out + 63) / 64, num_seqs), dim3(256), 0,
                       st, P);
  MUX_HIP_TRY(hipGetLastError());
  return MUXA_OK;
}
