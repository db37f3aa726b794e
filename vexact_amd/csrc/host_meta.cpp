// Host-side (CPU) step metadata and KV block allocator: the integer work the inference loop does
// before every step, as native code behind the same C ABI as the kernels. No device code here.
//   * vx_host_step_metadata: slot mapping, positions, query_start_loc, context lengths and block
//     tables of one step, written straight into buffers of a captured bucket's size with the
//     static-buffer padding (replaces the Python loops of _prepare_gen_ctx and the padding of
//     prepare_cudagraph_gen_ctx, vexact/inferencer/inferencer.py:193-291, 306-324)
//   * vx_kv_allocator_*: lowest-free-id block allocator (KVCacheManager,
//     vexact/batch_invariant_ops/kv_cache_context.py:141-217), a min-heap instead of a set scan
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <functional>
#include <new>
#include <queue>
#include <vector>

// status codes of the C ABI (the same values as the kernels' entry points return)
enum : int { VX_OK = 0, VX_ERR_ARG = -1 };

extern "C" {

// requests s = 0..num_reqs-1: num_computed[s] = context length after this step, tokens_this_step[s]
// = query tokens of this step, block ids block_ids[block_offsets[s] .. block_offsets[s+1]).
// Outputs are sized for the bucket: positions / slot_mapping [cap_tokens], query_start_loc
// [cap_seqs + 1], context_lens [cap_seqs], block_tables [cap_seqs, max_blocks]. Padding: tokens past
// the step get slot -1 and position 0; sequences past the step get query_start_loc = total tokens,
// context length 0 and an all-zero block-table row; unused block-table entries of real rows are -1.
// seq_order [cap_seqs] (optional) receives the sequences sorted by context length, longest first,
// ties and padding in index order: the order in which the decode attention kernel should take them.
// Returns VX_OK and the step's token count / longest query in *total_tokens / *max_seqlen_q, or
// VX_ERR_ARG when the step does not fit the bucket, a request has too few blocks for its context,
// or its counts are inconsistent.
int vx_host_step_metadata(int64_t num_reqs, const int64_t* num_computed, const int64_t* tokens_this_step,
                          const int32_t* block_ids, const int64_t* block_offsets, int32_t page_size,
                          int64_t max_blocks, int64_t cap_tokens, int64_t cap_seqs, int64_t* positions,
                          int32_t* slot_mapping, int32_t* query_start_loc, int32_t* context_lens,
                          int32_t* block_tables, int32_t* seq_order, int64_t* total_tokens, int32_t* max_seqlen_q) {
  if (num_reqs < 0 || page_size <= 0 || max_blocks <= 0 || cap_tokens < 0 || cap_seqs < num_reqs) return VX_ERR_ARG;
  if (!positions || !slot_mapping || !query_start_loc || !context_lens || !block_tables) return VX_ERR_ARG;
  if (num_reqs > 0 && (!num_computed || !tokens_this_step || !block_ids || !block_offsets)) return VX_ERR_ARG;
  int64_t total = 0;
  int64_t maxq = 0;
  for (int64_t s = 0; s < num_reqs; s++) {
    const int64_t n = tokens_this_step[s], done = num_computed[s];
    const int64_t nb = block_offsets[s + 1] - block_offsets[s];
    if (n < 0 || done < n || nb < 0 || nb > max_blocks) return VX_ERR_ARG;
    if ((done + page_size - 1) / page_size > nb) return VX_ERR_ARG;  // context does not fit its blocks
    if (done > 0x7fffffffLL) return VX_ERR_ARG;
    total += n;
    maxq = std::max(maxq, n);
  }
  if (total > cap_tokens || total > 0x7fffffffLL) return VX_ERR_ARG;

  int64_t i = 0;
  query_start_loc[0] = 0;
  for (int64_t s = 0; s < num_reqs; s++) {
    const int64_t n = tokens_this_step[s], done = num_computed[s];
    const int32_t* ids = block_ids + block_offsets[s];
    const int64_t nb = block_offsets[s + 1] - block_offsets[s];
    int32_t* row = block_tables + s * max_blocks;
    std::memcpy(row, ids, (size_t)nb * sizeof(int32_t));
    std::fill(row + nb, row + max_blocks, -1);
    for (int64_t pos = done - n; pos < done; pos++, i++) {
      positions[i] = pos;
      slot_mapping[i] = (int32_t)((int64_t)ids[pos / page_size] * page_size + pos % page_size);
    }
    context_lens[s] = (int32_t)done;
    query_start_loc[s + 1] = (int32_t)i;
  }
  for (; i < cap_tokens; i++) {
    positions[i] = 0;
    slot_mapping[i] = -1;
  }
  for (int64_t s = num_reqs; s < cap_seqs; s++) {
    query_start_loc[s + 1] = (int32_t)total;
    context_lens[s] = 0;
    std::fill(block_tables + s * max_blocks, block_tables + (s + 1) * max_blocks, 0);
  }
  if (seq_order) {
    for (int64_t s = 0; s < cap_seqs; s++) seq_order[s] = (int32_t)s;
    std::stable_sort(seq_order, seq_order + cap_seqs,
                     [&](int32_t a, int32_t b) { return context_lens[a] > context_lens[b]; });
  }
  if (total_tokens) *total_tokens = total;
  if (max_seqlen_q) *max_seqlen_q = (int32_t)maxq;
  return VX_OK;
}

// ---- block allocator: always hands out the lowest free ids ----------------------------------
struct VxKvAllocator {
  std::priority_queue<int32_t, std::vector<int32_t>, std::greater<int32_t>> heap;
  std::vector<uint8_t> is_free;
  int64_t num_free;
};

void* vx_kv_allocator_create(int64_t num_blocks) {
  if (num_blocks < 0 || num_blocks > 0x7fffffffLL) return nullptr;
  VxKvAllocator* a = new (std::nothrow) VxKvAllocator();
  if (!a) return nullptr;
  std::vector<int32_t> ids((size_t)num_blocks);
  for (int64_t b = 0; b < num_blocks; b++) ids[(size_t)b] = (int32_t)b;
  a->heap = std::priority_queue<int32_t, std::vector<int32_t>, std::greater<int32_t>>(std::greater<int32_t>(), std::move(ids));
  a->is_free.assign((size_t)num_blocks, 1);
  a->num_free = num_blocks;
  return a;
}

void vx_kv_allocator_destroy(void* h) { delete static_cast<VxKvAllocator*>(h); }

int64_t vx_kv_allocator_num_free(const void* h) { return h ? static_cast<const VxKvAllocator*>(h)->num_free : -1; }

// Blocks needed so that a request holding num_current_blocks covers total_tokens. Writes the new
// ids (ascending) to out and returns their number (0 if none are needed); returns -1, allocating
// nothing, when fewer than that are free or out_capacity is too small.
int64_t vx_kv_allocator_allocate(void* h, int64_t total_tokens, int64_t num_current_blocks, int32_t page_size,
                                 int32_t* out, int64_t out_capacity) {
  VxKvAllocator* a = static_cast<VxKvAllocator*>(h);
  if (!a || page_size <= 0 || total_tokens < 0 || num_current_blocks < 0) return -1;
  const int64_t delta = (total_tokens + page_size - 1) / page_size - num_current_blocks;
  if (delta <= 0) return 0;
  if (a->num_free < delta || out_capacity < delta || !out) return -1;
  for (int64_t i = 0; i < delta; i++) {
    const int32_t b = a->heap.top();
    a->heap.pop();
    a->is_free[(size_t)b] = 0;
    out[i] = b;
  }
  a->num_free -= delta;
  return delta;
}

// Returns blocks to the pool; ids that are out of range or already free are ignored (as the reference
// ignores ids it did not hand out). Returns the number actually freed.
int64_t vx_kv_allocator_free(void* h, const int32_t* ids, int64_t n) {
  VxKvAllocator* a = static_cast<VxKvAllocator*>(h);
  if (!a || (n > 0 && !ids)) return -1;
  int64_t freed = 0;
  for (int64_t i = 0; i < n; i++) {
    const int32_t b = ids[i];
    if (b < 0 || (size_t)b >= a->is_free.size() || a->is_free[(size_t)b]) continue;
    a->is_free[(size_t)b] = 1;
    a->heap.push(b);
    freed++;
  }
  a->num_free += freed;
  return freed;
}

}  // extern "C"
