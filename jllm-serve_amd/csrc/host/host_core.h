// The host side of the engine that is native: the page pool and the builder of a step's index arrays. Plain C
// entry points (called through ctypes), no GPU code: this library loads on a machine without a GPU.
#pragma once
#include <stdint.h>

extern "C" {

// ---- page pool: a page is either free or held; alloc never returns a held page; the release of the last reference
// makes it free at once (the contract of the reference's pool, kv/KvPool.java:249-302)
void* jllm_pool_new(int num_pages);
void jllm_pool_delete(void* pool);
int jllm_pool_alloc(void* pool);                               // page id, or -1 when no page is free
int jllm_pool_alloc_many(void* pool, int n, int32_t* out);     // n pages or none: 0, or -1 when fewer are free
int jllm_pool_retain(void* pool, int page);                    // 0, or -1 when the page is not held
int jllm_pool_release(void* pool, int page);                   // references left, or -1 when the page is not held
int jllm_pool_refs(void* pool, int page);                      // -1 for a page that does not exist
int jllm_pool_free_pages(void* pool);
int jllm_pool_high_water(void* pool);
int64_t jllm_pool_allocations(void* pool);
int jllm_pool_free_list(void* pool, int32_t* out);             // copies the free list, next page to be handed out last
int jllm_pool_set_free_list(void* pool, const int32_t* order, int n);  // the same pages in another order: 0 / -1
int jllm_pool_check(void* pool, int* page);                    // 0; 1 a page twice on the free list; 2 references and list disagree

// ---- a step's index arrays, in this order: token ids [T], positions [T], row -> request [T], state slots [R],
// selected rows [S], then per group of layers: cache slot of every row [T] (page * page_size + offset, -1 for a
// padded row) and the block tables [R][width] (entries never read are 0, a valid page).
struct JllmStepSizes {
  int32_t T, R, S, width, max_context;
};
// Entry i brings n_tokens[i] >= 1 tokens (concatenated in `tokens`, tokens_len in all) at positions pos0[i] .., wants
// want_counts[i] of its places (concatenated in `wants`, wants_len in all, each below n_tokens[i]), and its block table
// in group g is row table_rows[i] (below arena_rows) of arena[g] (arena_stride[g] entries per row, table_lens[g][row]
// of them in use). pad_rows > 0: the arrays describe that many single-row requests (the extra ones read one key of
// page 0, store nothing and have pad_state_slot, a row of the state tensors that no live request holds, as their
// state) and every row is selected.
struct JllmStepBatch {
  int32_t n_entries;
  const int32_t* n_tokens;
  const int32_t* pos0;
  const int32_t* state_slots;
  const int32_t* tokens;
  int64_t tokens_len;
  const int32_t* want_counts;
  const int32_t* wants;
  int64_t wants_len;
  int32_t pad_rows;
  int32_t pad_state_slot;
  int32_t min_width;
  int32_t page_size;
  int32_t n_groups;
  int32_t arena_rows;
  const int32_t* const* arena;
  const int64_t* arena_stride;
  const int32_t* table_rows;
  const int32_t* const* table_lens;
};
// Returns the number of int32 written; -1 when `capacity` is too small (sizes are filled in, nothing else is
// written); -2 when a row would be written into a page that was given back or that the table does not have; -3 when
// the batch contradicts itself (a count or position below zero, a wanted place outside its entry, sums that differ
// from tokens_len / wants_len, a table row outside the arena, a table longer than its row, a page size that is no
// power of two): nothing is read beyond the stated lengths.
int64_t jllm_step_layout(const JllmStepBatch* batch, int32_t* out, int64_t capacity, JllmStepSizes* sizes);

int jllm_host_abi_version();
}
