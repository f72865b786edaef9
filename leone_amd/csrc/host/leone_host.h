// The C interface of the host library: cache manager, scheduler and step layout behind opaque
// handles.  Calls return 0 or a count on success and a negative code on failure; the message of the
// last failure on the calling thread is leone_host_last_error().  A failed call changes nothing.
#pragma once

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    LEONE_HOST_MISUSE = -1,          // the cache manager was used against its contract
    LEONE_HOST_OUT_OF_PAGES = -2,    // see leone_cache_shortage
    LEONE_HOST_OUT_OF_SLOTS = -3,
    LEONE_HOST_SCHEDULER = -4,
    LEONE_HOST_STEP_REFUSED = -5,
    LEONE_HOST_INVALID = -6,
    LEONE_HOST_SAMPLER = -7,
};

const char* leone_host_last_error(void);

// ---- cache manager.  groups: n_groups x (num_pages, page_tokens, window or 0).
void* leone_cache_create(const int* groups, int n_groups, int max_requests, int max_context);
void leone_cache_destroy(void* cache);
int leone_cache_admit(void* cache, int64_t request);                                  // the state slot
int leone_cache_fork(void* cache, int64_t parent, int64_t child, int tokens);         // tokens the child holds
int leone_cache_truncate(void* cache, int64_t request, int position);
int leone_cache_reserve(void* cache, int64_t request, int tokens);
int leone_cache_commit(void* cache, int64_t request, int tokens);                     // tokens < 0: as reserved
int leone_cache_rollback(void* cache, int64_t request);
int leone_cache_release(void* cache, int64_t request);
int leone_cache_has(void* cache, int64_t request);
int leone_cache_requests(void* cache, int64_t* out, int capacity);                    // admitted, ascending
int leone_cache_length(void* cache, int64_t request);
int leone_cache_pending(void* cache, int64_t request);
int leone_cache_slot(void* cache, int64_t request);
int leone_cache_table(void* cache, int64_t request, int group, int* out, int capacity);   // blocks in the table
int leone_cache_pages_needed(void* cache, int64_t request, int tokens, int* out);         // one count per group
int leone_cache_free_pages(void* cache, int group);
int leone_cache_free_list(void* cache, int group, int* out, int capacity);
int leone_cache_free_slots(void* cache);
int leone_cache_free_slot_list(void* cache, int* out, int capacity);
int leone_cache_holders(void* cache, int group, int page);
int leone_cache_shared_pages(void* cache, int group);
int leone_cache_high_water(void* cache, int group);
int leone_cache_log_freed(void* cache, int on);                                       // note pages as they become free
int leone_cache_drain_freed(void* cache, int group, int* out, int capacity);          // the notes so far; clears them
int leone_cache_max_blocks(void* cache, int group);
void leone_cache_shortage(int* group, int* needed, int* free);   // of the last LEONE_HOST_OUT_OF_PAGES

// ---- scheduler.  policy: max_live_requests, max_queued_requests, max_step_tokens,
// prefill_chunk_tokens, max_prompt_tokens, max_output_tokens.  The cache must outlive the scheduler.
void* leone_scheduler_create(void* cache, const int64_t* policy);
void leone_scheduler_destroy(void* scheduler);
// 0 queued, else the reject reason (1 prompt-limit, 2 output-limit, 3 context-limit, 4 kv-capacity,
// 5 queue-limit, 6 duplicate).  eos < 0: no end token.
int leone_scheduler_submit(void* scheduler, int64_t request, const int32_t* prompt, int prompt_tokens,
                           int64_t max_new_tokens, int eos);
int leone_scheduler_cancel(void* scheduler, int64_t request);
int leone_scheduler_has_work(void* scheduler);
int leone_scheduler_plan(void* scheduler);     // number of entries
// The planned entries: request, start, count, sample for each.
int leone_scheduler_planned(void* scheduler, int64_t* requests, int* starts, int* counts, int* samples, int capacity);
// One step beyond the planned one, before its tokens are known (Scheduler::plan_ahead): number of entries, 0 if
// the next step cannot be known yet; leone_scheduler_ahead lists them as leone_scheduler_planned does.
int leone_scheduler_plan_ahead(void* scheduler);
int leone_scheduler_ahead(void* scheduler, int64_t* requests, int* starts, int* counts, int* samples, int capacity);
int leone_scheduler_complete(void* scheduler, const int64_t* requests, const int32_t* tokens, int n);   // finished now
int leone_scheduler_abort(void* scheduler);
int leone_scheduler_history(void* scheduler, int64_t request, int32_t* out, int capacity);    // tokens known
int leone_scheduler_tokens(void* scheduler, int64_t request, int start, int count, int32_t* out);   // history [start, start + count)
int leone_scheduler_request_info(void* scheduler, int64_t request, int* prompt_tokens, int* preemptions);
int leone_scheduler_live(void* scheduler, int64_t* out, int capacity);
int leone_scheduler_queued(void* scheduler, int64_t* out, int capacity);
int leone_scheduler_finished_count(void* scheduler);
// reason: 0 eos, 1 length, 2 cancelled, 3 aborted.
int leone_scheduler_finished_info(void* scheduler, int index, int64_t* request, int* reason, int* preemptions,
                                  int* prompt_tokens, int* generated_tokens);
int leone_scheduler_finished_tokens(void* scheduler, int index, int32_t* prompt, int32_t* generated);
int leone_scheduler_event_count(void* scheduler);
// kinds: 0 reject (a = reason), 1 submit, 2 step begins (a = entries), 3 step entry (a = start,
// b = count, c = sample), 4 admit, 5 preempt (a = tokens known), 6 token (a = position, b = token),
// 7 finish (a = reason).  Copies events [first, first + count).
int leone_scheduler_events(void* scheduler, int first, int count, int* kinds, int64_t* requests, int* a, int* b, int* c);
void leone_scheduler_stats(void* scheduler, int64_t* out15);

// ---- step layout.  Entries are given flat: request, token count and wanted count per entry, then
// all tokens and all wanted places in entry order.  shape: vocab_size, all_rows_wanted, the number of
// row tilings, then (tile_rows, min_rows, group_tiles) of each.  Returns the words the packed step takes;
// writes nothing but `sections` (6 + tilings + groups offsets) if `capacity` is smaller.  summary: rows,
// max_position, wanted, decode_only, then (tiled rows, tiles) of each tiling.  placed: per entry in running
// order given_index, slot, first_row, count, start.
long leone_step_pack(void* cache, int n_entries, const int64_t* requests, const int* counts, const int* want_counts,
                     const int32_t* tokens, const int32_t* wants, const int* shape, int32_t* out, long capacity,
                     long* sections, int* summary, int* placed);

// ---- sampling on the host, in double.  `rows` rows of `vocab` float logits; row r is drawn at
// temperature[r] after its stage_counts[r] truncation stages (kinds 0 top-k, 1 top-p, 2 min-p with
// their values, one row's stages after the other's) with the uniform value uniform[r]; tokens[r] is the
// token, -1 for a row without a finite logit.
int leone_sample_rows(const float* logits, int rows, int vocab, const double* temperature, const int* stage_counts,
                      const int* stage_kinds, const double* stage_values, const double* uniform, int* tokens);

// ---- scalar single-precision reference of the kernel entry points, on host memory (scalar_reference.cpp).
// Arguments as the kernels', float32 only, no stream; for comparison, never on the product path.
int leone_ref_embed(const float* table, const int* tokens, float* out, int rows, int hidden, int vocab);
int leone_ref_add_rmsnorm(float* x, const float* delta, int planes, long plane, const float* gain, float eps,
                          float* y, const int* rows, int n_rows, int hidden);
int leone_ref_rope_table(float* cos_out, float* sin_out, double theta, int rotary_dim, int positions);
int leone_ref_qk_norm_rope_write(const float* qkv, int planes, long plane, float* q_out, float* k_pool, float* v_pool,
                                 const float* q_gain, const float* k_gain, float eps, const float* cos_table,
                                 const float* sin_table, int table_positions, int rotary_dim, int pairing,
                                 const int* positions, const int* row_entry, const int* block_table, int max_blocks,
                                 int rows, int q_heads, int kv_heads, int head_dim, int page_tokens, int write_cache);
int leone_ref_attention(const float* q, float* out, const float* k_pool, const float* v_pool, const int* positions,
                        const int* row_entry, const int* block_table, int max_blocks, int rows, int q_heads,
                        int kv_heads, int head_dim, int page_tokens, float scale, int window);
int leone_ref_gemm(const float* a, const float* b, float* c, int m, int n, int k);
int leone_ref_swiglu(const float* gate_up, float* out, int rows, int ffn);
int leone_ref_argmax(const float* logits, int* out, int rows, int vocab);
int leone_ref_sample_temperature(const float* logits, const double* temperature, const double* uniform, int* out,
                                 int rows, int vocab);

#ifdef __cplusplus
}
#endif
