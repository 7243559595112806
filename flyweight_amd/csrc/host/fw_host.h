// Host side of the engine behind a flat C ABI: the cache's bookkeeping (page pools, block
// tables, state slots) and the continuous-batching scheduler. Nothing here touches the GPU; the
// Python package holds the tensors and launches the kernels, and asks this library who holds
// which page and what the next step runs. Built with the host compiler alone.
//
// Conventions: a request is a 64-bit id chosen by the caller. Functions return >= 0 on success
// and a negative code on error, with the text in fwh_last_error() (per thread). FWH_OUT_OF_PAGES
// is the one expected failure: nothing was changed.
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FWH_ERROR (-1)
#define FWH_OUT_OF_PAGES (-2)
#define FWH_NO_PAGE (-1)

const char* fwh_last_error(void);
int fwh_abi_version(void);

// ---- a LIFO pool of page (or slot) ids: the id given back last is handed out next ---------------
void* fwh_pool_create(int size);
void fwh_pool_destroy(void* pool);
int fwh_pool_alloc(void* pool);                 // id, or FWH_OUT_OF_PAGES
int fwh_pool_free(void* pool, int id);          // FWH_ERROR if the id is not held
int fwh_pool_size(void* pool);
int fwh_pool_free_count(void* pool);
int fwh_pool_peak(void* pool);                  // most ids out at any time
int fwh_pool_is_held(void* pool, int id);

// ---- the cache: page groups (window 0: every key is kept), block tables, slots --------------------
void* fwh_cache_create(int num_groups, const int* windows, int num_pages, int max_requests, int page_size,
                       int max_pages_per_request);
// the same with a pool size per group (a group that keeps a window needs fewer pages than one that keeps every key)
void* fwh_cache_create_sized(int num_groups, const int* windows, const int* pages, int max_requests, int page_size,
                             int max_pages_per_request);
void fwh_cache_destroy(void* cache);
void* fwh_cache_group_pool(void* cache, int group);     // borrowed: lives as long as the cache
void* fwh_cache_slot_pool(void* cache);
int fwh_cache_admit(void* cache, int64_t request);      // the slot; FWH_OUT_OF_PAGES when no slot is free
int fwh_cache_reserve(void* cache, int64_t request, int new_length);    // all groups or nothing
int fwh_cache_commit(void* cache, int64_t request, int new_length);     // windowed groups give pages back
// pages behind the first token_count tokens go back to the pools (unused reservations, or a
// sequence cut back: the length becomes token_count if it was longer)
int fwh_cache_truncate(void* cache, int64_t request, int token_count);
int fwh_cache_truncate_batch(void* cache, const int64_t* requests, const int* token_counts, int count);
int fwh_cache_release(void* cache, int64_t request);
int fwh_cache_is_live(void* cache, int64_t request);
int fwh_cache_slot_of(void* cache, int64_t request);
int fwh_cache_length_of(void* cache, int64_t request);
int fwh_cache_pages_missing(void* cache, int64_t request, int new_length, int* per_group);
int fwh_cache_table(void* cache, int64_t request, int group, int* pages, int capacity);     // its length
// rows of block tables for a batch: pages given back read as page 0 (they are never looked at)
int fwh_cache_fill_tables(void* cache, int group, const int64_t* requests, int count, int stride, int* rows);
int fwh_cache_longest_table(void* cache, int group, const int64_t* requests, int count);     // blocks of the longest of these tables
// for a whole batch: lengths and slots (FWH_ERROR names the first request that is not live);
// reservations for all or for none; the new lengths
int fwh_cache_describe(void* cache, const int64_t* requests, int count, int* lengths, int* slots);
int fwh_cache_reserve_batch(void* cache, const int64_t* requests, const int* new_lengths, int count);
int fwh_cache_commit_batch(void* cache, const int64_t* requests, const int* new_lengths, int count);
int fwh_cache_live(void* cache, int64_t* requests, int capacity);       // how many are live
int fwh_cache_check(void* cache);                       // no page lost, held twice or free while held

// ---- the scheduler ---------------------------------------------------------------------------------
// Event kinds as the reference numbers them (native/include/flyweight_v2.h:413-417).
#define FWH_EVENT_TOKEN 0
#define FWH_EVENT_FINISHED 1
#define FWH_EVENT_ERROR 2
#define FWH_EVENT_PREFILL 3

// vocab_size: token ids of prompts and stop tokens are checked against it at submit (0: not known, not checked).
void* fwh_scheduler_create(void* cache, int max_positions, int max_batch_tokens, int chunk_size, int max_live,
                           int max_queued, int vocab_size);
void fwh_scheduler_destroy(void* scheduler);
int64_t fwh_scheduler_submit(void* scheduler, const int* prompt, int prompt_len, int max_new_tokens,
                             const int* stop_tokens, int num_stop);    // the request's id (>= 1)
int fwh_scheduler_cancel(void* scheduler, int64_t request);            // 1 if it was still going
// Ends one request with an error (text kept for fwh_request_error): it leaves the queue or gives
// back its pages and slot, and leaves the plan made last, whose other segments and reservations
// stand; its error event comes out of the next completion. 1 if it was still going.
int fwh_scheduler_fail(void* scheduler, int64_t request, const char* message);
int fwh_scheduler_has_work(void* scheduler);
int fwh_scheduler_preemptions(void* scheduler);
int fwh_scheduler_queue(void* scheduler, int which, int64_t* requests, int capacity);   // 0 waiting, 1 running
// Plans the next step (reserving its pages) and keeps the plan until the next call.
// counts: segments, tokens, preempted, failed, admitted, cancelled, and the most tokens that a
// sequence of the plan reaches or that its block tables cover (what a step's tables must hold).
int fwh_scheduler_schedule(void* scheduler, int counts[7]);
int fwh_plan_segments(void* scheduler, int64_t* requests, int* num_tokens, int* wants_logits, int* tokens);
int fwh_plan_list(void* scheduler, int which, int64_t* requests);      // 0 preempted, 1 failed, 2 admitted, 3 cancelled
// After the step: the token drawn for every segment that wanted logits. Events (request, token or
// progress, kind) come back; returns their number (at most 2 per segment plus failed and cancelled).
int fwh_scheduler_complete(void* scheduler, const int64_t* requests, const int* tokens, int count,
                           int64_t* event_requests, int* event_values, int* event_kinds, int capacity);
// A decode step planned and finished without a list per request on the caller's side. If the plan
// made last is one token for each of its requests, each wanting logits, and nothing else happened
// in it (nobody admitted, preempted, failed or cancelled), fwh_plan_fill_decode writes what a
// captured decode step uploads: the tokens, the positions they get (the requests' lengths), the
// requests' slots, and for every page group the rows of the block tables ([group][row][stride],
// group_stride ints apart); returns the number of rows, or FWH_NOT_DECODE_ONLY and writes nothing.
// fwh_scheduler_complete_ordered is fwh_scheduler_complete with the tokens given in the order
// of the plan's segments that wanted logits.
// fwh_plan_steps_ahead: how many further steps of this batch may follow such a plan before the
// host looks again (at most `limit`): the plan holds every running request, there is no place for a waiting request right now (no free
// slot, or as many live requests as allowed), every request has that many positions left in the
// context beyond the one this plan produces, and at least one request has that many tokens to go.
// A caller may then run those steps on the device, feeding each step's tokens to the next, before
// it hands any of them over, with fwh_scheduler_hold_admissions(steps) so that the plans it then
// asks for are those steps. A request that ends on the way (a stop token, its last token) is
// missing from the plans after it (the others keep their order), and the tokens its row went on to
// draw are dropped; whoever waits is admitted by the first plan after the held ones. requests: the
// plan's requests in row order (optional).
#define FWH_NOT_DECODE_ONLY (-3)
int fwh_plan_fill_decode(void* scheduler, int capacity, int* tokens, int* positions, int* slots, int table_stride,
                         int* tables, int group_stride);
int fwh_plan_steps_ahead(void* scheduler, int limit, int64_t* requests, int capacity);
// For each segment of the plan made last, in order: the tokens its request may still generate
// after the one this plan gives it (0: the plan's token is its last). Returns the number written.
int fwh_plan_budgets(void* scheduler, int* budgets, int capacity);
int fwh_scheduler_complete_ordered(void* scheduler, const int* tokens, int count, int64_t* event_requests,
                                   int* event_values, int* event_kinds, int capacity);
// info: computed, live, finished, cancelled, admitted_at, preemptions, prompt length, generated length, max_new_tokens
int fwh_request_info(void* scheduler, int64_t request, int info[9]);
int fwh_request_generated(void* scheduler, int64_t request, int* tokens, int capacity);
const char* fwh_request_error(void* scheduler, int64_t request);       // "" if none
int fwh_scheduler_hold_admissions(void* scheduler, int plans);       // the next `plans` plans admit nobody
int fwh_scheduler_forget(void* scheduler, int64_t request);            // drops a finished request's record

#ifdef __cplusplus
}
#endif
