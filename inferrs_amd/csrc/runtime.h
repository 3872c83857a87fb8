// C entry points of the host runtime: the cache manager (pages, block tables, state slots),
// the assembly of a step's arrays, and the scheduler.  No GPU is touched here; the library is
// plain C++.  Functions return 0 (or a non-negative value) on success and a negative code
// after leaving a message for iar_last_error().  Requests are named by 64-bit keys that the
// caller chooses.
#pragma once

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define IAR_ABI_VERSION 1
#define IAR_RELEASED (-1)

// error codes
#define IAR_ERROR (-1)          // a misuse: see the message
#define IAR_NO_PAGES (-2)       // not an error of use: the pool cannot serve the request now

const char* iar_last_error(void);
int iar_abi_version(void);

// ---- cache manager --------------------------------------------------------------------------
// windows[g] < 0: group g keeps every key; else only the last windows[g] positions.
void* iar_cache_create(int page_size, int max_seqs, int n_groups, const int* windows, const int* num_pages);
void iar_cache_destroy(void* cache);
int iar_cache_add_sequence(void* cache, int64_t key);              // -> state slot
int iar_cache_free_sequence(void* cache, int64_t key);
int iar_cache_has_sequence(void* cache, int64_t key);
int iar_cache_num_sequences(void* cache);
int iar_cache_length(void* cache, int64_t key);
int iar_cache_reserved(void* cache, int64_t key);
int iar_cache_state_slot(void* cache, int64_t key);
int iar_cache_reserve(void* cache, int64_t key, int n_new);        // 0, or IAR_NO_PAGES (nothing taken)
int iar_cache_can_reserve(void* cache, int n, const int64_t* keys, const int* n_new);   // 1 / 0
int iar_cache_commit(void* cache, int64_t key, int n_new);
// For a whole batch at once: how many of the keys are live; the greatest cached length; and
// "every request i holds reservations for at least n_tokens[i] tokens", topped up for all or for none.
int iar_cache_count_live(void* cache, int n, const int64_t* keys);
int iar_cache_max_length(void* cache, int n, const int64_t* keys);
int iar_cache_ensure_reserved(void* cache, int n, const int64_t* keys, const int* n_tokens);   // 0 or IAR_NO_PAGES
int iar_cache_commit_many(void* cache, int n, const int64_t* keys, const int* n_new);
int iar_cache_table_size(void* cache, int64_t key, int group);
int iar_cache_table(void* cache, int64_t key, int group, int* out, int capacity);       // -> entries written
int iar_cache_set_table(void* cache, int64_t key, int group, const int* pages, int n);  // for tests of the addressing
int iar_cache_slot_ids(void* cache, int64_t key, int group, int start, int n, int* out);
int iar_cache_num_free(void* cache, int group);
int iar_cache_num_pages(void* cache, int group);
int iar_cache_free_slots(void* cache);
int iar_cache_pool_allocate(void* cache, int group, int n, int* out);   // raw pool access, for tests: n or IAR_NO_PAGES
int iar_cache_pool_free(void* cache, int group, const int* pages, int n);
int iar_cache_slot_allocate(void* cache);                                 // raw slot access, for tests: id or IAR_NO_PAGES
int iar_cache_slot_free(void* cache, int slot);
int iar_cache_check_invariants(void* cache);

// ---- step assembly --------------------------------------------------------------------------
// Writes into `out` (int32, `capacity` words), one after the other: token ids [n], positions [n],
// token->request [n], cu_tokens [s+1], state slots [s], wanted rows [w], and per group slots [n]
// and the block table [s, max_pages].  Requests with one token are put first (in their order),
// the others after them; wanted rows keep the caller's order.  meta (16 ints): 0 total words,
// 1 n tokens, 2 n requests, 3 n wanted, 4 max_pages, 5 max_q_len, 6 max_kv_len, 7 n_single,
// 8 max_kv_single, 9 max_kv_multi, 10 n_groups.  order_out [s]: the caller's index of each request
// in the new order.  pad_pages <= 0: as wide as needed; otherwise the tables are that wide and the bounds 6, 8 and 9
// are at least the tokens that so many pages hold, so that they are the same for every step of that width.
int iar_build_step(void* cache, int n_entries, const int64_t* keys, const int* q_lens, const int* tokens,
                   const int* want_counts, const int* want, int pad_pages, int advance, int32_t* out,
                   long long capacity, int* meta, int* order_out);
long long iar_step_words(void* cache, int n_entries, const int64_t* keys, const int* q_lens, int n_want,
                         int pad_pages, int advance);

// ---- scheduler ------------------------------------------------------------------------------
void* iar_sched_create(void* cache, int max_batch_size, int max_tokens_per_step, int prefill_chunk,
                       int max_seq_len, const int* stop_ids, int n_stop);
void iar_sched_destroy(void* sched);
// > 1: a prompt portion that does not end its prompt is cut so that the step's tokens are a multiple of this (0, 1: off)
int iar_sched_set_row_multiple(void* sched, int row_multiple);
int iar_sched_add(void* sched, int64_t key, const int* prompt, int n_prompt, int max_tokens, int bypass_stop,
                  const int* extra_stop, int n_extra);
// A request that already has a cache entry (its first tokens were put there by other means) joins
// the running requests: tokens = prompt then output so far.  Returns the number of cached tokens.
int iar_sched_adopt(void* sched, int64_t key, const int* tokens, int n_tokens, int n_prompt, int max_tokens,
                    int bypass_stop, const int* extra_stop, int n_extra);
int iar_sched_num_waiting(void* sched);
int iar_sched_num_running(void* sched);
int iar_sched_waiting(void* sched, int64_t* out, int capacity);    // in queue order
int iar_sched_running(void* sched, int64_t* out, int capacity);    // in order of admission
// Decide the next step and reserve its pages.  Returns the number of entries.
int iar_sched_plan(void* sched);
int iar_sched_plan_entries(void* sched, int64_t* keys, int* starts, int* counts, int* samples);
int iar_sched_plan_tokens(void* sched, int entry, int* out, int capacity);
int iar_sched_plan_preempted(void* sched, int64_t* out, int capacity);
int iar_sched_plan_failed(void* sched, int64_t* out, int capacity);
const char* iar_sched_failure(void* sched, int64_t key);
// The planned step ran: sampled[i] is the token drawn for the i-th entry that samples.  Returns the
// number of requests that finished; their keys and reasons (0 stop, 1 length) go to the outputs.
int iar_sched_commit(void* sched, const int* sampled, int n_sampled, int64_t* finished, int* reasons, int capacity);
// A run of decode steps queued at once (see Engine.decode_chain): commits one token for each of
// `keys` that still runs.
int iar_sched_commit_decode(void* sched, int n, const int64_t* keys, const int* tokens, int64_t* finished,
                            int* reasons, int capacity);
// state of one request: 0 computed, 1 n output, 2 status (0 waiting, 1 running, 2 finished), 3 preemptions, 4 n prompt
int iar_sched_request_state(void* sched, int64_t key, int* out5);
int iar_sched_request_output(void* sched, int64_t key, int* out, int capacity);
// End a waiting or running request now (a stop string matched, the client went away): its cache entry
// is given back.  Entries of the current plan that belong to it are dropped.
int iar_sched_finish(void* sched, int64_t key);
int iar_sched_forget(void* sched, int64_t key);                     // drop a finished request's record

#ifdef __cplusplus
}
#endif
