// C entry points of the host runtime library: the page allocator, the cache
// manager (pages, block tables, state slots of every live request) and the
// packing of a step's index arrays. Nothing here touches the GPU. Requests are
// named by 64-bit handles the caller chooses. Functions return 0 or a
// non-negative result on success and a negative IMPARO_E_* code otherwise.
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define IMPARO_E_OUT_OF_PAGES (-1)   // nothing was changed
#define IMPARO_E_NOT_LIVE (-2)
#define IMPARO_E_ALREADY_LIVE (-3)
#define IMPARO_E_SHRINK (-4)
#define IMPARO_E_DOUBLE_FREE (-5)
#define IMPARO_E_RANGE (-6)
#define IMPARO_E_BUSY (-7)           // the pool is not untouched
#define IMPARO_E_CAPACITY (-8)       // the output buffer is too small
#define IMPARO_E_LOST_PAGE (-9)      // check: a page is neither free nor held
#define IMPARO_E_SHARED_PAGE (-10)   // check: a page is held twice, or held and free
#define IMPARO_E_SLOTS (-11)         // check: slots lost or held twice
#define IMPARO_E_TWICE (-12)         // begin_step: a request appears twice
#define IMPARO_E_EMPTY (-13)         // begin_step: a request brings no tokens
#define IMPARO_E_POSITIONS (-14)     // begin_step: a request would pass the model's positions
#define IMPARO_E_TOKEN (-15)         // begin_step: a token id outside the vocabulary
#define IMPARO_E_WANT (-16)          // begin_step: a wanted place outside the request's tokens

typedef struct ImparoPool ImparoPool;
typedef struct ImparoCache ImparoCache;

// ---- a pool of pages: the lowest free page first, always
ImparoPool* imparo_pool_new(int n_pages);
void imparo_pool_delete(ImparoPool* p);
int imparo_pool_alloc(ImparoPool* p);                 // page | IMPARO_E_OUT_OF_PAGES
int imparo_pool_free(ImparoPool* p, int page);        // 0 | IMPARO_E_DOUBLE_FREE | IMPARO_E_RANGE
int imparo_pool_n_free(const ImparoPool* p);
int imparo_pool_n_pages(const ImparoPool* p);
int imparo_pool_high_water(const ImparoPool* p);
int imparo_pool_is_free(const ImparoPool* p, int page);
int imparo_pool_scramble(ImparoPool* p, uint64_t seed);   // only while every page is free

// the hash of the sources this library was built from, as the build computed it
const char* imparo_host_source_hash();

// ---- the cache manager: n_groups paged groups (window 0 = keep every position), each with a pool
// of n_pages[g] pages, and n_slots state slots
ImparoCache* imparo_cache_new(int n_groups, const int32_t* windows, int page_size, const int32_t* n_pages,
                              int n_slots);
void imparo_cache_delete(ImparoCache* c);
ImparoPool* imparo_cache_group_pool(ImparoCache* c, int group);
ImparoPool* imparo_cache_slot_pool(ImparoCache* c);
int imparo_cache_admit(ImparoCache* c, int64_t req);                     // slot | E_ALREADY_LIVE | E_OUT_OF_PAGES (no slot)
int imparo_cache_release(ImparoCache* c, int64_t req);
// pages for positions below new_length in every group, all or nothing; what it took stays
// revocable (imparo_cache_rollback) until the next commit of the request
int imparo_cache_reserve(ImparoCache* c, int64_t req, int new_length);
int imparo_cache_rollback(ImparoCache* c, int64_t req);
int imparo_cache_commit(ImparoCache* c, int64_t req, int new_length);    // pages a window has passed are given back
int imparo_cache_is_live(const ImparoCache* c, int64_t req);
int imparo_cache_length(const ImparoCache* c, int64_t req);
int imparo_cache_slot(const ImparoCache* c, int64_t req);
int imparo_cache_table_len(const ImparoCache* c, int group, int64_t req);
int imparo_cache_table_copy(const ImparoCache* c, int group, int64_t req, int32_t* out, int capacity);
int imparo_cache_pages_needed(const ImparoCache* c, int64_t req, int new_length, int32_t* per_group);
int imparo_cache_first_needed_page(const ImparoCache* c, int group, int next_position);
int imparo_cache_n_live(const ImparoCache* c);
int imparo_cache_page_size(const ImparoCache* c);
int imparo_cache_n_groups(const ImparoCache* c);
int imparo_cache_live_requests(const ImparoCache* c, int64_t* out, int capacity);
int imparo_cache_check(const ImparoCache* c);

// ---- a step's bookkeeping, one call for the whole batch (rows as for imparo_cache_pack).
// begin: checks the batch (no request twice, at least one token each, length + tokens within
// max_position, token ids in [0, vocab), wanted places inside the row's tokens), then admits
// the requests that are not live (new_slots[r] = the slot taken, else -1: the caller clears
// that slot's device state) and reserves pages for every row's new length. All or nothing: on
// failure everything this call did is undone. info = {the failing row or -1, the widest block
// table of the batch in pages, 1 if what ran out was slots}. Returns 0, IMPARO_E_OUT_OF_PAGES (pages, or slots) or the
// check's code. abort undoes a begin whose step did not run; end commits every row.
int imparo_cache_begin_step(ImparoCache* c, int n_rows, const int64_t* reqs, const int32_t* n_tokens,
                            const int32_t* tokens, const int32_t* n_want, const int32_t* want, int vocab,
                            int max_position, int32_t* new_slots, int32_t* info);
int imparo_cache_abort_step(ImparoCache* c, int n_rows, const int64_t* reqs, const int32_t* new_slots);
int imparo_cache_end_step(ImparoCache* c, int n_rows, const int64_t* reqs, const int32_t* n_tokens);

// ---- a step's index arrays, packed for one host-to-device copy.
// Layout (int32): tokens[T] | positions[T] | row_of_token[T] | seg_start[R] | seg_len[R] | slot[R] |
// row lists[R] (rows with one token first, then the others) | want[W] | tables[G][R][P].
// P = table_width, or the widest table of the batch if table_width is 0. `layout` receives
// {T, R, W, G, P, n_single, n_multi, max_seg_len, max_context, total}.
// Returns the number of int32 written, or a negative code; lengths are those before the step.
int64_t imparo_cache_pack(const ImparoCache* c, int n_rows, const int64_t* reqs, const int32_t* n_tokens,
                          const int32_t* tokens, const int32_t* n_want, const int32_t* want, int table_width,
                          int32_t* out, int64_t capacity, int32_t* layout);

// ---- the scheduler's decisions (admission, portions under a token budget, pre-emption).
// It knows requests by the same handles the cache manager uses, and only their sizes: how
// many tokens wait to be fed, how many were fed, how many were generated. Token values,
// sampling and the model step stay with the caller:
//     n = imparo_sched_plan(...)      choose this step's batch (admits, pre-empts)
//     ... run the step ...
//     imparo_sched_advance(s)         the step ran
//     imparo_sched_token(s, id, ..)   once per request whose logits were sampled
typedef struct ImparoSched ImparoSched;

#define IMPARO_EV_ADMIT 1
#define IMPARO_EV_WAIT 2       // the head of the line does not fit yet
#define IMPARO_EV_PREEMPT 3    // gave back its pages and slot; recomputes prompt ++ generated later
#define IMPARO_EV_FAIL 4       // does not fit the cache even alone; it has left

ImparoSched* imparo_sched_new(ImparoCache* cache, int max_batch_tokens, int max_running, int portion);
void imparo_sched_delete(ImparoSched* s);
// 0 queued | 1 finished at once (max_tokens <= 0) | IMPARO_E_ALREADY_LIVE
int imparo_sched_add(ImparoSched* s, int64_t id, int prompt_len, int max_tokens);
// Fills one line per planned request: offset into its pending tokens (-1: its sampled
// token), how many tokens, whether logits are wanted at the last one. Events (what was
// decided on the way) go to ev_ids/ev_kinds. Returns the number of planned requests.
int imparo_sched_plan(ImparoSched* s, int64_t* ids, int32_t* offsets, int32_t* counts, int32_t* wants, int capacity,
                      int64_t* ev_ids, int32_t* ev_kinds, int ev_capacity, int32_t* n_events);
void imparo_sched_advance(ImparoSched* s);
// A token was sampled for `id`: is_stop ends the reply unsent. Returns 0 (goes on), 1 (finished: stop),
// 2 (finished: reached max_tokens; the token counts). The caller frees what a finished request holds.
int imparo_sched_token(ImparoSched* s, int64_t id, int is_stop);
// For a caller that reports tokens before it has read them (is_stop = 0, while the next step
// is queued already): the token turned out to be a stop token. The request leaves, wherever
// it stands, running or back in the waiting line. The caller frees what it holds.
int imparo_sched_retract(ImparoSched* s, int64_t id);
int imparo_sched_drop_waiting_head(ImparoSched* s, int64_t* id);   // 1 and the id, or 0 if nobody waits
int imparo_sched_n_waiting(const ImparoSched* s);
int imparo_sched_n_running(const ImparoSched* s);
int imparo_sched_waiting(const ImparoSched* s, int64_t* out, int capacity);
int imparo_sched_running(const ImparoSched* s, int64_t* out, int capacity);

// ---- plain float32 statements of what the GPU kernels compute (reference_ops.cpp), for tests.
// Arrays are dense and row-major; nothing here is used by the engine.
void imparo_ref_embed(const float* table, const int32_t* ids, float* x, int n_tokens, int width);
void imparo_ref_rms_norm(const float* x, const float* w, float eps, float* y, int rows, int width);
void imparo_ref_gemm(const float* x, const float* w, const float* bias, float* y, int m, int n, int k);
void imparo_ref_swiglu(const float* gate, const float* up, float* out, int64_t count);
void imparo_ref_head_norm_rope(const float* x, const float* w, float eps, const int32_t* positions,
                               const float* inv_freq, int n_freq, float* y, int n_tokens, int heads, int head_dim);
void imparo_ref_attention(const float* q, const float* k, const float* v, const int32_t* q_positions, float* out,
                          int n_queries, int heads, int kv_heads, int head_dim, float scale, int window);
void imparo_ref_short_conv(const float* bcx, const float* w, const float* bias, float* state, float* y, int n_tokens,
                           int width, int taps);
void imparo_ref_argmax(const float* logits, int32_t* out, int rows, int vocab);
void imparo_ref_sample(const float* logits, const float* temperature, const float* uniform, int32_t* out, int rows,
                       int vocab);

#ifdef __cplusplus
}
#endif
