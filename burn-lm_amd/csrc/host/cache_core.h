// Host-side core of the cache and of step assembly: which sequence holds which pages, how long
// each sequence is, and the index arrays a step hands to the kernels.  Plain C++, no GPU calls;
// the storage the pages point into is owned by the caller.
//
// Every function returns 0 on success; otherwise a code below, after storing a message that
// blm_host_last_error() gives back.  A failing call changes nothing.
#pragma once

#ifdef __cplusplus
extern "C" {
#endif

#define BLM_HOST_ABI 4

#define BLM_OK 0
#define BLM_E_FULL 1      // no free slot, or not enough free pages
#define BLM_E_OVERFLOW 2  // a sequence would grow past the longest context
#define BLM_E_USAGE 3     // a slot that is not open, a page given back twice, bad arguments

int blm_host_abi_version();
const char* blm_host_last_error();

// ---- a pool of page numbers ---------------------------------------------------------------
typedef struct BlmPool BlmPool;
BlmPool* blm_pool_new(int n_pages);
void blm_pool_free(BlmPool*);
int blm_pool_n_free(const BlmPool*);
int blm_pool_take(BlmPool*, int n, int* out);            // BLM_E_FULL if fewer than n are free
int blm_pool_give(BlmPool*, int n, const int* pages);    // BLM_E_USAGE if one of them is not out
int blm_pool_free_list(const BlmPool*, int* out);        // the free pages, next to be handed out last
int blm_pool_is_out(const BlmPool*, int page);

// ---- the cache's bookkeeping ----------------------------------------------------------------
// Groups of layers with the same need share pages; group g has n_pages[g] pages of page_size
// tokens and keeps the last windows[g] keys of a sequence (0: all of them).
typedef struct BlmCache BlmCache;
BlmCache* blm_cache_new(int n_groups, const int* n_pages, const int* windows, int page_size, int max_seqs,
                        int max_context);
void blm_cache_free(BlmCache*);
int blm_cache_open(BlmCache*, int* slot);
int blm_cache_close(BlmCache*, int slot);
int blm_cache_length(const BlmCache*, int slot);         // -1 if the slot is not open
// Pages for n sequences that grow by n_new[i] tokens each: all of them or none.  On
// BLM_E_OVERFLOW detail[0] is the length asked for and detail[1] the maximum.
int blm_cache_reserve(BlmCache*, int n, const int* slots, const int* n_new, int* detail);
// The reserved step has run: the sequence is n longer; pages that fell out of a window go back.
int blm_cache_advance(BlmCache*, int slot, int n);
// the same for the n sequences of a step, each by counts[i]: checked for all of them first
int blm_cache_advance_all(BlmCache*, int n, const int* slots, const int* counts);
// lengths of n slots; BLM_E_USAGE if one is not open
int blm_cache_lengths(const BlmCache*, int n, const int* slots, int* out);
int blm_cache_table_len(const BlmCache*, int group, int slot);   // -1 if the slot is not open
int blm_cache_table(const BlmCache*, int group, int slot, int* out);
// rows of `width` page numbers for the given slots, -1 where a sequence has no page (a slot < 0
// gives a row of -1); BLM_E_USAGE if a table is wider than `width`
int blm_cache_page_table(const BlmCache*, int group, int n, const int* slots, int width, int* out);
BlmPool* blm_cache_pool(BlmCache*, int group);
int blm_cache_n_free_slots(const BlmCache*);
int blm_cache_free_slots(const BlmCache*, int* out);
int blm_cache_live_slots(const BlmCache*, int* out);     // ascending; returns their number

// ---- step assembly ----------------------------------------------------------------------------
// The index arrays of one step, written into `out` (int32) back to back:
//   token ids [T], positions [T], sequence of each token [T], slots [B], first token of each
//   sequence [B + 1], lengths after the step [B], wanted rows [R], then for every group a page
//   table [B, width]
// for n sequences that bring counts[i] tokens (tokens: all of them in order) and ask for
// want_counts[i] places (wants: places within each sequence's own tokens).  Lengths are the
// cache's, before advance.
// Padding to the shape of a recorded graph: B = max(n, pad_seqs_to), T = max(tokens, pad_tokens_to).
// A padded step must ask for exactly one place per sequence (R = B).  Padding sequences bring no
// token (slot -1, length 0, their wanted row is row 0 and is dropped by the caller); padding tokens
// stand behind the real ones and belong to no sequence (token 0, position 0, sequence -1).
// meta: T, R, most tokens of one sequence, greatest length after the step.  The caller sizes
// `out` with blm_step_size.  vocab > 0: every token id must lie in [0, vocab) (BLM_E_USAGE names the
// first that does not); wanted places outside a sequence's tokens are refused likewise.
long long blm_step_size(int n_groups, int T, int B, int R, int width);
int blm_step_fill(const BlmCache*, int n, const int* slots, const int* counts, const int* tokens,
                  const int* want_counts, const int* wants, int pad_seqs_to, int pad_tokens_to, int width,
                  int* out, long long cap, int* meta, int vocab);
// The same checks without writing anything: slots open, counts positive, tokens in the vocabulary,
// wanted places inside each sequence's tokens.
int blm_step_check(const BlmCache*, int n, const int* slots, const int* counts, const int* tokens,
                   const int* want_counts, const int* wants, int vocab);

#ifdef __cplusplus
}
#endif
