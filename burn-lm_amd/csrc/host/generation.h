// Host-side bookkeeping of the generation loop and of the step function's decisions: how requests
// are cut into batches, which sequences of a batch may run one step ahead of the host, what a
// sequence's next token means for it (stop token, sample_len reached, context full), and into which
// recorded shape a step falls.  Plain C++, no GPU calls.  The reference keeps the same decisions in
// compiled code: the loop bound and token buffer in crates/burn-lm-llama/src/generation/generate.rs:
// 50-64, the stop test in generation/context.rs:116-171.
#pragma once

#ifdef __cplusplus
extern "C" {
#endif

// ---- batches ------------------------------------------------------------------------------------
// Cuts n requests, in order, into batches that fit: at most batch_size sequences and n_slots slots,
// and pages enough for every sequence of a batch to reach min(prompt + sample_len, max_context).
// batch_of[i] receives the batch number of request i, or -1 for a request that would not fit if it
// had all n_pages to itself; returns the number of batches.
int blm_plan_batches(int n, const int* prompt_lens, int sample_len, int batch_size, int max_context, int page_size,
                     int n_pages, int n_slots, int* batch_of);

// Cuts the prompts of one batch (n sequences, prompt_lens[i] > 0 tokens each) into steps of at most
// `budget` tokens: the sequences in order, a step filled before the next one starts, a prompt cut
// wherever a step is full.  Piece p says that step piece_step[p] brings sequence piece_seq[p] its
// tokens piece_from[p] .. + piece_count[p]; pieces come in the order of the steps and, within a step,
// of the sequences.  Returns the number of pieces, or -1 for bad sizes or more than max_pieces
// (n + total / budget + 1 always suffice).
int blm_plan_prompt_steps(int n, const int* prompt_lens, int budget, int max_pieces, int* piece_step, int* piece_seq,
                          int* piece_from, int* piece_count);

// ---- one generation ------------------------------------------------------------------------------
#define BLM_GEN_GOES_ON 0
#define BLM_GEN_STOP 1      // the token is a stop token
#define BLM_GEN_LENGTH 2    // sample_len tokens made, or the context is full
#define BLM_GEN_DROPPED -1  // the sequence had ended before; this token of a step run ahead is ignored

typedef struct BlmGen BlmGen;
BlmGen* blm_gen_new(int n_requests, const int* prompt_lens, int sample_len, int max_context, int n_stop,
                    const int* stop_ids);
void blm_gen_free(BlmGen*);
// A batch starts: its prompts have run in one step and each request's first token is pending.
int blm_gen_start(BlmGen*, int n, const int* requests);
// The live entries (indices into the live batch) that can take one more step before their pending
// token is known: not dropped, the pending token is not their last by sample_len, and the context has
// room for it.  Returns their number.
int blm_gen_ahead_rows(const BlmGen*, int* rows);
// The step for these entries has been started with the pending tokens taken on the device.
int blm_gen_launched(BlmGen*, int n, const int* rows);
// The pending tokens are known, one per live entry.  reasons[k] says what entry k's token means
// (BLM_GEN_*).  Afterwards the live batch is: the entries of the launched step if there was one (those
// that have just ended are dropped: their next token will be ignored), else the entries that go on
// (they are one token longer: the caller feeds them their token in a plain step).  Returns the
// number of live entries that still go on (0: the batch is done).
int blm_gen_take(BlmGen*, const int* tokens, int* reasons);
// The live batch: request of every entry and whether it is dropped; returns the number of entries.
int blm_gen_live(const BlmGen*, int* requests, int* dropped);
int blm_gen_count(const BlmGen*, int request);    // tokens made for a request so far

// ---- the sampler's random numbers -----------------------------------------------------------------
// out[k] = the uniform number in [0, 1) (24 bits) of (seed, requests[k], indices[k]): three rounds of
// the splitmix64 finaliser, a pure function of its arguments, so that a request's draws do not depend
// on its batch mates.
void blm_uniforms(unsigned long long seed, int n, const int* requests, const int* indices, float* out);

// ---- recorded shapes ------------------------------------------------------------------------------
// The bucket key (sequences, tokens or 0 for a decode step, page-table width) of a step of n
// sequences that bring counts[i] tokens, hold lengths[i] and want the places wants (want_counts[i]
// each), or key[0] = -1 if such a step is not replayed from a recorded graph: it is if every
// sequence wants exactly its last token, the sequences fit a batch bucket, and either every sequence
// brings one token (decode) or the tokens fit a token bucket and there are at most prompt_max_seqs.
void blm_step_key(int n, const int* counts, const int* lengths, const int* want_counts, const int* wants,
                  int n_batch_buckets, const int* batch_buckets, int n_token_buckets, const int* token_buckets,
                  int prompt_max_seqs, int page_size, int table_width, int* key);

#ifdef __cplusplus
}
#endif
