#include "generation.h"

#include <algorithm>
#include <unordered_set>
#include <vector>

extern "C" int blm_plan_batches(int n, const int* prompt_lens, int sample_len, int batch_size, int max_context,
                                int page_size, int n_pages, int n_slots, int* batch_of) {
  const int most = std::max(1, std::min(batch_size, n_slots));
  int batch = 0, in_batch = 0;
  long long used = 0;
  for (int i = 0; i < n; ++i) {
    const long long reach = std::min<long long>((long long)prompt_lens[i] + sample_len, max_context);
    const long long need = (reach + page_size - 1) / page_size;
    if (need > n_pages) {       // it would not fit if it had the cache to itself: the caller answers it with an error
      batch_of[i] = -1;
      continue;
    }
    if (in_batch > 0 && (in_batch >= most || used + need > n_pages)) {
      ++batch;
      in_batch = 0;
      used = 0;
    }
    batch_of[i] = batch;
    ++in_batch;
    used += need;
  }
  return in_batch > 0 ? batch + 1 : batch;
}

extern "C" int blm_plan_prompt_steps(int n, const int* prompt_lens, int budget, int max_pieces, int* piece_step,
                                     int* piece_seq, int* piece_from, int* piece_count) {
  if (n < 0 || budget <= 0) return -1;
  int pieces = 0, step = 0;
  long long room = budget;
  for (int i = 0; i < n; ++i) {
    if (prompt_lens[i] <= 0) return -1;
    int from = 0;
    while (from < prompt_lens[i]) {
      if (room == 0) {
        ++step;
        room = budget;
      }
      const int take = (int)std::min<long long>(room, prompt_lens[i] - from);
      if (pieces >= max_pieces) return -1;
      piece_step[pieces] = step;
      piece_seq[pieces] = i;
      piece_from[pieces] = from;
      piece_count[pieces] = take;
      ++pieces;
      from += take;
      room -= take;
    }
  }
  return pieces;
}

struct BlmGen {
  int sample_len, max_context;
  std::unordered_set<int> stops;
  std::vector<int> prompt_len, count, reason, length;   // per request; length: tokens its sequence holds
  std::vector<int> live;        // requests of the live batch, in entry order
  std::vector<char> dropped;    // per live entry
  std::vector<int> launched;    // live entries whose next step is already running
  bool has_launched = false;
};

extern "C" BlmGen* blm_gen_new(int n_requests, const int* prompt_lens, int sample_len, int max_context, int n_stop,
                               const int* stop_ids) {
  if (n_requests < 0 || sample_len < 0 || max_context <= 0 || n_stop < 0) return nullptr;
  BlmGen* g = new BlmGen();
  g->sample_len = sample_len;
  g->max_context = max_context;
  g->stops.insert(stop_ids, stop_ids + n_stop);
  g->prompt_len.assign(prompt_lens, prompt_lens + n_requests);
  g->count.assign(n_requests, 0);
  g->reason.assign(n_requests, BLM_GEN_GOES_ON);
  g->length.assign(n_requests, 0);
  return g;
}

extern "C" void blm_gen_free(BlmGen* g) { delete g; }

extern "C" int blm_gen_start(BlmGen* g, int n, const int* requests) {
  for (int k = 0; k < n; ++k)
    if (requests[k] < 0 || requests[k] >= (int)g->count.size()) return 1;
  g->live.assign(requests, requests + n);
  g->dropped.assign(n, 0);
  g->launched.clear();
  g->has_launched = false;
  for (int k = 0; k < n; ++k) g->length[requests[k]] = g->prompt_len[requests[k]];
  return 0;
}

extern "C" int blm_gen_ahead_rows(const BlmGen* g, int* rows) {
  int n = 0;
  for (int k = 0; k < (int)g->live.size(); ++k) {
    const int i = g->live[k];
    if (!g->dropped[k] && g->count[i] + 1 < g->sample_len && g->length[i] + 1 <= g->max_context) rows[n++] = k;
  }
  return n;
}

extern "C" int blm_gen_launched(BlmGen* g, int n, const int* rows) {
  for (int k = 0; k < n; ++k)
    if (rows[k] < 0 || rows[k] >= (int)g->live.size()) return 1;
  g->launched.assign(rows, rows + n);
  g->has_launched = true;
  for (int k = 0; k < n; ++k) g->length[g->live[rows[k]]] += 1;   // the pending token has been fed
  return 0;
}

extern "C" int blm_gen_take(BlmGen* g, const int* tokens, int* reasons) {
  const int n = (int)g->live.size();
  std::vector<char> in_launched(n, 0);
  if (g->has_launched)
    for (int k : g->launched) in_launched[k] = 1;
  std::vector<int> survivors;
  for (int k = 0; k < n; ++k) {
    if (g->dropped[k]) {
      reasons[k] = BLM_GEN_DROPPED;
      continue;
    }
    const int i = g->live[k];
    g->count[i] += 1;
    int r = BLM_GEN_GOES_ON;
    if (g->stops.count(tokens[k])) r = BLM_GEN_STOP;
    else if (g->count[i] >= g->sample_len) r = BLM_GEN_LENGTH;
    else if (g->length[i] + (in_launched[k] ? 0 : 1) > g->max_context) r = BLM_GEN_LENGTH;
    g->reason[i] = r;
    reasons[k] = r;
    if (r == BLM_GEN_GOES_ON) survivors.push_back(i);
  }
  int going = 0;
  if (g->has_launched) {
    std::vector<int> next;
    next.reserve(g->launched.size());
    for (int k : g->launched) next.push_back(g->live[k]);
    g->live.swap(next);
    g->dropped.assign(g->live.size(), 0);
    for (int k = 0; k < (int)g->live.size(); ++k) {
      g->dropped[k] = g->reason[g->live[k]] != BLM_GEN_GOES_ON;
      going += !g->dropped[k];
    }
  } else {
    g->live.swap(survivors);
    g->dropped.assign(g->live.size(), 0);
    for (int i : g->live) g->length[i] += 1;   // the caller feeds each its token in a plain step
    going = (int)g->live.size();
  }
  g->launched.clear();
  g->has_launched = false;
  return going;
}

extern "C" int blm_gen_live(const BlmGen* g, int* requests, int* dropped) {
  for (int k = 0; k < (int)g->live.size(); ++k) {
    requests[k] = g->live[k];
    dropped[k] = g->dropped[k];
  }
  return (int)g->live.size();
}

extern "C" int blm_gen_count(const BlmGen* g, int request) {
  return request >= 0 && request < (int)g->count.size() ? g->count[request] : -1;
}

static inline unsigned long long splitmix64(unsigned long long x) {
  x += 0x9E3779B97F4A7C15ULL;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ULL;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBULL;
  return x ^ (x >> 31);
}

extern "C" void blm_uniforms(unsigned long long seed, int n, const int* requests, const int* indices, float* out) {
  const unsigned long long s = splitmix64(seed);
  for (int k = 0; k < n; ++k) {
    unsigned long long x = splitmix64(s ^ ((unsigned long long)(requests[k] + 1LL) * 0xD1B54A32D192ED03ULL));
    x = splitmix64(x ^ ((unsigned long long)(indices[k] + 1LL) * 0x8CB92BA72F3D8DD7ULL));
    out[k] = (float)(x >> 40) / 16777216.0f;
  }
}

static int bucket_of(int v, int n, const int* buckets) {
  for (int i = 0; i < n; ++i)
    if (v <= buckets[i]) return buckets[i];
  return -1;
}

extern "C" void blm_step_key(int n, const int* counts, const int* lengths, const int* want_counts, const int* wants,
                             int n_batch_buckets, const int* batch_buckets, int n_token_buckets, const int* token_buckets,
                             int prompt_max_seqs, int page_size, int table_width, int* key) {
  key[0] = -1;
  key[1] = key[2] = 0;
  long long tokens = 0;
  int most = 0, w = 0;
  for (int i = 0; i < n; ++i) {
    if (want_counts[i] != 1 || wants[w] != counts[i] - 1) return;
    w += want_counts[i];
    tokens += counts[i];
    most = std::max(most, lengths[i] + counts[i]);
  }
  const int B = bucket_of(n, n_batch_buckets, batch_buckets);
  if (B < 0 || n <= 0) return;
  int T = 0;
  if (tokens != n) {
    T = tokens > 2147483647LL ? -1 : bucket_of((int)tokens, n_token_buckets, token_buckets);
    if (T < 0 || B > prompt_max_seqs) return;
  }
  const int pages = (most + page_size - 1) / page_size;
  int width = 8;
  while (width < pages) width *= 2;
  key[0] = B;
  key[1] = T;
  key[2] = std::min(width, std::max(table_width, 1));
}
