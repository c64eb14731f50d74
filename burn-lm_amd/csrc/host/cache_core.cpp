// See cache_core.h.
#include "cache_core.h"

#include <stdarg.h>
#include <stdio.h>

#include <algorithm>
#include <vector>

static thread_local char g_error[512];

static int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

extern "C" int blm_host_abi_version() { return BLM_HOST_ABI; }
extern "C" const char* blm_host_last_error() { return g_error; }

// ---- pool ---------------------------------------------------------------------------------------
struct BlmPool {
  int n_pages;
  std::vector<int> free_list;   // back() is handed out next
  std::vector<char> out;        // out[p]: page p is held by somebody
};

// The pages are handed out in a fixed scrambled order, not 0, 1, 2, ...: sequences that get their pages in
// one go would otherwise lie at equal distances of a power of two in memory (64 pages of 64 KB: 4 MB), and the
// blocks of a decode attention, which read the same page number of every sequence at the same time, then
// meet in the same memory channels (measured at a context of 4,096: batch 8 16.3 us a layer against 14.5 with
// scattered pages, batch 32 48.2 against 42.3, batch 64 94.4 against 82.8; heads of 128 at batch 64 185
// against 162).  A cache that has served a while is scattered anyway; this makes a fresh one so.
static void pool_init(BlmPool& p, int n_pages) {
  p.n_pages = n_pages;
  p.free_list.resize(n_pages);
  for (int i = 0; i < n_pages; ++i) p.free_list[i] = i;
  unsigned long long state = 0x9E3779B97F4A7C15ull;   // splitmix64 with a fixed seed: the same order in every run
  for (int i = n_pages - 1; i > 0; --i) {
    state += 0x9E3779B97F4A7C15ull;
    unsigned long long z = state;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    const int j = (int)(z % (unsigned long long)(i + 1));
    std::swap(p.free_list[i], p.free_list[j]);
  }
  p.out.assign(n_pages, 0);
}

static int pool_take(BlmPool& p, int n, int* out) {
  if (n < 0) return fail(BLM_E_USAGE, "a negative number of pages was asked for");
  if (n > (int)p.free_list.size())
    return fail(BLM_E_FULL, "%d pages wanted, %d free of %d", n, (int)p.free_list.size(), p.n_pages);
  for (int i = 0; i < n; ++i) {
    const int page = p.free_list.back();
    p.free_list.pop_back();
    p.out[page] = 1;
    out[i] = page;
  }
  return BLM_OK;
}

static int pool_give(BlmPool& p, int n, const int* pages) {
  for (int i = 0; i < n; ++i) {
    const int page = pages[i];
    bool again = false;
    for (int j = 0; j < i; ++j) again = again || pages[j] == page;
    if (page < 0 || page >= p.n_pages || !p.out[page] || again)
      return fail(BLM_E_USAGE, "page %d given back but not handed out (freed twice?)", page);
  }
  for (int i = 0; i < n; ++i) {
    p.out[pages[i]] = 0;
    p.free_list.push_back(pages[i]);
  }
  return BLM_OK;
}

extern "C" BlmPool* blm_pool_new(int n_pages) {
  if (n_pages < 0) return nullptr;
  BlmPool* p = new BlmPool();
  pool_init(*p, n_pages);
  return p;
}
extern "C" void blm_pool_free(BlmPool* p) { delete p; }
extern "C" int blm_pool_n_free(const BlmPool* p) { return (int)p->free_list.size(); }
extern "C" int blm_pool_take(BlmPool* p, int n, int* out) { return pool_take(*p, n, out); }
extern "C" int blm_pool_give(BlmPool* p, int n, const int* pages) { return pool_give(*p, n, pages); }
extern "C" int blm_pool_free_list(const BlmPool* p, int* out) {
  std::copy(p->free_list.begin(), p->free_list.end(), out);
  return (int)p->free_list.size();
}
extern "C" int blm_pool_is_out(const BlmPool* p, int page) {
  return page >= 0 && page < p->n_pages && p->out[page];
}

// ---- cache ----------------------------------------------------------------------------------------
struct Group {
  int window;
  BlmPool pool;
  std::vector<std::vector<int>> tables;   // per slot: page of each page index, -1 once released
};

struct BlmCache {
  int page_size, max_seqs, max_context;
  std::vector<Group> groups;
  std::vector<int> length;       // per slot, -1: not open
  std::vector<int> free_slots;   // back() is opened next
};

static inline int pages_for(const BlmCache& c, int length) { return (length + c.page_size - 1) / c.page_size; }

// pages wholly before the window of the next query are never read again
static inline int first_needed_page(const BlmCache& c, const Group& g, int length_after) {
  if (g.window <= 0) return 0;
  const int first_key = std::max(0, length_after - g.window + 1);
  return first_key / c.page_size;
}

static inline bool is_open(const BlmCache& c, int slot) { return slot >= 0 && slot < c.max_seqs && c.length[slot] >= 0; }

extern "C" BlmCache* blm_cache_new(int n_groups, const int* n_pages, const int* windows, int page_size, int max_seqs,
                                   int max_context) {
  if (n_groups < 0 || page_size <= 0 || max_seqs <= 0 || max_context <= 0) return nullptr;
  BlmCache* c = new BlmCache();
  c->page_size = page_size;
  c->max_seqs = max_seqs;
  c->max_context = max_context;
  c->groups.resize(n_groups);
  for (int g = 0; g < n_groups; ++g) {
    c->groups[g].window = windows[g];
    pool_init(c->groups[g].pool, n_pages[g]);
    c->groups[g].tables.resize(max_seqs);
  }
  c->length.assign(max_seqs, -1);
  c->free_slots.resize(max_seqs);
  for (int i = 0; i < max_seqs; ++i) c->free_slots[i] = max_seqs - 1 - i;   // slot 0 first
  return c;
}
extern "C" void blm_cache_free(BlmCache* c) { delete c; }

extern "C" int blm_cache_open(BlmCache* c, int* slot) {
  if (c->free_slots.empty()) return fail(BLM_E_FULL, "all %d sequence slots are in use", c->max_seqs);
  *slot = c->free_slots.back();
  c->free_slots.pop_back();
  c->length[*slot] = 0;
  for (Group& g : c->groups) g.tables[*slot].clear();
  return BLM_OK;
}

extern "C" int blm_cache_close(BlmCache* c, int slot) {
  if (!is_open(*c, slot)) return fail(BLM_E_USAGE, "slot %d is not open (closed twice?)", slot);
  for (Group& g : c->groups) {
    std::vector<int> held;
    for (int p : g.tables[slot])
      if (p >= 0) held.push_back(p);
    const int rc = pool_give(g.pool, (int)held.size(), held.data());
    if (rc) return rc;
    g.tables[slot].clear();
  }
  c->length[slot] = -1;
  c->free_slots.push_back(slot);
  return BLM_OK;
}

extern "C" int blm_cache_length(const BlmCache* c, int slot) { return is_open(*c, slot) ? c->length[slot] : -1; }

extern "C" int blm_cache_reserve(BlmCache* c, int n, const int* slots, const int* n_new, int* detail) {
  std::vector<int> wanted(c->groups.size(), 0);
  for (int i = 0; i < n; ++i) {
    const int slot = slots[i];
    if (!is_open(*c, slot)) return fail(BLM_E_USAGE, "slot %d is not open", slot);
    for (int j = 0; j < i; ++j)
      if (slots[j] == slot) return fail(BLM_E_USAGE, "slot %d appears twice in one step", slot);
    if (n_new[i] <= 0) return fail(BLM_E_USAGE, "slot %d: a step must bring at least one token", slot);
    const long long after = (long long)c->length[slot] + n_new[i];
    if (after > c->max_context) {
      if (detail) { detail[0] = (int)std::min<long long>(after, 2147483647LL); detail[1] = c->max_context; }
      return fail(BLM_E_OVERFLOW, "context length exceeded: %lld tokens, maximum %d", after, c->max_context);
    }
    for (size_t g = 0; g < c->groups.size(); ++g)
      wanted[g] += pages_for(*c, (int)after) - (int)c->groups[g].tables[slot].size();
  }
  for (size_t g = 0; g < c->groups.size(); ++g) {
    const BlmPool& pool = c->groups[g].pool;
    if (wanted[g] > (int)pool.free_list.size())
      return fail(BLM_E_FULL, "the step needs %d more pages of %d tokens, %d are free of %d", wanted[g], c->page_size,
                  (int)pool.free_list.size(), pool.n_pages);
  }
  for (int i = 0; i < n; ++i) {
    const int slot = slots[i];
    const int after = c->length[slot] + n_new[i];
    for (Group& g : c->groups) {
      std::vector<int>& table = g.tables[slot];
      const int more = pages_for(*c, after) - (int)table.size();
      if (more > 0) {
        const size_t at = table.size();
        table.resize(at + more);
        pool_take(g.pool, more, table.data() + at);   // cannot fail: counted above
      }
    }
  }
  return BLM_OK;
}

extern "C" int blm_cache_advance(BlmCache* c, int slot, int n) {
  if (!is_open(*c, slot)) return fail(BLM_E_USAGE, "slot %d is not open", slot);
  if (n < 0 || c->length[slot] + n > c->max_context) return fail(BLM_E_USAGE, "slot %d cannot advance by %d", slot, n);
  for (const Group& g : c->groups)
    if (pages_for(*c, c->length[slot] + n) > (int)g.tables[slot].size())
      return fail(BLM_E_USAGE, "slot %d advances by %d tokens that no page was reserved for", slot, n);
  c->length[slot] += n;
  for (Group& g : c->groups) {
    std::vector<int>& table = g.tables[slot];
    const int first = std::min<int>(first_needed_page(*c, g, c->length[slot]), (int)table.size());
    for (int i = 0; i < first; ++i) {
      if (table[i] >= 0) {
        const int rc = pool_give(g.pool, 1, &table[i]);
        if (rc) return rc;
        table[i] = -1;
      }
    }
  }
  return BLM_OK;
}

extern "C" int blm_cache_advance_all(BlmCache* c, int n, const int* slots, const int* counts) {
  for (int i = 0; i < n; ++i) {
    if (!is_open(*c, slots[i])) return fail(BLM_E_USAGE, "slot %d is not open", slots[i]);
    if (counts[i] < 0 || c->length[slots[i]] + counts[i] > c->max_context)
      return fail(BLM_E_USAGE, "slot %d cannot advance by %d", slots[i], counts[i]);
    for (const Group& g : c->groups)
      if (pages_for(*c, c->length[slots[i]] + counts[i]) > (int)g.tables[slots[i]].size())
        return fail(BLM_E_USAGE, "slot %d advances by %d tokens that no page was reserved for", slots[i], counts[i]);
  }
  for (int i = 0; i < n; ++i) {
    const int rc = blm_cache_advance(c, slots[i], counts[i]);
    if (rc) return rc;
  }
  return BLM_OK;
}

extern "C" int blm_cache_lengths(const BlmCache* c, int n, const int* slots, int* out) {
  for (int i = 0; i < n; ++i) {
    if (!is_open(*c, slots[i])) return fail(BLM_E_USAGE, "slot %d is not open", slots[i]);
    out[i] = c->length[slots[i]];
  }
  return BLM_OK;
}

extern "C" int blm_cache_table_len(const BlmCache* c, int group, int slot) {
  if (group < 0 || group >= (int)c->groups.size() || !is_open(*c, slot)) return -1;
  return (int)c->groups[group].tables[slot].size();
}

extern "C" int blm_cache_table(const BlmCache* c, int group, int slot, int* out) {
  if (group < 0 || group >= (int)c->groups.size()) return fail(BLM_E_USAGE, "no group %d", group);
  if (!is_open(*c, slot)) return fail(BLM_E_USAGE, "slot %d is not open", slot);
  const std::vector<int>& t = c->groups[group].tables[slot];
  std::copy(t.begin(), t.end(), out);
  return BLM_OK;
}

static int page_rows(const BlmCache& c, int group, int n, const int* slots, int width, int* out) {
  const Group& g = c.groups[group];
  for (int i = 0; i < n; ++i) {
    int* row = out + (size_t)i * width;
    int have = 0;
    if (slots[i] >= 0) {
      if (!is_open(c, slots[i])) return fail(BLM_E_USAGE, "slot %d is not open", slots[i]);
      const std::vector<int>& t = g.tables[slots[i]];
      if ((int)t.size() > width) return fail(BLM_E_USAGE, "page table wider than asked for");
      have = (int)t.size();
      std::copy(t.begin(), t.end(), row);
    }
    std::fill(row + have, row + width, -1);
  }
  return BLM_OK;
}

extern "C" int blm_cache_page_table(const BlmCache* c, int group, int n, const int* slots, int width, int* out) {
  if (group < 0 || group >= (int)c->groups.size() || width < 0) return fail(BLM_E_USAGE, "no group %d", group);
  return page_rows(*c, group, n, slots, width, out);
}

extern "C" BlmPool* blm_cache_pool(BlmCache* c, int group) {
  return (group >= 0 && group < (int)c->groups.size()) ? &c->groups[group].pool : nullptr;
}
extern "C" int blm_cache_n_free_slots(const BlmCache* c) { return (int)c->free_slots.size(); }
extern "C" int blm_cache_free_slots(const BlmCache* c, int* out) {
  std::copy(c->free_slots.begin(), c->free_slots.end(), out);
  return (int)c->free_slots.size();
}
extern "C" int blm_cache_live_slots(const BlmCache* c, int* out) {
  int k = 0;
  for (int s = 0; s < c->max_seqs; ++s)
    if (c->length[s] >= 0) out[k++] = s;
  return k;
}

// ---- step assembly ----------------------------------------------------------------------------------
extern "C" long long blm_step_size(int n_groups, int T, int B, int R, int width) {
  return 3LL * T + B + (B + 1) + B + R + (long long)n_groups * B * width;
}

extern "C" int blm_step_check(const BlmCache* c, int n, const int* slots, const int* counts, const int* tokens,
                              const int* want_counts, const int* wants, int vocab) {
  if (n <= 0) return fail(BLM_E_USAGE, "a step needs at least one sequence");
  long long src = 0, wsrc = 0;
  for (int i = 0; i < n; ++i) {
    if (!is_open(*c, slots[i])) return fail(BLM_E_USAGE, "slot %d is not open", slots[i]);
    if (counts[i] <= 0) return fail(BLM_E_USAGE, "slot %d: a step must bring at least one token per sequence", slots[i]);
    if (want_counts[i] < 0) return fail(BLM_E_USAGE, "slot %d: bad want count", slots[i]);
    if (vocab > 0)
      for (int k = 0; k < counts[i]; ++k)
        if (tokens[src + k] < 0 || tokens[src + k] >= vocab)
          return fail(BLM_E_USAGE, "slot %d: token %d is outside the vocabulary of %d", slots[i], tokens[src + k], vocab);
    src += counts[i];
    for (int k = 0; k < want_counts[i]; ++k)
      if (wants[wsrc + k] < 0 || wants[wsrc + k] >= counts[i])
        return fail(BLM_E_USAGE, "slot %d: wanted place %d is outside this step's %d tokens", slots[i], wants[wsrc + k], counts[i]);
    wsrc += want_counts[i];
  }
  return BLM_OK;
}

extern "C" int blm_step_fill(const BlmCache* c, int n, const int* slots, const int* counts, const int* tokens,
                             const int* want_counts, const int* wants, int pad_seqs_to, int pad_tokens_to, int width,
                             int* out, long long cap, int* meta, int vocab) {
  if (n <= 0) return fail(BLM_E_USAGE, "a step needs at least one sequence");
  if (vocab > 0) {
    const int rc = blm_step_check(c, n, slots, counts, tokens, want_counts, wants, vocab);
    if (rc) return rc;
  }
  const int B = std::max(n, pad_seqs_to);
  long long real = 0, R = 0;
  int max_new = 0, max_after = 0;
  for (int i = 0; i < n; ++i) {
    if (!is_open(*c, slots[i])) return fail(BLM_E_USAGE, "slot %d is not open", slots[i]);
    if (counts[i] <= 0 || want_counts[i] < 0) return fail(BLM_E_USAGE, "slot %d: bad token or want count", slots[i]);
    real += counts[i];
    R += want_counts[i];
    max_new = std::max(max_new, counts[i]);
    max_after = std::max(max_after, c->length[slots[i]] + counts[i]);
  }
  const long long T = std::max(real, (long long)pad_tokens_to);
  if (B > n || T > real) {
    for (int i = 0; i < n; ++i)
      if (want_counts[i] != 1) return fail(BLM_E_USAGE, "only a step of one wanted place per sequence can be padded");
    R = B;
  }
  if (T > 2147483647LL || R > 2147483647LL) return fail(BLM_E_USAGE, "step too large");
  const int G = (int)c->groups.size();
  if (blm_step_size(G, (int)T, B, (int)R, width) > cap) return fail(BLM_E_USAGE, "the step's buffer is too small");
  int* tok = out;
  int* pos = tok + T;
  int* seq = pos + T;
  int* slot_out = seq + T;
  int* cu = slot_out + B;
  int* after = cu + B + 1;
  int* rows = after + B;
  int* tables = rows + R;
  int t = 0, r = 0, src = 0, wsrc = 0;
  cu[0] = 0;
  for (int i = 0; i < n; ++i) {
    const int past = c->length[slots[i]];
    const int base = t;
    for (int k = 0; k < counts[i]; ++k, ++t) {
      tok[t] = tokens[src++];
      pos[t] = past + k;
      seq[t] = i;
    }
    for (int k = 0; k < want_counts[i]; ++k) {
      const int w = wants[wsrc++];
      if (w < 0 || w >= counts[i]) return fail(BLM_E_USAGE, "slot %d: wanted place %d is outside this step's %d tokens", slots[i], w, counts[i]);
      rows[r++] = base + w;
    }
    slot_out[i] = slots[i];
    cu[i + 1] = t;
    after[i] = past + counts[i];
  }
  for (int i = n; i < B; ++i) {   // padding sequences: no tokens, no slot
    rows[r++] = 0;
    slot_out[i] = -1;
    cu[i + 1] = t;
    after[i] = 0;
  }
  for (; t < T; ++t) {   // padding tokens: of no sequence
    tok[t] = 0; pos[t] = 0; seq[t] = -1;
  }
  for (int g = 0; g < G; ++g) {
    const int rc = page_rows(*c, g, B, slot_out, width, tables + (size_t)g * B * width);
    if (rc) return rc;
  }
  meta[0] = (int)T; meta[1] = (int)R; meta[2] = max_new; meta[3] = max_after;
  return BLM_OK;
}
