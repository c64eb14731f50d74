// A driver for AddressSanitizer / UndefinedBehaviorSanitizer builds of the native host code: the
// cache core, the generation bookkeeping and the plain C++ references of the kernels, compiled
// together with this file and run on the CPU (tests/test_native_sanitizers.py does both).  No
// Python and no ctypes in between: the sanitizers see every access the libraries make.
//
// It replays what the Python tests do through ctypes: random open / reserve / advance / close
// traffic on a cache of two groups (one windowed) with the books checked after every move, step
// assembly with and without padding, refused arguments, a generation with stop tokens that runs
// one step ahead of its tokens, batch and prompt planning, and each kernel reference on small
// inputs.  Any book-keeping fault aborts with a message; a memory fault is the sanitizer's to report.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <set>
#include <vector>

#include "cache_core.h"
#include "generation.h"

extern "C" {
void ref_embed_gather(const float* table, const int* ids, float* out, int T, int D);
void ref_add_rmsnorm(float* h, const float* delta, int n_planes, long long plane_stride, const float* gamma, float* out,
                     const int* rows, int T, int D, float eps, int write_h);
void ref_swiglu(const float* gate_up, float* out, int T, int I);
void ref_linear(const float* A, const float* W, float* C, int M, int N, int K);
void ref_gated_linear(const float* A, const float* W, float* C, int M, int I, int K);
void ref_argmax(const float* logits, int* out, int R, int V, int ld);
void ref_sample(const float* logits, const float* uniforms, int* out, int R, int V, int ld, float temperature, float top_p);
}

#define CHECK(cond)                                                                  \
  do {                                                                               \
    if (!(cond)) {                                                                   \
      std::fprintf(stderr, "%s:%d: check failed: %s\n", __FILE__, __LINE__, #cond);  \
      std::abort();                                                                  \
    }                                                                                \
  } while (0)

struct Rng {
  uint64_t s;
  explicit Rng(uint64_t seed) : s(seed) {}
  uint64_t next() {
    s += 0x9E3779B97F4A7C15ULL;
    uint64_t x = s;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ULL;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBULL;
    return x ^ (x >> 31);
  }
  int below(int n) { return (int)(next() % (uint64_t)n); }
  double unit() { return (double)(next() >> 11) / 9007199254740992.0; }
};

// No page lost, none held twice, tables as long as the lengths say, windows give back what fell out.
static void check_books(BlmCache* c, const std::map<int, int>& live, int page, const int* n_pages, const int* windows,
                        int n_groups) {
  for (int g = 0; g < n_groups; ++g) {
    BlmPool* pool = blm_cache_pool(c, g);
    std::vector<int> free_list(n_pages[g]);
    const int n_free = blm_pool_free_list(pool, free_list.data());
    CHECK(n_free == blm_pool_n_free(pool));
    std::set<int> seen(free_list.begin(), free_list.begin() + n_free);
    CHECK((int)seen.size() == n_free);
    for (const auto& [slot, len] : live) {
      CHECK(blm_cache_length(c, slot) == len);
      const int tl = blm_cache_table_len(c, g, slot);
      CHECK(tl == (len + page - 1) / page);
      std::vector<int> table(std::max(tl, 1));
      CHECK(blm_cache_table(c, g, slot, table.data()) == BLM_OK);
      const int first_key = windows[g] ? std::max(0, len - windows[g] + 1) : 0;
      for (int i = 0; i < tl; ++i) {
        const bool held = i >= first_key / page;
        CHECK((table[i] >= 0) == held);
        if (table[i] >= 0) {
          CHECK(table[i] < n_pages[g]);
          CHECK(seen.insert(table[i]).second);        // neither free nor in another table
          CHECK(blm_pool_is_out(pool, table[i]) == 1);
        }
      }
    }
    CHECK((int)seen.size() <= n_pages[g]);
  }
}

static void cache_traffic(uint64_t seed) {
  Rng rnd(seed);
  const int page = 16, n_groups = 2, max_seqs = 5, max_context = 96;
  const int n_pages[2] = {20, 20}, windows[2] = {0, 24};
  BlmCache* c = blm_cache_new(n_groups, n_pages, windows, page, max_seqs, max_context);
  CHECK(c != nullptr);
  std::map<int, int> live;
  const int growths[5] = {1, 1, 1, 7, 30};
  for (int move = 0; move < 800; ++move) {
    const double r = rnd.unit();
    if (r < 0.25 && blm_cache_n_free_slots(c) > 0) {
      int slot = -1;
      CHECK(blm_cache_open(c, &slot) == BLM_OK && slot >= 0 && slot < max_seqs && !live.count(slot));
      live[slot] = 0;
    } else if (r < 0.4 && !live.empty()) {
      auto it = live.begin();
      std::advance(it, rnd.below((int)live.size()));
      CHECK(blm_cache_close(c, it->first) == BLM_OK);
      CHECK(blm_cache_close(c, it->first) == BLM_E_USAGE);      // closing twice is refused, not done
      live.erase(it);
    } else if (!live.empty()) {
      std::vector<int> slots, grow;
      for (const auto& [slot, len] : live)
        if (rnd.below(2) || slots.empty()) {
          slots.push_back(slot);
          grow.push_back(growths[rnd.below(5)]);
        }
      int detail[2] = {0, 0};
      const int rc = blm_cache_reserve(c, (int)slots.size(), slots.data(), grow.data(), detail);
      CHECK(rc == BLM_OK || rc == BLM_E_FULL || rc == BLM_E_OVERFLOW);
      if (rc == BLM_OK) {
        if (rnd.below(2)) {
          CHECK(blm_cache_advance_all(c, (int)slots.size(), slots.data(), grow.data()) == BLM_OK);
        } else {
          for (size_t i = 0; i < slots.size(); ++i) CHECK(blm_cache_advance(c, slots[i], grow[i]) == BLM_OK);
        }
        for (size_t i = 0; i < slots.size(); ++i) live[slots[i]] += grow[i];
      }
    }
    check_books(c, live, page, n_pages, windows, n_groups);
    // every fourth move: the live sequences' next step, assembled with and without padding
    if (move % 4 == 0 && !live.empty()) {
      std::vector<int> slots, counts, tokens, want_counts, wants;
      int most = 0;
      for (const auto& [slot, len] : live) {
        const int n = 1 + rnd.below(3);
        if (len + n > max_context) continue;
        slots.push_back(slot);
        counts.push_back(n);
        for (int t = 0; t < n; ++t) tokens.push_back(rnd.below(50));
        want_counts.push_back(1);
        wants.push_back(n - 1);
        most = std::max(most, len + n);
      }
      const int n = (int)slots.size();
      if (n > 0) {
        int detail[2];
        if (blm_cache_reserve(c, n, slots.data(), counts.data(), detail) == BLM_OK) {
          CHECK(blm_step_check(c, n, slots.data(), counts.data(), tokens.data(), want_counts.data(), wants.data(), 50) == BLM_OK);
          const int T = (int)tokens.size(), width = (most + page - 1) / page;
          for (int pad = 0; pad < 2; ++pad) {
            const int B = pad ? n + 2 : n, Tp = pad ? T + 5 : T;
            const long long size = blm_step_size(n_groups, Tp, B, B, width);
            std::vector<int> out((size_t)size, 12345);
            int meta[4];
            CHECK(blm_step_fill(c, n, slots.data(), counts.data(), tokens.data(), want_counts.data(), wants.data(),
                                pad ? B : 0, pad ? Tp : 0, width, out.data(), size, meta, 50) == BLM_OK);
            CHECK(meta[0] == Tp && meta[1] == B);
            // a buffer one word short is refused and nothing is written past it
            std::vector<int> tight((size_t)size - 1, 777);
            CHECK(blm_step_fill(c, n, slots.data(), counts.data(), tokens.data(), want_counts.data(), wants.data(),
                                pad ? B : 0, pad ? Tp : 0, width, tight.data(), size - 1, meta, 50) == BLM_E_USAGE);
          }
          // a token outside the vocabulary and a wanted place outside the tokens are refused
          std::vector<int> bad = tokens;
          bad.back() = 50;
          CHECK(blm_step_check(c, n, slots.data(), counts.data(), bad.data(), want_counts.data(), wants.data(), 50) == BLM_E_USAGE);
          std::vector<int> bad_wants = wants;
          bad_wants[0] = counts[0];
          CHECK(blm_step_check(c, n, slots.data(), counts.data(), tokens.data(), want_counts.data(), bad_wants.data(), 50) == BLM_E_USAGE);
          // the page table of the step, one row per slot and one for a padding slot
          std::vector<int> with_pad = slots;
          with_pad.push_back(-1);
          std::vector<int> table((size_t)(n + 1) * width);
          CHECK(blm_cache_page_table(c, 0, n + 1, with_pad.data(), width, table.data()) == BLM_OK);
          for (int w = 0; w < width; ++w) CHECK(table[(size_t)n * width + w] == -1);
          if (width > 1) CHECK(blm_cache_page_table(c, 0, n, slots.data(), width - 1, table.data()) == BLM_E_USAGE);
          CHECK(blm_cache_advance_all(c, n, slots.data(), counts.data()) == BLM_OK);
          for (int i = 0; i < n; ++i) live[slots[i]] += counts[i];
          check_books(c, live, page, n_pages, windows, n_groups);
        }
      }
    }
  }
  // wrong uses change nothing
  int slot = 99;
  CHECK(blm_cache_close(c, 99) == BLM_E_USAGE && blm_cache_length(c, -3) == -1);
  int one = 1, detail[2];
  CHECK(blm_cache_reserve(c, 1, &slot, &one, detail) == BLM_E_USAGE);
  for (const auto& [s, len] : live) CHECK(blm_cache_close(c, s) == BLM_OK);
  live.clear();
  check_books(c, live, page, n_pages, windows, n_groups);
  CHECK(blm_cache_n_free_slots(c) == max_seqs);
  for (int g = 0; g < n_groups; ++g) CHECK(blm_pool_n_free(blm_cache_pool(c, g)) == n_pages[g]);
  blm_cache_free(c);

  BlmPool* p = blm_pool_new(4);
  int got[4], twice[2] = {1, 1};
  CHECK(blm_pool_take(p, 5, got) == BLM_E_FULL && blm_pool_take(p, 4, got) == BLM_OK && blm_pool_n_free(p) == 0);
  CHECK(blm_pool_give(p, 2, twice) == BLM_E_USAGE && blm_pool_n_free(p) == 0);      // a page given back twice in one call
  CHECK(blm_pool_give(p, 4, got) == BLM_OK && blm_pool_give(p, 1, got) == BLM_E_USAGE);
  blm_pool_free(p);
}

// The toy model of the Python tests: next token = (sum of the sequence so far) mod vocab.
static void generation(uint64_t seed) {
  Rng rnd(seed);
  const int vocab = 50, sample_len = 9, max_context = 40;
  for (int round = 0; round < 40; ++round) {
    const int n = 1 + rnd.below(6);
    std::vector<std::vector<int>> seqs(n);
    std::vector<int> lens(n);
    for (int i = 0; i < n; ++i) {
      lens[i] = 1 + rnd.below(35);
      for (int t = 0; t < lens[i]; ++t) seqs[i].push_back(rnd.below(vocab));
    }
    const int stops[2] = {rnd.below(vocab), rnd.below(vocab)};
    // what a plain loop makes of each request
    std::vector<std::vector<int>> want(n);
    std::vector<int> why(n);
    for (int i = 0; i < n; ++i) {
      std::vector<int> s = seqs[i];
      why[i] = BLM_GEN_LENGTH;
      while ((int)want[i].size() < sample_len) {
        long long sum = 0;
        for (int t : s) sum += t;
        const int tok = (int)(sum % vocab);
        want[i].push_back(tok);
        if (tok == stops[0] || tok == stops[1]) { why[i] = BLM_GEN_STOP; break; }
        if ((int)s.size() + 1 > max_context) break;       // no room to feed it back
        s.push_back(tok);
      }
    }
    std::vector<int> batch_of(n);
    const int n_batches = blm_plan_batches(n, lens.data(), sample_len, 3, max_context, 16, 12, 4, batch_of.data());
    CHECK(n_batches >= 1);
    BlmGen* g = blm_gen_new(n, lens.data(), sample_len, max_context, 2, stops);
    CHECK(g != nullptr);
    std::vector<std::vector<int>> made(n);
    std::vector<int> reason(n, BLM_GEN_GOES_ON);
    const bool ahead = round % 2 == 1;
    for (int b = 0; b < n_batches; ++b) {
      std::vector<int> ids;
      for (int i = 0; i < n; ++i)
        if (batch_of[i] == b) ids.push_back(i);
      CHECK(!ids.empty() && (int)ids.size() <= 3);
      // prompt planning: the pieces cover every prompt once, in order, within the budget
      std::vector<int> plens;
      for (int i : ids) plens.push_back(lens[i]);
      const int budget = 1 + rnd.below(40), most = (int)ids.size() + 200;
      std::vector<int> ps(most), pq(most), pf(most), pc(most);
      const int pieces = blm_plan_prompt_steps((int)ids.size(), plens.data(), budget, most, ps.data(), pq.data(), pf.data(), pc.data());
      CHECK(pieces >= (int)ids.size());
      std::vector<int> fed(ids.size(), 0), in_step(pieces + 1, 0);
      for (int p = 0; p < pieces; ++p) {
        CHECK(pf[p] == fed[pq[p]] && pc[p] > 0 && (p == 0 || ps[p] >= ps[p - 1]));
        fed[pq[p]] += pc[p];
        in_step[ps[p]] += pc[p];
        CHECK(in_step[ps[p]] <= budget);
      }
      for (size_t k = 0; k < ids.size(); ++k) CHECK(fed[k] == plens[k]);
      CHECK(blm_plan_prompt_steps((int)ids.size(), plens.data(), budget, 0, ps.data(), pq.data(), pf.data(), pc.data()) == -1);

      std::vector<std::vector<int>> state;      // the sequence of every live entry as the "device" knows it
      for (int i : ids) state.push_back(seqs[i]);
      CHECK(blm_gen_start(g, (int)ids.size(), ids.data()) == 0);
      std::vector<int> live = ids;
      std::vector<int> pending;                  // one token per live entry
      for (auto& s : state) {
        long long sum = 0;
        for (int t : s) sum += t;
        pending.push_back((int)(sum % vocab));
      }
      while (true) {
        std::vector<int> rows(live.size() + 1), next_pending;
        std::vector<std::vector<int>> next_state;
        int n_rows = 0;
        bool launched = false;
        if (ahead) {
          n_rows = blm_gen_ahead_rows(g, rows.data());
          CHECK(n_rows >= 0 && n_rows <= (int)live.size());
          if (n_rows > 0) {
            CHECK(blm_gen_launched(g, n_rows, rows.data()) == 0);
            launched = true;
            for (int k = 0; k < n_rows; ++k) {
              std::vector<int> s = state[rows[k]];
              s.push_back(pending[rows[k]]);
              long long sum = 0;
              for (int t : s) sum += t;
              next_pending.push_back((int)(sum % vocab));
              next_state.push_back(s);
            }
          }
        }
        std::vector<int> reasons(live.size());
        const int going = blm_gen_take(g, pending.data(), reasons.data());
        for (size_t k = 0; k < live.size(); ++k) {
          if (reasons[k] == BLM_GEN_DROPPED) continue;
          made[live[k]].push_back(pending[k]);
          if (reasons[k] != BLM_GEN_GOES_ON) reason[live[k]] = reasons[k];
        }
        std::vector<int> now(ids.size() + 1), dropped(ids.size() + 1);
        const int n_live = blm_gen_live(g, now.data(), dropped.data());
        if (launched) {
          CHECK(n_live == n_rows);
          live.assign(now.begin(), now.begin() + n_live);
          state = next_state;
          pending = next_pending;
          if (going == 0) break;
          continue;
        }
        if (n_live == 0) break;
        // a plain step: every survivor is fed its token
        std::vector<std::vector<int>> st2;
        std::vector<int> pend2;
        for (int k2 = 0; k2 < n_live; ++k2) {
          size_t k = 0;
          while (live[k] != now[k2]) ++k;
          std::vector<int> s = state[k];
          s.push_back(pending[k]);
          long long sum = 0;
          for (int t : s) sum += t;
          pend2.push_back((int)(sum % vocab));
          st2.push_back(s);
        }
        live.assign(now.begin(), now.begin() + n_live);
        state = st2;
        pending = pend2;
      }
    }
    for (int i = 0; i < n; ++i) {
      CHECK(made[i] == want[i]);
      CHECK(reason[i] == why[i]);
      CHECK(blm_gen_count(g, i) == (int)want[i].size());
    }
    CHECK(blm_gen_count(g, n) == -1);
    int bad = n;
    CHECK(blm_gen_start(g, 1, &bad) == 1);
    blm_gen_free(g);
  }
  CHECK(blm_gen_new(1, nullptr, -1, 8, 0, nullptr) == nullptr);
  // uniforms: in [0, 1), a function of (seed, request, index) alone
  int reqs[3] = {0, 7, 7}, idx[3] = {0, 3, 3};
  float u[3];
  blm_uniforms(12345, 3, reqs, idx, u);
  CHECK(u[1] == u[2] && u[0] != u[1] && u[0] >= 0.f && u[0] < 1.f);
  // recorded shapes
  int counts[3] = {1, 1, 1}, lengths[3] = {10, 700, 3}, want_counts[3] = {1, 1, 1}, wants[3] = {0, 0, 0}, key[3];
  const int bb[4] = {1, 2, 4, 8}, tb[3] = {64, 128, 256};
  blm_step_key(3, counts, lengths, want_counts, wants, 4, bb, 3, tb, 16, 64, 64, key);
  CHECK(key[0] == 4 && key[1] == 0 && key[2] == 16);
  wants[1] = 5;
  blm_step_key(3, counts, lengths, want_counts, wants, 4, bb, 3, tb, 16, 64, 64, key);
  CHECK(key[0] == -1);
}

static void references() {
  Rng rnd(3);
  const int T = 5, D = 24, I = 16, V = 37;
  std::vector<float> table(V * D), h(T * D), delta(2 * T * D), gamma(D), out(T * D), w(2 * I * D), act(T * I), gu(T * 2 * I),
      logits(T * (V + 3)), uni(T);
  for (auto* v : {&table, &h, &delta, &gamma, &w, &gu, &logits}) for (float& x : *v) x = (float)(rnd.unit() * 2 - 1);
  for (float& x : uni) x = (float)rnd.unit();
  std::vector<int> ids(T), rows = {4, 0}, picked(T);
  for (int& i : ids) i = rnd.below(V);
  ref_embed_gather(table.data(), ids.data(), out.data(), T, D);
  CHECK(out[0] == table[(size_t)ids[0] * D]);
  ref_add_rmsnorm(h.data(), delta.data(), 2, (long long)T * D, gamma.data(), out.data(), nullptr, T, D, 1e-5f, 1);
  ref_add_rmsnorm(h.data(), nullptr, 0, 0, gamma.data(), out.data(), rows.data(), 2, D, 1e-5f, 0);
  ref_linear(h.data(), w.data(), act.data(), T, I, D);
  ref_gated_linear(h.data(), w.data(), act.data(), T, I, D);
  ref_swiglu(gu.data(), act.data(), T, I);
  ref_argmax(logits.data(), picked.data(), T, V, V + 3);
  for (int p : picked) CHECK(p >= 0 && p < V);
  ref_sample(logits.data(), uni.data(), picked.data(), T, V, V + 3, 0.8f, 0.9f);
  for (int p : picked) CHECK(p >= 0 && p < V);
  for (float x : act) CHECK(std::isfinite(x));
}

int main() {
  CHECK(blm_host_abi_version() == BLM_HOST_ABI);
  for (uint64_t seed = 0; seed < 3; ++seed) cache_traffic(seed);
  generation(11);
  references();
  std::puts("native host code: clean");
  return 0;
}
