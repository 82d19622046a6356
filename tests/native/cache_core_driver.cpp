// Random orders of requests against the native cache core, built with the address and undefined-behaviour
// sanitizers (host code only): add, reserve (single and in batches), commit, truncate, release, decode
// packing, with the core's own invariant check after every operation and a model of what every request holds.
#include <stdio.h>
#include <stdlib.h>

#include <map>
#include <random>
#include <vector>

extern "C" {
void* cc_create(int n_groups, const int* rule, const int* params, int page_size, const int* num_pages, int max_requests);
void cc_destroy(void*);
int cc_add(void*);
int cc_release(void*, int);
int cc_num_tokens(void*, int);
int cc_pages_needed(void*, int, int, int*);
int cc_reserve(void*, int, const int*, const int*, int*);
int cc_commit(void*, int, const int*, const int*);
int cc_truncate(void*, int, int);
int cc_table_len(void*, int, int);
int cc_table(void*, int, int, int*);
int cc_slots(void*, int, int, int, int, int*);
void cc_free_pages(void*, int*);
int cc_check(void*);
int cc_fill_decode(void*, int, const int*, const int*, int, int, const int*, int*);
const char* cc_last_error();
}

#define REQUIRE(cond)                                                                   \
  do {                                                                                  \
    if (!(cond)) {                                                                      \
      fprintf(stderr, "line %d: %s failed (%s)\n", __LINE__, #cond, cc_last_error());  \
      exit(1);                                                                          \
    }                                                                                   \
  } while (0)

int main(int argc, char** argv) {
  const unsigned seed = argc > 1 ? (unsigned)atoi(argv[1]) : 1;
  std::mt19937 rng(seed);
  auto pick = [&](int n) { return (int)(rng() % (unsigned)n); };
  const int kinds[2] = {0, 1}, windows[8] = {0, 0, 0, 0, 24, 0, 0, 0}, pages[2] = {40, 14};
  const int page_size = 4 << pick(3), max_req = 5;
  void* c = cc_create(2, kinds, windows, page_size, pages, max_req);
  REQUIRE(c != nullptr);
  std::map<int, int> live;  // slot -> tokens committed
  long ops = 0, refused = 0;
  for (int it = 0; it < 4000; ++it, ++ops) {
    const int op = pick(100);
    if (op < 12 && (int)live.size() < max_req) {
      const int s = cc_add(c);
      REQUIRE(s >= 0 && !live.count(s));
      live[s] = 0;
    } else if (op < 70 && !live.empty()) {
      // a step: a few requests, some with one token, some with a portion
      std::vector<int> reqs, n_new;
      for (auto& kv : live)
        if (pick(2)) {
          reqs.push_back(kv.first);
          n_new.push_back(pick(3) ? 1 : 1 + pick(40));
        }
      if (reqs.empty()) continue;
      int before[2], after[2], info[3];
      cc_free_pages(c, before);
      const int rc = cc_reserve(c, (int)reqs.size(), reqs.data(), n_new.data(), info);
      REQUIRE(rc == 0 || rc == 1);
      cc_free_pages(c, after);
      if (rc == 1) {  // refused: nothing changed, and the report is true
        REQUIRE(before[0] == after[0] && before[1] == after[1]);
        REQUIRE(info[0] > info[1] && info[1] == before[info[2]]);
        ++refused;
        auto victim = live.begin();
        std::advance(victim, pick((int)live.size()));
        REQUIRE(cc_release(c, victim->first) == 0);
        live.erase(victim);
      } else {
        bool all_single = true;
        for (int n : n_new) all_single = all_single && n == 1;
        if (all_single) {
          const int rows = 8, width = 64;
          int scratch[2] = {pages[0], pages[1]};
          std::vector<int> out(4 * rows + 2 * rows * (width + 1), -1), toks(reqs.size(), 7);
          REQUIRE(cc_fill_decode(c, (int)reqs.size(), reqs.data(), toks.data(), rows, width, scratch, out.data()) == 0);
          for (size_t i = 0; i < reqs.size(); ++i) {
            REQUIRE(out[rows + i] == live[reqs[i]] && out[2 * rows + i] == live[reqs[i]] + 1 && out[3 * rows + i] == reqs[i]);
            for (int g = 0; g < 2; ++g) {
              int slot;
              REQUIRE(cc_slots(c, reqs[i], g, live[reqs[i]], 1, &slot) == 0);
              REQUIRE(out[4 * rows + 2 * rows * width + g * rows + i] == slot);
            }
          }
        }
        for (size_t i = 0; i < reqs.size(); ++i) {
          // every position of the new tokens has a row in both groups
          std::vector<int> rows_of(n_new[i]);
          for (int g = 0; g < 2; ++g) REQUIRE(cc_slots(c, reqs[i], g, live[reqs[i]], n_new[i], rows_of.data()) == 0);
          live[reqs[i]] += n_new[i];
        }
        REQUIRE(cc_commit(c, (int)reqs.size(), reqs.data(), n_new.data()) == 0);
        for (size_t i = 0; i < reqs.size(); ++i) REQUIRE(cc_num_tokens(c, reqs[i]) == live[reqs[i]]);
      }
    } else if (op < 78 && !live.empty()) {
      auto r = live.begin();
      std::advance(r, pick((int)live.size()));
      // (a window group cannot take back pages it gave away: such a truncation is refused, nothing changes)
      const int keep = r->second - pick(std::min(r->second, 8) + 1);
      int before[2], after[2];
      cc_free_pages(c, before);
      if (cc_truncate(c, r->first, keep) == 0) {
        r->second = keep;
      } else {
        cc_free_pages(c, after);
        REQUIRE(before[0] == after[0] && before[1] == after[1] && cc_num_tokens(c, r->first) == r->second);
      }
      REQUIRE(cc_truncate(c, r->first, r->second + 1) != 0);   // beyond what is cached: refused
    } else if (op < 90 && !live.empty()) {
      auto r = live.begin();
      std::advance(r, pick((int)live.size()));
      REQUIRE(cc_release(c, r->first) == 0);
      REQUIRE(cc_release(c, r->first) != 0);              // twice: refused
      live.erase(r);
    }
    REQUIRE(cc_check(c) == 0);
  }
  for (auto& kv : live) REQUIRE(cc_release(c, kv.first) == 0);
  int freep[2];
  cc_free_pages(c, freep);
  REQUIRE(freep[0] == pages[0] && freep[1] == pages[1] && cc_check(c) == 0);
  cc_destroy(c);
  printf("ok seed %u page_size %d ops %ld refused %ld\n", seed, page_size, ops, refused);
  return 0;
}
