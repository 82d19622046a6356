// Host bookkeeping of the paged cache, in C++ behind a C interface: page pools (LIFO free lists with
// conservation checks), per-request block tables per cache group, groups whose queries stop seeing old keys
// and give those pages back, state slots, and the packing of a step's device inputs (a decode step's, and
// any mixed step's).  It never touches device memory.
//
// The reference keeps the same bookkeeping natively: a LIFO page allocator whose invariant is
// available + in_use == total (/root/reference/engine/src/kv_cache.rs:762-795,
// /root/reference/kernel-api/src/lib.rs:604-618), block tables with an "empty" marker
// (/root/reference/engine/src/kv_cache.rs:836-893), growth by ceil(n / block) - have pages (:975-984)
// and a need/free report when the pool cannot meet it
// (/root/reference/engine/src/cutile_kv_cache.rs:31-44).  Here a table is per request and group, empty
// entries are -1, and a failed reservation changes nothing.
//
// A live request is named by its state slot (0 .. max_requests - 1), handed out by cc_add.
// Every function returns 0 on success unless said otherwise; cc_last_error() explains a failure.
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <string>
#include <vector>

namespace {

thread_local std::string g_error;

int fail(const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_error = buf;
  return -1;
}

struct Pool {
  int num_pages = 0;
  std::vector<int> free_list;  // LIFO: the most recently freed page is handed out first
  std::vector<uint8_t> held;

  explicit Pool(int n) : num_pages(n), held(n, 0) {
    free_list.reserve(n);
    for (int p = n - 1; p >= 0; --p) free_list.push_back(p);
  }
  int num_free() const { return (int)free_list.size(); }
  int alloc() {
    const int p = free_list.back();
    free_list.pop_back();
    held[p] = 1;
    return p;
  }
  int release(int p) {
    if (p < 0 || p >= num_pages) return fail("page %d out of range", p);
    if (!held[p]) return fail("page %d freed twice (or never allocated)", p);
    held[p] = 0;
    free_list.push_back(p);
    return 0;
  }
  // every page is either free or held, exactly once
  int check() const {
    std::vector<uint8_t> on_list(num_pages, 0);
    for (int p : free_list) {
      if (p < 0 || p >= num_pages) return fail("free list holds page %d out of range", p);
      if (on_list[p]) return fail("page %d is on the free list twice", p);
      if (held[p]) return fail("free page %d is marked held", p);
      on_list[p] = 1;
    }
    int n_held = 0;
    for (int p = 0; p < num_pages; ++p) n_held += held[p];
    if (n_held + (int)free_list.size() != num_pages) return fail("a page was lost");
    return 0;
  }
};

struct Request {
  bool live = false;
  int num_tokens = 0;                      // tokens whose keys and values are in the cache
  std::vector<std::vector<int>> tables;    // per group: logical page -> physical page, -1 = none
  std::vector<int> first_live;             // per group: first logical page still held
};

// ---- what a group's queries can still see ------------------------------------------------------
// A group's rule is data: a code into RULES and up to RULE_PARAMS integers.  A rule gives the first key that
// a query at position `pos` can see; it must never decrease as pos grows, because the pages below it go back
// to the pool for good.  Another rule is one more function and one more line of the table; the host side
// names the codes in one place (tempura_amd/cache/rules.py).
enum { RULE_PARAMS = 4 };
typedef int (*FirstVisible)(int pos, const int* params);
int rule_all(int, const int*) { return 0; }                                        // every key, always
int rule_last_n(int pos, const int* p) { return p[0] > 0 ? std::max(0, pos - p[0] + 1) : 0; }   // a window of p[0] keys
int rule_chunk(int pos, const int* p) { return p[0] > 0 ? pos / p[0] * p[0] : 0; }  // the query's own chunk of p[0] positions
const FirstVisible RULES[] = {rule_all, rule_last_n, rule_chunk};
const int NUM_RULES = (int)(sizeof(RULES) / sizeof(RULES[0]));

struct Core {
  int page_size = 0, max_requests = 0;
  std::vector<int> rule, params;   // per group: code, RULE_PARAMS integers
  std::vector<Pool> pools;
  std::vector<Request> reqs;
  std::vector<int> free_state;

  int n_groups() const { return (int)pools.size(); }
  // first logical page a query at position `start` can still see
  int first_needed(int g, int start) const { return RULES[rule[g]](start, &params[(size_t)g * RULE_PARAMS]) / page_size; }
  // pages group g must allocate so that the request can take n_new more tokens
  int pages_needed(const Request& r, int g, int n_new) const {
    const int end = r.num_tokens + n_new;
    const int last_page = end > 0 ? (end - 1) / page_size : -1;
    const int lo = std::max(first_needed(g, r.num_tokens), r.first_live[g]);
    // every entry from first_live up to the table's end holds a page (pages are given back only below
    // first_live), so what is missing is what lies beyond the table
    return std::max(0, last_page + 1 - std::max(lo, (int)r.tables[g].size()));
  }
  Request* live(int req) {
    if (req < 0 || req >= max_requests || !reqs[req].live) {
      fail("request slot %d is not live", req);
      return nullptr;
    }
    return &reqs[req];
  }
  void grow(Request& r, int n_new) {
    const int end = r.num_tokens + n_new;
    const int last_page = (end - 1) / page_size;
    for (int g = 0; g < n_groups(); ++g) {
      const int lo = std::max(first_needed(g, r.num_tokens), r.first_live[g]);
      std::vector<int>& table = r.tables[g];
      const int have = (int)table.size();
      if ((int)table.size() <= last_page) table.resize(last_page + 1, -1);
      // pages that a window has already passed (below lo) stay unallocated
      for (int lp = std::max(lo, have); lp <= last_page; ++lp) table[lp] = pools[g].alloc();
      if (lo > have) r.first_live[g] = std::max(r.first_live[g], std::min(lo, (int)table.size()));
    }
  }
  void commit(Request& r, int n_new) {
    r.num_tokens += n_new;
    for (int g = 0; g < n_groups(); ++g) {
      const int keep_from = first_needed(g, r.num_tokens);
      std::vector<int>& table = r.tables[g];
      const int stop = std::min(keep_from, (int)table.size());
      for (int lp = r.first_live[g]; lp < stop; ++lp)
        if (table[lp] >= 0) {
          pools[g].release(table[lp]);
          table[lp] = -1;
        }
      r.first_live[g] = std::max(r.first_live[g], stop);
    }
  }
};

}  // namespace

extern "C" {

const char* cc_last_error() { return g_error.c_str(); }

// ---- the cache manager -----------------------------------------------------------------------
// rule[g]: a code into RULES; params: RULE_PARAMS integers per group.
void* cc_create(int n_groups, const int* rule, const int* params, int page_size, const int* num_pages,
                int max_requests) {
  if (page_size <= 0 || n_groups < 0 || max_requests < 0) {
    fail("page_size must be positive");
    return nullptr;
  }
  for (int g = 0; g < n_groups; ++g)
    if (rule[g] < 0 || rule[g] >= NUM_RULES) {
      fail("group %d: unknown visibility rule %d (the core has %d)", g, rule[g], NUM_RULES);
      return nullptr;
    }
  Core* c = new Core;
  c->page_size = page_size;
  c->max_requests = max_requests;
  for (int g = 0; g < n_groups; ++g) {
    if (num_pages[g] < 0) {
      delete c;
      fail("num_pages must be >= 0");
      return nullptr;
    }
    c->rule.push_back(rule[g]);
    for (int i = 0; i < RULE_PARAMS; ++i) c->params.push_back(params[(size_t)g * RULE_PARAMS + i]);
    c->pools.emplace_back(num_pages[g]);
  }
  c->reqs.resize(max_requests);
  for (int s = max_requests - 1; s >= 0; --s) c->free_state.push_back(s);
  return c;
}
void cc_destroy(void* h) { delete (Core*)h; }

// Start tracking a request; returns its state slot, or -1 when every slot is taken.
int cc_add(void* h) {
  Core* c = (Core*)h;
  if (c->free_state.empty()) return fail("no free state slot: %d requests are live", c->max_requests);
  const int s = c->free_state.back();
  c->free_state.pop_back();
  Request& r = c->reqs[s];
  r.live = true;
  r.num_tokens = 0;
  r.tables.assign(c->n_groups(), {});
  r.first_live.assign(c->n_groups(), 0);
  return s;
}

// The request has ended: every page and its state slot go back.
int cc_release(void* h, int req) {
  Core* c = (Core*)h;
  Request* r = c->live(req);
  if (!r) return -1;
  for (int g = 0; g < c->n_groups(); ++g)
    for (int p : r->tables[g])
      if (p >= 0 && c->pools[g].release(p) != 0) return -1;
  r->live = false;
  r->tables.clear();
  c->free_state.push_back(req);
  return 0;
}

int cc_num_tokens(void* h, int req) {
  Request* r = ((Core*)h)->live(req);
  return r ? r->num_tokens : -1;
}

// The largest token count among the given requests.
int cc_max_tokens(void* h, int n, const int* reqs) {
  Core* c = (Core*)h;
  int m = 0;
  for (int i = 0; i < n; ++i) {
    Request* r = c->live(reqs[i]);
    if (!r) return -1;
    m = std::max(m, r->num_tokens);
  }
  return m;
}

int cc_pages_needed(void* h, int req, int n_new, int* out) {
  Core* c = (Core*)h;
  Request* r = c->live(req);
  if (!r) return -1;
  for (int g = 0; g < c->n_groups(); ++g) out[g] = c->pages_needed(*r, g, n_new);
  return 0;
}

// Pages for n_new[i] more tokens of every request reqs[i], or nothing: returns 1 and fills
// info = {need, free, group} when a group's pool cannot meet the sum.
int cc_reserve(void* h, int n, const int* reqs, const int* n_new, int* info) {
  Core* c = (Core*)h;
  const int G = c->n_groups();
  std::vector<long> total(G, 0);
  for (int i = 0; i < n; ++i) {
    Request* r = c->live(reqs[i]);
    if (!r) return -1;
    if (n_new[i] <= 0) return fail("reserve needs at least one token");
    for (int g = 0; g < G; ++g) total[g] += c->pages_needed(*r, g, n_new[i]);
  }
  for (int g = 0; g < G; ++g)
    if (total[g] > c->pools[g].num_free()) {
      info[0] = (int)total[g];
      info[1] = c->pools[g].num_free();
      info[2] = g;
      return 1;
    }
  for (int i = 0; i < n; ++i) c->grow(c->reqs[reqs[i]], n_new[i]);
  return 0;
}

// n_new[i] tokens of reqs[i] were written; pages that a window has passed go back.
int cc_commit(void* h, int n, const int* reqs, const int* n_new) {
  Core* c = (Core*)h;
  for (int i = 0; i < n; ++i) {
    Request* r = c->live(reqs[i]);
    if (!r) return -1;
    c->commit(*r, n_new[i]);
  }
  return 0;
}

// Forget tokens past num_tokens and return whole pages beyond them.
int cc_truncate(void* h, int req, int num_tokens) {
  Core* c = (Core*)h;
  Request* r = c->live(req);
  if (!r) return -1;
  if (num_tokens > r->num_tokens || num_tokens < 0) return fail("truncate beyond what is cached");
  // a window group has given pages back for good: it cannot go back to where a query would need them
  for (int g = 0; g < c->n_groups(); ++g)
    if (num_tokens < r->num_tokens && c->first_needed(g, num_tokens) < r->first_live[g])
      return fail("group %d has given back pages that the truncated request would need", g);
  const int keep = (num_tokens + c->page_size - 1) / c->page_size;
  for (int g = 0; g < c->n_groups(); ++g) {
    std::vector<int>& table = r->tables[g];
    for (int lp = keep; lp < (int)table.size(); ++lp)
      if (table[lp] >= 0) c->pools[g].release(table[lp]);
    if ((int)table.size() > keep) table.resize(keep);
  }
  r->num_tokens = num_tokens;
  return 0;
}

int cc_table_len(void* h, int req, int g) {
  Request* r = ((Core*)h)->live(req);
  return r ? (int)r->tables[g].size() : -1;
}
int cc_table(void* h, int req, int g, int* out) {
  Request* r = ((Core*)h)->live(req);
  if (!r) return -1;
  std::copy(r->tables[g].begin(), r->tables[g].end(), out);
  return 0;
}

// Physical cache rows (page * page_size + offset) of positions start .. start + n - 1.
int cc_slots(void* h, int req, int g, int start, int n, int* out) {
  Core* c = (Core*)h;
  Request* r = c->live(req);
  if (!r) return -1;
  const std::vector<int>& table = r->tables[g];
  for (int i = 0; i < n; ++i) {
    const int pos = start + i, lp = pos / c->page_size;
    if (pos < 0 || lp >= (int)table.size() || table[lp] < 0)
      return fail("positions %d..%d have no page reserved", start, start + n - 1);
    out[i] = table[lp] * c->page_size + pos % c->page_size;
  }
  return 0;
}

void cc_free_pages(void* h, int* out) {
  Core* c = (Core*)h;
  for (int g = 0; g < c->n_groups(); ++g) out[g] = c->pools[g].num_free();
}
int cc_num_live(void* h) {
  Core* c = (Core*)h;
  return c->max_requests - (int)c->free_state.size();
}

// Share of held token places that hold no token (/root/reference/engine/src/kv_cache.rs:1066-1074).
double cc_waste_ratio(void* h) {
  Core* c = (Core*)h;
  long held = 0, used = 0;
  for (const Pool& p : c->pools) held += (long)(p.num_pages - p.num_free()) * c->page_size;
  if (held == 0) return 0.0;
  for (const Request& r : c->reqs)
    if (r.live)
      for (int g = 0; g < c->n_groups(); ++g) used += std::max(0, r.num_tokens - r.first_live[g] * c->page_size);
  return std::max(0.0, 1.0 - (double)used / (double)held);
}

// No page lost, held twice or free while in a table; state slots likewise.
int cc_check(void* h) {
  Core* c = (Core*)h;
  for (int g = 0; g < c->n_groups(); ++g) {
    const Pool& pool = c->pools[g];
    if (pool.check() != 0) return -1;
    std::vector<uint8_t> seen(pool.num_pages, 0);
    int n_seen = 0;
    for (const Request& r : c->reqs) {
      if (!r.live) continue;
      for (int p : r.tables[g]) {
        if (p < 0) continue;
        if (p >= pool.num_pages) return fail("group %d: page %d out of range", g, p);
        if (seen[p]) return fail("group %d: page %d is in two tables", g, p);
        if (!pool.held[p]) return fail("group %d: page %d is in a table but free", g, p);
        seen[p] = 1;
        ++n_seen;
      }
    }
    const int held = pool.num_pages - pool.num_free();
    if (n_seen != held) return fail("group %d: %d pages held by no request", g, held - n_seen);
  }
  std::vector<uint8_t> slot_free(c->max_requests, 0);
  for (int s : c->free_state) {
    if (s < 0 || s >= c->max_requests || slot_free[s]) return fail("a state slot is on the free list twice");
    if (c->reqs[s].live) return fail("a held state slot is on the free list");
    slot_free[s] = 1;
  }
  int n_live = 0;
  for (const Request& r : c->reqs) n_live += r.live;
  if (n_live + (int)c->free_state.size() != c->max_requests) return fail("a state slot was lost");
  return 0;
}

// The device inputs of a decode step (one new token per request) in one packed int32 buffer of `rows`
// rows (rows >= n; the rest is padding that reads and writes the scratch page):
//   tokens[rows] positions[rows] context_lens[rows] state_slots[rows]
//   then per group block_tables[rows, width], then per group slot_mapping[rows].
// Pages must have been reserved for the new token.  scratch_page[g] is the spare page of group g.
int cc_fill_decode(void* h, int n, const int* reqs, const int* tokens, int rows, int width, const int* scratch_page,
                   int* out) {
  Core* c = (Core*)h;
  const int G = c->n_groups();
  if (n > rows) return fail("%d requests do not fit %d rows", n, rows);
  int* tok = out;
  int* pos = out + rows;
  int* ctxl = out + 2 * rows;
  int* slot = out + 3 * rows;
  int* tables = out + 4 * rows;
  int* maps = tables + (size_t)G * rows * width;
  for (int i = 0; i < rows; ++i) {
    tok[i] = 0;
    pos[i] = 0;
    ctxl[i] = 1;  // a padded row: one key, in the scratch page
    slot[i] = c->max_requests;
  }
  for (int g = 0; g < G; ++g) {
    std::fill(tables + (size_t)g * rows * width, tables + (size_t)(g + 1) * rows * width, scratch_page[g]);
    std::fill(maps + (size_t)g * rows, maps + (size_t)(g + 1) * rows, scratch_page[g] * c->page_size);
  }
  for (int i = 0; i < n; ++i) {
    Request* r = c->live(reqs[i]);
    if (!r) return -1;
    const int p = r->num_tokens;
    tok[i] = tokens[i];
    pos[i] = p;
    ctxl[i] = p + 1;
    slot[i] = reqs[i];
    for (int g = 0; g < G; ++g) {
      const std::vector<int>& table = r->tables[g];
      if ((int)table.size() > width) return fail("a block table of %d pages does not fit width %d", (int)table.size(), width);
      int* bt = tables + ((size_t)g * rows + i) * width;
      // pages a window has given back stay pointed at the scratch page; no query reads them
      for (size_t lp = 0; lp < table.size(); ++lp)
        if (table[lp] >= 0) bt[lp] = table[lp];
      const int lp = p / c->page_size;
      if (lp >= (int)table.size() || table[lp] < 0) return fail("position %d has no page reserved", p);
      maps[(size_t)g * rows + i] = table[lp] * c->page_size + p % c->page_size;
    }
  }
  return 0;
}

// A whole step in one call: check it, reserve its pages, and pack its device inputs into one int32 buffer.
// Request reqs[i] brings n_new[i] tokens (tokens: all of them, flattened) and wants the logits at n_want[i] of
// its places (want: indices into its own tokens, flattened).  With N tokens, R requests and M wanted places:
//   tokens[N] positions[N] token_req[N] cu_seqlens[R + 1] context_lens[R] state_slots[R] logit_rows[M]
//   then per group block_tables[R, width_g], then per group slot_mapping[N]
// width_g is the longest table of the step in group g (at least 1); entries without a page point at the
// scratch page.  meta receives {N, M, total, largest n_new, largest context, requests with one token, widths...}.
// Returns 0; 1 when a pool cannot give the step's pages (meta = {need, free, group}); 2 when `capacity` ints
// do not hold the buffer (meta[2] says how many are needed); -1 for a step that is refused (a token outside
// the vocabulary, a wanted place outside its tokens, a request twice, a length above max_positions).  With
// 1, 2 or a refused step nothing has changed: no page is reserved and nothing is written.
int cc_fill_step(void* h, int n, const int* reqs, const int* n_new, const int* tokens, const int* n_want, const int* want,
                 int vocab, int max_positions, const int* scratch_page, int* out, long capacity, int* meta) {
  Core* c = (Core*)h;
  const int G = c->n_groups(), ps = c->page_size;
  if (n <= 0) return fail("a step needs at least one entry");
  long N = 0, M = 0;
  int max_q = 0, max_ctx = 0, singles = 0;
  std::vector<int> width(G, 1);
  std::vector<long> need(G, 0);
  std::vector<uint8_t> in_step(c->max_requests, 0);
  for (int i = 0; i < n; ++i) {
    Request* r = c->live(reqs[i]);
    if (!r) return -1;
    if (in_step[reqs[i]]) return fail("entry %d: its request appears twice in one step", i);
    in_step[reqs[i]] = 1;
    if (n_new[i] <= 0) return fail("entry %d: a step entry needs at least one token", i);
    if (n_want[i] < 0) return fail("entry %d: negative count of wanted places", i);
    const long end = (long)r->num_tokens + n_new[i];
    if (end > max_positions) return fail("entry %d: %ld tokens exceed max positions %d", i, end, max_positions);
    for (int j = 0; j < n_new[i]; ++j) {
      const int t = tokens[N + j];
      if (t < 0 || t >= vocab) return fail("entry %d: token id %d outside the vocabulary of %d", i, t, vocab);
    }
    for (int j = 0; j < n_want[i]; ++j) {
      const int w = want[M + j];
      if (w < 0 || w >= n_new[i]) return fail("entry %d: wanted place %d outside its %d tokens", i, w, n_new[i]);
    }
    N += n_new[i];
    M += n_want[i];
    max_q = std::max(max_q, n_new[i]);
    max_ctx = std::max(max_ctx, (int)end);
    singles += n_new[i] == 1;
    for (int g = 0; g < G; ++g) {
      // every new position must get a page: a rule whose first visible key lies beyond the query's own position
      // (a fault of a newly registered rule) would leave the step's first tokens without one; refused here,
      // before anything is reserved or written
      if (std::max(c->first_needed(g, r->num_tokens), r->first_live[g]) > r->num_tokens / ps)
        return fail("entry %d: position %d has no page in group %d (its rule hides the position from its own query)", i,
                    r->num_tokens, g);
      width[g] = std::max(width[g], std::max((int)r->tables[g].size(), (int)((end + ps - 1) / ps)));
      need[g] += c->pages_needed(*r, g, n_new[i]);
    }
  }
  for (int g = 0; g < G; ++g)
    if (need[g] > c->pools[g].num_free()) {
      meta[0] = (int)need[g];
      meta[1] = c->pools[g].num_free();
      meta[2] = g;
      return 1;
    }
  long total = 3 * N + (n + 1) + 2L * n + M + (long)G * N;
  for (int g = 0; g < G; ++g) total += (long)n * width[g];
  if (total > 0x7fffffffL) return fail("the step's inputs exceed 2^31 integers");
  meta[0] = (int)N;
  meta[1] = (int)M;
  meta[2] = (int)total;
  meta[3] = max_q;
  meta[4] = max_ctx;
  meta[5] = singles;
  for (int g = 0; g < G; ++g) meta[6 + g] = width[g];
  if (total > capacity) return 2;
  for (int i = 0; i < n; ++i) c->grow(c->reqs[reqs[i]], n_new[i]);

  int* tok = out;
  int* pos = tok + N;
  int* treq = pos + N;
  int* cu = treq + N;
  int* ctxl = cu + (n + 1);
  int* slot = ctxl + n;
  int* rows = slot + n;
  int* tables = rows + M;
  int* maps = tables;
  for (int g = 0; g < G; ++g) maps += (long)n * width[g];
  long t0 = 0, w0 = 0;
  cu[0] = 0;
  for (int i = 0; i < n; ++i) {
    const Request& r = c->reqs[reqs[i]];
    const int cnt = n_new[i];
    for (int j = 0; j < cnt; ++j) {
      tok[t0 + j] = tokens[t0 + j];
      pos[t0 + j] = r.num_tokens + j;
      treq[t0 + j] = i;
    }
    for (int j = 0; j < n_want[i]; ++j) rows[w0 + j] = (int)t0 + want[w0 + j];
    cu[i + 1] = (int)(t0 + cnt);
    ctxl[i] = r.num_tokens + cnt;
    slot[i] = reqs[i];
    t0 += cnt;
    w0 += n_want[i];
  }
  int* bt = tables;
  int* mp = maps;
  for (int g = 0; g < G; ++g) {
    const int wd = width[g];
    t0 = 0;
    for (int i = 0; i < n; ++i) {
      const Request& r = c->reqs[reqs[i]];
      const std::vector<int>& table = r.tables[g];
      int* row = bt + (long)i * wd;
      // pages a rule has given back, and what lies past the table, point at the scratch page; no query reads them
      for (int lp = 0; lp < wd; ++lp) row[lp] = (lp < (int)table.size() && table[lp] >= 0) ? table[lp] : scratch_page[g];
      for (int j = 0; j < n_new[i]; ++j) {
        const int p = r.num_tokens + j, lp = p / ps;
        if (lp >= (int)table.size() || table[lp] < 0) return fail("entry %d: position %d has no page in group %d", i, p, g);
        mp[t0 + j] = table[lp] * ps + p % ps;
      }
      t0 += n_new[i];
    }
    bt += (long)n * wd;
    mp += N;
  }
  return 0;
}

}  // extern "C"
