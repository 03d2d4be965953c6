// Host side of the paged cache, natively: which pages are free, which a request holds in each group of
// layers, state slots, and the packing of one step's batch into the int32 arrays the kernels read.
// No GPU call is made here; the library is loaded through ctypes like the kernel libraries.
//
// Pages: a LIFO stack of free page numbers with in-use flags, so that a double free or a page outside the
// pool fails loudly in O(1) (infernum/src/block_allocator.rs:27-110 searches the free list instead).
// Block tables: per group and request the pages in the order of positions, page_size tokens each
// (block_allocator.rs:119-198); in a window group the pages that every later query's window has passed go
// back to the pool and leave NO_PAGE behind (the reference keeps them, TABNINE.md:53).
// A step: requests that bring one token first, portions of prompts after them; all arrays in one buffer in
// segments aligned to 16 bytes, so that one copy takes them to the device (the reference uploads four
// tensors per decode step, infernum/src/backend.rs:209-241).
//
// Every call that can fail returns IA_HOST_ERROR and leaves a message that ia_cache_error / ia_pool_error
// returns; nothing is changed by a failed call unless its comment says so.
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

namespace {

constexpr int NO_PAGE = -1;
constexpr int IA_HOST_ERROR = -2;
constexpr int KIND_FULL = 0, KIND_WINDOW = 1;

struct Pool {
  int num_pages = 0;
  std::vector<int> free_;          // back() is handed out next
  std::vector<uint8_t> used;
  std::string error;

  explicit Pool(int n) : num_pages(n), used((size_t)n, 0) {
    free_.reserve((size_t)n);
    for (int p = n - 1; p >= 0; --p) free_.push_back(p);   // page 0 first
  }
  int num_free() const { return (int)free_.size(); }
  int allocate() {
    if (free_.empty()) return -1;
    const int p = free_.back();
    free_.pop_back();
    used[(size_t)p] = 1;
    return p;
  }
  int release(int p) {
    if (p < 0 || p >= num_pages) {
      error = "page " + std::to_string(p) + " is outside the pool of " + std::to_string(num_pages);
      return IA_HOST_ERROR;
    }
    if (!used[(size_t)p]) {
      error = "page " + std::to_string(p) + " is freed twice";
      return IA_HOST_ERROR;
    }
    used[(size_t)p] = 0;
    free_.push_back(p);
    return 0;
  }
};

struct Table {
  std::vector<int> pages;
  int64_t num_tokens = 0;
  int first_live = 0;              // pages before this index have been given back
};

struct Group {
  int kind = KIND_FULL;
  int window = 0;
  int page_size = 1;
  Pool pool;
  std::unordered_map<int64_t, Table> tables;
  Group(int kind_, int window_, int page_size_, int num_pages) : kind(kind_), window(window_), page_size(page_size_), pool(num_pages) {}

  int pages_for(int64_t tokens) const { return (int)((tokens + page_size - 1) / page_size); }
  int pages_missing(const Table& t, int64_t n_new) const {
    return std::max(0, pages_for(t.num_tokens + n_new) - (int)t.pages.size());
  }
};

struct Cache {
  int page_size = 1;
  std::vector<Group> groups;
  int num_slots = 0;
  std::vector<int> free_slots;
  std::vector<uint8_t> slot_used;
  std::unordered_map<int64_t, int> slot_of;
  std::unordered_map<int64_t, int64_t> tokens;
  std::vector<int> last_freed;     // (group, page) pairs of the last commit or release
  std::vector<int32_t> packed;     // the last packed step
  std::string error;

  bool admitted(int64_t req) const { return slot_of.find(req) != slot_of.end(); }
  int fail(const std::string& msg) {
    error = msg;
    return IA_HOST_ERROR;
  }
};

std::string req_name(int64_t req) { return "request #" + std::to_string(req); }

inline int64_t align4(int64_t n) { return (n + 3) & ~(int64_t)3; }

}  // namespace

extern "C" {

// ------------------------------------------------------------------------------------------- page pool
void* ia_pool_create(int num_pages) { return num_pages > 0 ? new Pool(num_pages) : nullptr; }
void ia_pool_destroy(void* h) { delete static_cast<Pool*>(h); }
const char* ia_pool_error(void* h) { return static_cast<Pool*>(h)->error.c_str(); }
int ia_pool_num_pages(void* h) { return static_cast<Pool*>(h)->num_pages; }
int ia_pool_num_free(void* h) { return static_cast<Pool*>(h)->num_free(); }
int ia_pool_allocate(void* h) { return static_cast<Pool*>(h)->allocate(); }
// n pages into out, or none at all (returns 0)
int ia_pool_allocate_many(void* h, int n, int* out) {
  Pool* p = static_cast<Pool*>(h);
  if (n > p->num_free()) return 0;
  for (int i = 0; i < n; ++i) out[i] = p->allocate();
  return 1;
}
int ia_pool_free(void* h, int page) { return static_cast<Pool*>(h)->release(page); }
int ia_pool_is_used(void* h, int page) {
  Pool* p = static_cast<Pool*>(h);
  return page >= 0 && page < p->num_pages && p->used[(size_t)page];
}

// ------------------------------------------------------------------------------------------- the cache
// kinds[g]: 0 = all keys, 1 = a window of windows[g] keys.  Every group has num_pages pages of page_size.
void* ia_cache_create(int n_groups, const int* kinds, const int* windows, int page_size, int num_pages, int num_slots) {
  if (n_groups < 0 || page_size <= 0 || num_pages <= 0 || num_slots < 0) return nullptr;
  Cache* c = new Cache();
  c->page_size = page_size;
  for (int g = 0; g < n_groups; ++g) c->groups.emplace_back(kinds[g], windows[g], page_size, num_pages);
  c->num_slots = num_slots;
  c->slot_used.assign((size_t)num_slots, 0);
  for (int s = num_slots - 1; s >= 0; --s) c->free_slots.push_back(s);
  return c;
}
void ia_cache_destroy(void* h) { delete static_cast<Cache*>(h); }
const char* ia_cache_error(void* h) { return static_cast<Cache*>(h)->error.c_str(); }
// the pool of group g, for the ia_pool_* calls (owned by the cache)
void* ia_cache_group_pool(void* h, int g) { return &static_cast<Cache*>(h)->groups[(size_t)g].pool; }
int ia_cache_num_free_slots(void* h) { return (int)static_cast<Cache*>(h)->free_slots.size(); }
int ia_cache_num_requests(void* h) { return (int)static_cast<Cache*>(h)->slot_of.size(); }
int ia_cache_has(void* h, int64_t req) { return static_cast<Cache*>(h)->admitted(req) ? 1 : 0; }

// state slots alone (a pool of indices; the cache's requests use the same calls inside)
int ia_cache_acquire_slot(void* h) {
  Cache* c = static_cast<Cache*>(h);
  if (c->free_slots.empty()) return -1;
  const int s = c->free_slots.back();
  c->free_slots.pop_back();
  c->slot_used[(size_t)s] = 1;
  return s;
}
int ia_cache_release_slot(void* h, int slot) {
  Cache* c = static_cast<Cache*>(h);
  if (slot < 0 || slot >= c->num_slots || !c->slot_used[(size_t)slot])
    return c->fail("state slot " + std::to_string(slot) + " is released twice or was never taken");
  c->slot_used[(size_t)slot] = 0;
  c->free_slots.push_back(slot);
  return 0;
}

// empty block tables and a state slot for the request: the slot, -1 when none is free
int ia_cache_admit(void* h, int64_t req) {
  Cache* c = static_cast<Cache*>(h);
  if (c->admitted(req)) return c->fail(req_name(req) + " is admitted twice");
  const int slot = ia_cache_acquire_slot(h);
  if (slot < 0) return -1;
  c->slot_of[req] = slot;
  c->tokens[req] = 0;
  for (Group& g : c->groups) g.tables[req] = Table();
  return slot;
}

int ia_cache_state_slot(void* h, int64_t req) {
  Cache* c = static_cast<Cache*>(h);
  auto it = c->slot_of.find(req);
  if (it == c->slot_of.end()) return c->fail(req_name(req) + " is not admitted");
  return it->second;
}

int64_t ia_cache_num_tokens(void* h, int64_t req) {
  Cache* c = static_cast<Cache*>(h);
  auto it = c->tokens.find(req);
  if (it == c->tokens.end()) return c->fail(req_name(req) + " is not admitted");
  return it->second;
}

// per group, the pages that n_new more tokens would take from the pool; admitted = 0: a request that
// holds nothing yet
int ia_cache_pages_needed(void* h, int admitted, int64_t req, int64_t n_new, int* out) {
  Cache* c = static_cast<Cache*>(h);
  for (size_t g = 0; g < c->groups.size(); ++g) {
    Group& grp = c->groups[g];
    if (admitted && c->admitted(req)) out[g] = grp.pages_missing(grp.tables[req], n_new);
    else out[g] = grp.pages_for(n_new);
  }
  return 0;
}

// how many more tokens of the request the pools can hold, promised[g] pages of each already spoken for
int64_t ia_cache_tokens_that_fit(void* h, int admitted, int64_t req, const int* promised) {
  Cache* c = static_cast<Cache*>(h);
  int64_t best = (int64_t)1 << 60;
  for (size_t g = 0; g < c->groups.size(); ++g) {
    Group& grp = c->groups[g];
    const int64_t avail = std::max<int64_t>(0, (int64_t)grp.pool.num_free() - (promised ? promised[g] : 0));
    int64_t room;
    if (admitted && c->admitted(req)) {
      const Table& t = grp.tables[req];
      room = ((int64_t)t.pages.size() + avail) * grp.page_size - t.num_tokens;
    } else {
      room = avail * grp.page_size;
    }
    best = std::min(best, room);
  }
  return std::max<int64_t>(best, 0);
}

int ia_cache_can_reserve(void* h, int64_t req, int64_t n_new) {
  Cache* c = static_cast<Cache*>(h);
  if (!c->admitted(req)) return c->fail(req_name(req) + " is not admitted");
  for (Group& g : c->groups)
    if (g.pages_missing(g.tables[req], n_new) > g.pool.num_free()) return 0;
  return 1;
}

// pages for the next n_new tokens in every group, or nothing at all (returns 0)
int ia_cache_reserve(void* h, int64_t req, int64_t n_new) {
  Cache* c = static_cast<Cache*>(h);
  const int ok = ia_cache_can_reserve(h, req, n_new);
  if (ok != 1) return ok;
  for (Group& g : c->groups) {
    Table& t = g.tables[req];
    for (int i = g.pages_missing(t, n_new); i > 0; --i) t.pages.push_back(g.pool.allocate());
  }
  return 1;
}

// the n_new tokens are stored; pages that a window has passed go back to the pool (ia_cache_last_freed)
int ia_cache_commit(void* h, int64_t req, int64_t n_new) {
  Cache* c = static_cast<Cache*>(h);
  if (!c->admitted(req)) return c->fail(req_name(req) + " is not admitted");
  for (Group& g : c->groups) {
    const Table& t = g.tables[req];
    if (t.num_tokens + n_new > (int64_t)t.pages.size() * g.page_size)
      return c->fail(req_name(req) + " stored " + std::to_string(t.num_tokens + n_new) + " tokens in " +
                     std::to_string(t.pages.size()) + " pages");
  }
  c->last_freed.clear();
  c->tokens[req] += n_new;
  for (size_t gi = 0; gi < c->groups.size(); ++gi) {
    Group& g = c->groups[gi];
    Table& t = g.tables[req];
    t.num_tokens += n_new;
    if (g.kind == KIND_WINDOW && g.window > 0) {
      // the next query stands at position num_tokens and sees keys >= num_tokens - window + 1
      const int64_t first_needed = std::max<int64_t>(0, t.num_tokens - g.window + 1) / g.page_size;
      const int stop = (int)std::min<int64_t>(first_needed, (int64_t)t.pages.size());
      while (t.first_live < stop) {
        const int p = t.pages[(size_t)t.first_live];
        if (p != NO_PAGE) {
          g.pool.release(p);
          c->last_freed.push_back((int)gi);
          c->last_freed.push_back(p);
          t.pages[(size_t)t.first_live] = NO_PAGE;
        }
        ++t.first_live;
      }
    }
  }
  return 0;
}

// the request is over: everything it holds goes back (ia_cache_last_freed)
int ia_cache_release(void* h, int64_t req) {
  Cache* c = static_cast<Cache*>(h);
  auto it = c->slot_of.find(req);
  if (it == c->slot_of.end()) return c->fail(req_name(req) + " is released but not admitted");
  const int slot = it->second;
  c->last_freed.clear();
  for (size_t gi = 0; gi < c->groups.size(); ++gi) {
    Group& g = c->groups[gi];
    Table& t = g.tables[req];
    for (size_t i = (size_t)t.first_live; i < t.pages.size(); ++i)
      if (t.pages[i] != NO_PAGE) {
        g.pool.release(t.pages[i]);
        c->last_freed.push_back((int)gi);
        c->last_freed.push_back(t.pages[i]);
      }
    g.tables.erase(req);
  }
  c->slot_of.erase(it);
  c->tokens.erase(req);
  return ia_cache_release_slot(h, slot);
}

// (group, page) pairs that the last commit or release gave back: the number of pairs; up to cap are copied
int ia_cache_last_freed(void* h, int* out, int cap) {
  Cache* c = static_cast<Cache*>(h);
  const int n = (int)c->last_freed.size() / 2;
  if (out) std::memcpy(out, c->last_freed.data(), sizeof(int) * 2 * (size_t)std::min(n, cap));
  return n;
}

// the block table of a request in a group: its length; up to cap pages are copied
int ia_cache_table(void* h, int g, int64_t req, int* pages, int cap, int64_t* num_tokens, int* first_live) {
  Cache* c = static_cast<Cache*>(h);
  if (g < 0 || g >= (int)c->groups.size()) return c->fail("no group " + std::to_string(g));
  auto it = c->groups[(size_t)g].tables.find(req);
  if (it == c->groups[(size_t)g].tables.end()) return c->fail(req_name(req) + " is not admitted");
  const Table& t = it->second;
  if (pages) std::memcpy(pages, t.pages.data(), sizeof(int) * std::min(t.pages.size(), (size_t)std::max(cap, 0)));
  if (num_tokens) *num_tokens = t.num_tokens;
  if (first_live) *first_live = t.first_live;
  return (int)t.pages.size();
}

// pages for a whole step, all or nothing: requests that are not admitted yet (admitted[i] == 0) count with
// empty tables and one state slot each.  1 = the step fits.
int ia_cache_step_fits(void* h, int n, const int64_t* reqs, const int* admitted, const int* q_lens) {
  Cache* c = static_cast<Cache*>(h);
  int fresh = 0;
  for (int i = 0; i < n; ++i) fresh += (admitted[i] && c->admitted(reqs[i])) ? 0 : 1;
  if (fresh > (int)c->free_slots.size()) return 0;
  for (Group& g : c->groups) {
    int64_t need = 0;
    for (int i = 0; i < n; ++i) {
      if (admitted[i] && c->admitted(reqs[i])) need += g.pages_missing(g.tables[reqs[i]], q_lens[i]);
      else need += g.pages_for(q_lens[i]);
    }
    if (need > g.pool.num_free()) return 0;
  }
  return 1;
}

// pages for q_lens[i] more tokens of every reqs[i] (all admitted), or nothing at all (returns 0)
int ia_cache_reserve_step(void* h, int n, const int64_t* reqs, const int* q_lens) {
  Cache* c = static_cast<Cache*>(h);
  for (int i = 0; i < n; ++i)
    if (!c->admitted(reqs[i])) return c->fail(req_name(reqs[i]) + " is not admitted");
  for (Group& g : c->groups) {
    int64_t need = 0;
    for (int i = 0; i < n; ++i) need += g.pages_missing(g.tables[reqs[i]], q_lens[i]);
    if (need > g.pool.num_free()) return 0;
  }
  for (int i = 0; i < n; ++i)
    for (Group& g : c->groups) {
      Table& t = g.tables[reqs[i]];
      for (int k = g.pages_missing(t, q_lens[i]); k > 0; --k) t.pages.push_back(g.pool.allocate());
    }
  return 1;
}

// undo of ia_cache_reserve_step for a step that did not run: pages beyond what each request's stored tokens
// need go back to the pools (ia_cache_last_freed names them)
int ia_cache_unreserve_step(void* h, int n, const int64_t* reqs) {
  Cache* c = static_cast<Cache*>(h);
  for (int i = 0; i < n; ++i)
    if (!c->admitted(reqs[i])) return c->fail(req_name(reqs[i]) + " is not admitted");
  c->last_freed.clear();
  for (int i = 0; i < n; ++i)
    for (size_t gi = 0; gi < c->groups.size(); ++gi) {
      Group& g = c->groups[gi];
      Table& t = g.tables[reqs[i]];
      const size_t keep = (size_t)g.pages_for(t.num_tokens);
      while (t.pages.size() > keep) {
        const int p = t.pages.back();
        t.pages.pop_back();
        if (p != NO_PAGE) {
          g.pool.release(p);
          c->last_freed.push_back((int)gi);
          c->last_freed.push_back(p);
        }
      }
    }
  return 0;
}

// ia_cache_commit for every entry of a step; ia_cache_last_freed then covers all of them.  Entries before
// a failing one stay committed.
int ia_cache_commit_step(void* h, int n, const int64_t* reqs, const int* q_lens) {
  Cache* c = static_cast<Cache*>(h);
  std::vector<int> freed;
  for (int i = 0; i < n; ++i) {
    const int rc = ia_cache_commit(h, reqs[i], q_lens[i]);
    if (rc != 0) return rc;
    freed.insert(freed.end(), c->last_freed.begin(), c->last_freed.end());
  }
  c->last_freed.swap(freed);
  return 0;
}

// every page is free or held by exactly one request; counts agree
int ia_cache_check(void* h) {
  Cache* c = static_cast<Cache*>(h);
  for (size_t gi = 0; gi < c->groups.size(); ++gi) {
    Group& g = c->groups[gi];
    std::unordered_map<int, int64_t> held;
    for (auto& kv : g.tables) {
      const Table& t = kv.second;
      for (size_t i = (size_t)t.first_live; i < t.pages.size(); ++i) {
        const int p = t.pages[i];
        if (p == NO_PAGE) continue;
        auto seen = held.find(p);
        if (seen != held.end())
          return c->fail("group " + std::to_string(gi) + ": page " + std::to_string(p) + " is held by " +
                         req_name(seen->second) + " and " + req_name(kv.first));
        if (p < 0 || p >= g.pool.num_pages || !g.pool.used[(size_t)p])
          return c->fail("group " + std::to_string(gi) + ": page " + std::to_string(p) + " of " + req_name(kv.first) +
                         " is marked free");
        held[p] = kv.first;
      }
      if (t.num_tokens > (int64_t)t.pages.size() * g.page_size)
        return c->fail("group " + std::to_string(gi) + ": " + req_name(kv.first) + " holds too few pages");
    }
    const int in_use = g.pool.num_pages - g.pool.num_free();
    if ((int)held.size() != in_use)
      return c->fail("group " + std::to_string(gi) + ": " + std::to_string(in_use) + " pages in use, " +
                     std::to_string(held.size()) + " held: a page is lost");
  }
  if ((int)c->slot_of.size() != c->num_slots - (int)c->free_slots.size())
    return c->fail("state slots in use do not match the admitted requests");
  std::vector<uint8_t> seen((size_t)c->num_slots, 0);
  for (auto& kv : c->slot_of) {
    if (seen[(size_t)kv.second]) return c->fail("two requests share a state slot");
    seen[(size_t)kv.second] = 1;
  }
  return 0;
}

// page * page_size + offset of positions start .. start + n - 1 of a request in a group (pages must be
// reserved)
int ia_cache_token_slots(void* h, int g, int64_t req, int64_t start, int n, int32_t* out) {
  Cache* c = static_cast<Cache*>(h);
  if (g < 0 || g >= (int)c->groups.size()) return c->fail("no group " + std::to_string(g));
  Group& grp = c->groups[(size_t)g];
  auto it = grp.tables.find(req);
  if (it == grp.tables.end()) return c->fail(req_name(req) + " is not admitted");
  const std::vector<int>& pages = it->second.pages;
  for (int i = 0; i < n; ++i) {
    const int64_t pos = start + i;
    const int64_t pi = pos / grp.page_size;
    if (pi >= (int64_t)pages.size() || pages[(size_t)pi] < 0)
      return c->fail(req_name(req) + " has no page for position " + std::to_string(pos));
    out[i] = (int32_t)((int64_t)pages[(size_t)pi] * grp.page_size + pos % grp.page_size);
  }
  return 0;
}

// ------------------------------------------------------------------------------------------- a step
// Entry i brings q_lens[i] tokens (tokens, entry after entry) of request reqs[i] and wants the logits at
// want_counts[i] places among them (wants, entry after entry).  Pages must be reserved.  Rows are ordered
// with the single tokens first.  bt_width > 0 widens the block tables to that many columns; bt_width < 0
// to the power of two (at least 8) that holds the longest table of any group.
//
// Segments of the buffer, each aligned to 4 values: 0 token ids, 1 positions, 2 row of each token,
// 3 first token of each row (n + 1), 4 tokens stored before the step per row, 5 state slots, 6 rows of the
// wanted logits, 7 prefill tiles (row, first query) pairs of tile_rows queries, the ones with the most
// keys before them first, then per group:
// 8 + 2 g slots of the tokens in the pages, 9 + 2 g block tables [n, columns].
//
// meta (int32): [0] buffer length, [1] single-token rows, [2] tiles, [3] wanted rows, [4] longest portion,
// [5] longest context + portion, [6] segments S, then S offsets, S sizes, per group the block table's
// columns, then the n entries in row order, then the n counts of tokens stored before.
// Returns 0, or IA_HOST_ERROR with nothing packed.
int ia_cache_pack_step(void* h, int n, const int64_t* reqs, const int* q_lens, const int32_t* tokens,
                       const int* want_counts, const int32_t* wants, int bt_width, int tile_rows, int32_t* meta,
                       int meta_cap) {
  Cache* c = static_cast<Cache*>(h);
  const int G = (int)c->groups.size();
  const int S = 8 + 2 * G;
  if (n <= 0 || tile_rows <= 0) return c->fail("a step needs entries");
  if (meta_cap < 7 + 2 * S + G + 2 * n) return c->fail("the meta buffer is too small");
  // row order: single tokens first, else as given
  std::vector<int> order((size_t)n);
  int num_decode = 0;
  {
    int k = 0;
    for (int i = 0; i < n; ++i)
      if (q_lens[i] == 1) order[(size_t)k++] = i;
    num_decode = k;
    for (int i = 0; i < n; ++i)
      if (q_lens[i] != 1) order[(size_t)k++] = i;
  }
  std::vector<int64_t> tok_start((size_t)n + 1, 0), want_start((size_t)n + 1, 0);
  for (int i = 0; i < n; ++i) {
    if (q_lens[i] <= 0) return c->fail("an entry brings no tokens");
    if (!c->admitted(reqs[i])) return c->fail(req_name(reqs[i]) + " is not admitted");
    tok_start[(size_t)i + 1] = tok_start[(size_t)i] + q_lens[i];
    want_start[(size_t)i + 1] = want_start[(size_t)i] + want_counts[i];
  }
  const int64_t N = tok_start[(size_t)n], R = want_start[(size_t)n];
  std::vector<int64_t> ctx((size_t)n), row_start((size_t)n + 1, 0), row_of_entry((size_t)n);
  int64_t max_q = 0, max_total = 0, tiles = 0;
  for (int r = 0; r < n; ++r) {
    const int e = order[(size_t)r];
    ctx[(size_t)r] = c->tokens[reqs[e]];
    row_start[(size_t)r + 1] = row_start[(size_t)r] + q_lens[e];
    row_of_entry[(size_t)e] = r;
    max_q = std::max<int64_t>(max_q, q_lens[e]);
    max_total = std::max<int64_t>(max_total, ctx[(size_t)r] + q_lens[e]);
    if (r >= num_decode) tiles += (q_lens[e] + tile_rows - 1) / tile_rows;
  }
  std::vector<int> cols((size_t)G, 1);
  int widest = 1;
  for (int g = 0; g < G; ++g)
    for (int i = 0; i < n; ++i) widest = std::max(widest, (int)c->groups[(size_t)g].tables[reqs[i]].pages.size());
  int pow2 = 8;
  while (pow2 < widest) pow2 *= 2;
  for (int g = 0; g < G; ++g) {
    int w = 1;
    if (bt_width > 0) w = bt_width;
    else if (bt_width < 0) w = pow2;
    else
      for (int i = 0; i < n; ++i) w = std::max(w, (int)c->groups[(size_t)g].tables[reqs[i]].pages.size());
    for (int i = 0; i < n; ++i)
      if ((int)c->groups[(size_t)g].tables[reqs[i]].pages.size() > w)
        return c->fail("a block table is wider than the " + std::to_string(w) + " columns asked for");
    cols[(size_t)g] = w;
  }
  std::vector<int64_t> sizes((size_t)S), offsets((size_t)S);
  sizes[0] = sizes[1] = sizes[2] = N;
  sizes[3] = n + 1;
  sizes[4] = sizes[5] = n;
  sizes[6] = R;
  sizes[7] = 2 * tiles;
  for (int g = 0; g < G; ++g) {
    sizes[(size_t)(8 + 2 * g)] = N;
    sizes[(size_t)(9 + 2 * g)] = (int64_t)n * cols[(size_t)g];
  }
  int64_t total = 0;
  for (int s = 0; s < S; ++s) {
    offsets[(size_t)s] = total;
    total += align4(std::max<int64_t>(sizes[(size_t)s], 1));
  }
  if (total > 0x7fffffff) return c->fail("the step is too large");
  std::vector<int32_t> buf((size_t)total, 0);
  int32_t* ids = buf.data() + offsets[0];
  int32_t* pos = buf.data() + offsets[1];
  int32_t* seq = buf.data() + offsets[2];
  int32_t* starts = buf.data() + offsets[3];
  int32_t* ctxs = buf.data() + offsets[4];
  int32_t* slots = buf.data() + offsets[5];
  int32_t* rows = buf.data() + offsets[6];
  int32_t* tile = buf.data() + offsets[7];
  int64_t t_at = 0;
  for (int r = 0; r < n; ++r) {
    const int e = order[(size_t)r];
    const int64_t q = q_lens[e], at = row_start[(size_t)r];
    for (int64_t j = 0; j < q; ++j) {
      ids[at + j] = tokens[tok_start[(size_t)e] + j];
      pos[at + j] = (int32_t)(ctx[(size_t)r] + j);
      seq[at + j] = r;
    }
    starts[r] = (int32_t)at;
    ctxs[r] = (int32_t)ctx[(size_t)r];
    slots[r] = c->slot_of[reqs[e]];
    for (int g = 0; g < G; ++g) {
      Group& grp = c->groups[(size_t)g];
      const std::vector<int>& pages = grp.tables[reqs[e]].pages;
      int32_t* sl = buf.data() + offsets[(size_t)(8 + 2 * g)] + at;
      for (int64_t j = 0; j < q; ++j) {
        const int64_t p = ctx[(size_t)r] + j, pi = p / grp.page_size;
        if (pi >= (int64_t)pages.size() || pages[(size_t)pi] < 0)
          return c->fail(req_name(reqs[e]) + " has no page for position " + std::to_string(p));
        sl[j] = (int32_t)((int64_t)pages[(size_t)pi] * grp.page_size + p % grp.page_size);
      }
      int32_t* bt = buf.data() + offsets[(size_t)(9 + 2 * g)] + (int64_t)r * cols[(size_t)g];
      for (int k = 0; k < cols[(size_t)g]; ++k) bt[k] = k < (int)pages.size() ? pages[(size_t)k] : NO_PAGE;
    }
  }
  starts[n] = (int32_t)N;
  // tiles with the most keys before them first: workgroups start in this order, and the long ones
  // must not start last
  {
    std::vector<std::pair<int64_t, std::pair<int, int>>> list;   // (keys before the tile, (row, first query))
    for (int r = num_decode; r < n; ++r)
      for (int64_t q0 = 0; q0 < q_lens[order[(size_t)r]]; q0 += tile_rows)
        list.push_back({ctx[(size_t)r] + q0, {r, (int)q0}});
    std::stable_sort(list.begin(), list.end(),
                     [](const auto& a, const auto& b) { return a.first > b.first; });
    for (const auto& t : list) {
      tile[t_at++] = t.second.first;
      tile[t_at++] = t.second.second;
    }
  }
  // wanted rows in the order of the entries as given and of their places
  int64_t w_at = 0;
  for (int e = 0; e < n; ++e)
    for (int64_t k = want_start[(size_t)e]; k < want_start[(size_t)e + 1]; ++k) {
      if (wants[k] < 0 || wants[k] >= q_lens[e]) return c->fail("a wanted place is outside its entry's tokens");
      rows[w_at++] = (int32_t)(row_start[(size_t)row_of_entry[(size_t)e]] + wants[k]);
    }
  c->packed.swap(buf);
  int m = 0;
  meta[m++] = (int32_t)total;
  meta[m++] = num_decode;
  meta[m++] = (int32_t)tiles;
  meta[m++] = (int32_t)R;
  meta[m++] = (int32_t)max_q;
  meta[m++] = (int32_t)max_total;
  meta[m++] = S;
  for (int s = 0; s < S; ++s) meta[m++] = (int32_t)offsets[(size_t)s];
  for (int s = 0; s < S; ++s) meta[m++] = (int32_t)sizes[(size_t)s];
  for (int g = 0; g < G; ++g) meta[m++] = cols[(size_t)g];
  for (int r = 0; r < n; ++r) meta[m++] = order[(size_t)r];
  for (int r = 0; r < n; ++r) meta[m++] = (int32_t)ctx[(size_t)r];
  return 0;
}

// ------------------------------------------------------------------------------------- scheduling
// The decisions of one scheduling step over the cache's counts (infernum-runtime/src/scheduler.rs:289-352 is
// the reference's step: decode every running request, admit first come first served without skipping).
// In this order: one token for every decoding request; the next portion of every running prompt; then
// admissions from the head of the queue while it fits (its first portion and one spare page per running
// request), all under one budget of tokens.  When a decoding request cannot get its page, or no request can
// move at all, the request admitted last is set back: it gives back what it holds (released here) and
// returns to the front of the queue; a request that is alone and still does not fit fails.
//
// Running requests come in the order of admission: rid (their number in the cache, -1 when they hold
// nothing yet), phase (1 = prompt, 2 = decoding, 3 = done but for a token that is still on its way: it keeps
// what it holds, does nothing, is never set back, and will give everything back soon, so a request that cannot
// move because of it waits instead of failing or setting others back) and tokens (prompt and generated).  The queue comes head
// first.  Actions are records of four ints (kind, index, a, b):
//   1 decode   index = running request
//   2 portion  index = running request, a = tokens already stored, b = tokens of the portion
//   3 set back index = running request (everything it held is released)
//   4 fail     index = running request (released), or queue position when a == 3;
//              a: 1 = too large while decoding, 2 = too large for its prompt, 3 = no free page with nothing running
//   5 admit    index = queue position, b = tokens of the first portion
// Portions and decodes of a request that is set back later in the step are taken out again.
// Returns the number of actions, or IA_HOST_ERROR.
int ia_sched_step(void* h, int n_running, const int64_t* run_rid, const int* run_phase, const int64_t* run_tokens,
                  int n_waiting, const int64_t* wait_tokens, int max_batch, int max_prefill, int max_step_tokens,
                  int step_multiple, int* actions, int cap) {
  Cache* c = static_cast<Cache*>(h);
  const size_t G = c->groups.size();
  struct Act { int kind, index, a, b; };
  std::vector<Act> acts;
  std::vector<int> live;                       // running requests still running, in the order of admission
  for (int i = 0; i < n_running; ++i) live.push_back(i);
  std::vector<int64_t> rid(run_rid, run_rid + n_running);
  std::vector<int64_t> promised(G, 0);
  std::vector<int> need(G, 0), prom32(G, 0);
  int64_t budget = max_step_tokens;
  int new_slots = 0, admitted_now = 0;
  bool any_set_back = false;

  auto pages_needed = [&](int64_t r, int64_t n) {
    ia_cache_pages_needed(h, r >= 0 ? 1 : 0, r >= 0 ? r : 0, n, need.data());
  };
  auto fits = [&](int64_t spare) {
    for (size_t g = 0; g < G; ++g)
      if (need[g] + spare + promised[g] > c->groups[g].pool.num_free()) return false;
    return true;
  };
  auto take = [&]() {
    for (size_t g = 0; g < G; ++g) promised[g] += need[g];
  };
  auto tokens_that_fit = [&](int64_t r) {
    for (size_t g = 0; g < G; ++g) prom32[g] = (int)promised[g];
    return ia_cache_tokens_that_fit(h, r >= 0 ? 1 : 0, r >= 0 ? r : 0, prom32.data());
  };
  auto planned = [&]() {
    for (const Act& a : acts)
      if (a.kind == 1 || a.kind == 2 || a.kind == 5) return true;
    return false;
  };
  // A portion that does not reach its prompt's end stops where the step's tokens are a multiple of step_multiple
  // (the rows of the products' tiles), if that leaves it at least half of what it could take.
  auto cut = [&](int64_t n, int64_t remaining) {
    if (step_multiple <= 1 || n >= remaining) return n;
    const int64_t used = (int64_t)max_step_tokens - budget;
    const int64_t whole = (used + n) / step_multiple * step_multiple;
    return (whole - used) * 2 >= n ? whole - used : n;
  };
  auto drop_from_live = [&](int s) { live.erase(std::find(live.begin(), live.end(), s)); };
  // the request admitted last among those that can be set back (-1: none), and whether one is on its way out
  auto last_movable = [&]() {
    for (size_t k = live.size(); k-- > 0;)
      if (run_phase[live[k]] != 3) return live[k];
    return -1;
  };
  auto movable_count = [&]() {
    int n = 0;
    for (int s : live) n += run_phase[s] != 3;
    return n;
  };
  auto any_leaving = [&]() {
    for (int s : live)
      if (run_phase[s] == 3) return true;
    return false;
  };
  std::vector<int> freed;                      // (group, page) pairs of everything released in this step
  auto release = [&](int s) {
    if (rid[(size_t)s] >= 0 && c->admitted(rid[(size_t)s])) {
      ia_cache_release(h, rid[(size_t)s]);
      freed.insert(freed.end(), c->last_freed.begin(), c->last_freed.end());
    }
    rid[(size_t)s] = -1;
  };
  auto set_back = [&](int victim) {
    drop_from_live(victim);
    release(victim);
    acts.erase(std::remove_if(acts.begin(), acts.end(),
                              [&](const Act& a) { return (a.kind == 1 || a.kind == 2) && a.index == victim; }),
               acts.end());
    acts.push_back({3, victim, 0, 0});
    any_set_back = true;
  };

  // one token for every decoding request
  for (size_t i = 0; i < live.size();) {
    const int s = live[i];
    if (run_phase[s] != 2) { ++i; continue; }
    if (rid[(size_t)s] < 0) return c->fail("a decoding request holds nothing in the cache");
    pages_needed(rid[(size_t)s], 1);
    if (fits(0)) {
      take();
      --budget;
      acts.push_back({1, s, 0, 0});
      ++i;
      continue;
    }
    if (any_leaving()) { ++i; continue; }     // pages come back when the leaving requests' tokens are in: wait
    const int victim = last_movable();
    if (victim == s && movable_count() == 1) {
      acts.push_back({4, s, 1, 0});
      drop_from_live(s);
      release(s);
      continue;
    }
    set_back(victim);     // the victim stood at or after i: position i now holds the next request (or none)
  }

  // next portions of running prompts
  bool blocked = false;
  for (size_t i = 0; i < live.size();) {
    const int s = live[i];
    if (run_phase[s] != 1) { ++i; continue; }
    if (budget <= 0) break;
    const int64_t r = (rid[(size_t)s] >= 0 && c->admitted(rid[(size_t)s])) ? rid[(size_t)s] : -1;
    const int64_t cached = r >= 0 ? c->tokens[r] : 0;
    int64_t n = std::min<int64_t>(std::min<int64_t>(run_tokens[s] - cached, max_prefill), budget);
    n = std::min<int64_t>(n, tokens_that_fit(r));
    if (n > 0) n = cut(n, run_tokens[s] - cached);
    if (n <= 0) {
      if (!planned() && !any_leaving()) {
        const int victim = last_movable();        // nobody can move: the last admitted request makes room
        if (victim == s && movable_count() == 1) {
          acts.push_back({4, s, 2, 0});
          drop_from_live(s);
          release(s);
          continue;
        }
        set_back(victim);
        continue;
      }
      blocked = true;
      break;
    }
    if (r < 0) ++new_slots;
    pages_needed(r, n);
    take();
    budget -= n;
    acts.push_back({2, s, (int)cached, (int)n});
    ++i;
  }

  // admissions, first come first served, while the head of the queue fits
  int w = 0;
  while (w < n_waiting && !blocked && !any_set_back && budget > 0 &&
         (int)live.size() + admitted_now < max_batch && (int)c->free_slots.size() - new_slots > 0) {
    const int64_t running_now = (int64_t)live.size() + admitted_now;
    int64_t n = cut(std::min<int64_t>(std::min<int64_t>(wait_tokens[w], max_prefill), budget), wait_tokens[w]);
    pages_needed(-1, n);
    // one page in hand for every running request, so that a newcomer is not set back at once
    if (!fits(running_now)) {
      if (running_now == 0 && !planned()) {
        // alone and still too large for one portion: shrink the portion to the pool
        n = std::min<int64_t>(n, tokens_that_fit(-1));
        if (n > 0) n = cut(n, wait_tokens[w]);
        if (n <= 0) {
          acts.push_back({4, w, 3, 0});
          ++w;
          continue;
        }
        pages_needed(-1, n);
      } else {
        break;
      }
    }
    acts.push_back({5, w, 0, (int)n});
    ++admitted_now;
    ++new_slots;
    take();
    budget -= n;
    ++w;
  }
  c->last_freed.swap(freed);                   // ia_cache_last_freed: all pages given back while deciding
  if ((int)acts.size() > cap) return c->fail("the action buffer is too small");
  for (size_t i = 0; i < acts.size(); ++i) {
    actions[4 * i] = acts[i].kind;
    actions[4 * i + 1] = acts[i].index;
    actions[4 * i + 2] = acts[i].a;
    actions[4 * i + 3] = acts[i].b;
  }
  return (int)acts.size();
}

// the buffer of the last packed step (valid until the next ia_cache_pack_step on this cache)
const int32_t* ia_cache_packed(void* h) { return static_cast<Cache*>(h)->packed.data(); }

}  // extern "C"
