// The host library under AddressSanitizer and UBSan, on the CPU: the cache's bookkeeping under a random order of
// requests (every page free or held once after every operation), and the interpreter of a step's program: random
// programs (arguments of every kind, conditions in every form, stand-ins for unsupported sizes) whose launchers are
// stand-ins that record what they were called with, against a plain evaluation of the same program written here.
// Built and run by tests/test_host_sanitized.py together with csrc/host_core.cpp and csrc/step_program.cpp.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <utility>
#include <vector>

extern "C" {
void* ia_cache_create(int, const int*, const int*, int, int, int);
void ia_cache_destroy(void*);
const char* ia_cache_error(void*);
int ia_cache_admit(void*, int64_t);
int ia_cache_has(void*, int64_t);
int64_t ia_cache_num_tokens(void*, int64_t);
int ia_cache_step_fits(void*, int, const int64_t*, const int*, const int*);
int ia_cache_reserve_step(void*, int, const int64_t*, const int*);
int ia_cache_unreserve_step(void*, int, const int64_t*);
int ia_cache_commit_step(void*, int, const int64_t*, const int*);
int ia_cache_release(void*, int64_t);
int ia_cache_check(void*);
int ia_cache_num_requests(void*);
int ia_cache_pack_step(void*, int, const int64_t*, const int*, const int32_t*, const int*, const int32_t*, int, int,
                       int32_t*, int);
const int32_t* ia_cache_packed(void*);
void* ia_program_create();
void ia_program_destroy(void*);
const char* ia_program_error(void*);
int ia_program_num_ops(void*);
long long ia_program_last_launches(void*);
int ia_program_add_op(void*, void*, const char*, const int64_t*, int, const int64_t*, int, int);
int ia_program_finish(void*, int, int);
int ia_program_run(void*, const int64_t*, int, void* const*, int, void*);
}

#define CHECK(cond)                                                              \
  do {                                                                           \
    if (!(cond)) {                                                               \
      std::fprintf(stderr, "%s:%d: check failed: %s\n", __FILE__, __LINE__, #cond); \
      std::exit(1);                                                              \
    }                                                                            \
  } while (0)

static long g_calls = 0;

static void cache_under_random_requests(unsigned seed) {
  std::mt19937 rng(seed);
  const int kinds[2] = {0, 1}, windows[2] = {0, 10};
  void* c = ia_cache_create(2, kinds, windows, 4, 40, 6);
  CHECK(c);
  std::vector<int64_t> live;
  int64_t next = 0;
  for (int it = 0; it < 4000; ++it) {
    const int op = (int)(rng() % 10);
    if (op < 2 && live.size() < 6) {
      CHECK(ia_cache_admit(c, next) >= 0);
      live.push_back(next++);
    } else if (op < 8 && !live.empty()) {
      // a step of some of the live requests
      std::vector<int64_t> reqs;
      std::vector<int> q, adm, wants_n;
      std::vector<int32_t> toks, wants;
      for (int64_t r : live)
        if (rng() % 3) {
          reqs.push_back(r);
          const int n = 1 + (rng() % 4 == 0 ? (int)(rng() % 9) : 0);
          q.push_back(n);
          adm.push_back(1);
          for (int k = 0; k < n; ++k) toks.push_back((int32_t)(rng() % 100));
          wants_n.push_back(1);
          wants.push_back(n - 1);
        }
      if (reqs.empty()) continue;
      const int n = (int)reqs.size();
      if (ia_cache_step_fits(c, n, reqs.data(), adm.data(), q.data()) != 1) {
        const size_t victim = rng() % live.size();           // out of pages: somebody goes
        CHECK(ia_cache_release(c, live[victim]) == 0);
        live.erase(live.begin() + (long)victim);
      } else {
        CHECK(ia_cache_reserve_step(c, n, reqs.data(), q.data()) == 1);
        if (rng() % 7 == 0) {
          CHECK(ia_cache_unreserve_step(c, n, reqs.data()) == 0);     // the step failed: nothing is stored
        } else {
          const int S = 8 + 2 * 2, meta_len = 7 + 2 * S + 2 + 2 * n;
          std::vector<int32_t> meta((size_t)meta_len);
          CHECK(ia_cache_pack_step(c, n, reqs.data(), q.data(), toks.data(), wants_n.data(), wants.data(),
                                   rng() % 2 ? -1 : 0, 64, meta.data(), meta_len) == 0);
          volatile int32_t last = ia_cache_packed(c)[meta[0] - 1];      // the whole buffer is readable
          (void)last;
          CHECK(ia_cache_commit_step(c, n, reqs.data(), q.data()) == 0);
        }
      }
    } else if (!live.empty()) {
      const size_t victim = rng() % live.size();
      CHECK(ia_cache_release(c, live[victim]) == 0);
      live.erase(live.begin() + (long)victim);
    }
    if (ia_cache_check(c) != 0) {
      std::fprintf(stderr, "seed %u, operation %d: %s\n", seed, it, ia_cache_error(c));
      std::exit(1);
    }
    CHECK(ia_cache_num_requests(c) == (int)live.size());
  }
  ia_cache_destroy(c);
}

// ---- the interpreter of a step's program: random programs against a plain evaluation written here
struct Seen { int op; std::vector<uint64_t> slots; };
static std::vector<Seen> g_seen;
static std::vector<int> g_unsupported;          // operations whose stand-in says "size unsupported"

template <int ID>
static int stand_in(const uint64_t* slots, int n) {
  Seen s;
  s.op = ID;
  s.slots.assign(slots, slots + n);             // reads every slot: one too few shows under the sanitizer
  g_seen.push_back(s);
  ++g_calls;
  for (int u : g_unsupported) if (u == ID) return 10002;
  return ID == 63 ? 77 : 0;                     // operation 63 fails with a code of its own
}

typedef int (*launcher_t)(const uint64_t*, int);
template <int... I>
static std::vector<launcher_t> stand_ins(std::integer_sequence<int, I...>) { return {&stand_in<I>...}; }

struct TTerm { int kind, var; int64_t lo, hi; int group; };
struct TArg { int kind, index; int64_t mul, add; };
struct TOp { std::vector<TArg> args; std::vector<TTerm> terms; int flags; };

static bool plain_term(const TTerm& t, const std::vector<int64_t>& vars) {
  const int64_t x = vars[(size_t)t.var];
  if (t.kind == 0) return t.lo <= x && x <= t.hi;
  if (x < 1) return false;
  int64_t b = (x - 1) / 16;
  if (b > 8) b = 8;
  return (t.lo >> b) & 1;
}

static bool plain_runs(const TOp& op, const std::vector<int64_t>& vars) {
  if (op.terms.empty()) return true;
  int groups = 0;
  for (const TTerm& t : op.terms) groups = t.group + 1 > groups ? t.group + 1 : groups;
  for (int g = 0; g < groups; ++g) {
    bool any = false, all = true;
    for (const TTerm& t : op.terms)
      if (t.group == g) { any = true; all = all && plain_term(t, vars); }
    if (any && all) return true;
  }
  return false;
}

static void interpreter_against_a_plain_evaluation(unsigned seed) {
  std::mt19937 rng(seed);
  const auto fns = stand_ins(std::make_integer_sequence<int, 63>{});
  const int n_vars = 5, n_ptrs = 3, n_ops = 20 + (int)(rng() % 40);
  void* p = ia_program_create();
  CHECK(p);
  std::vector<TOp> ops;
  for (int i = 0; i < n_ops; ++i) {
    TOp op;
    op.flags = (i > 0 && rng() % 6 == 0) ? 1 : 0;
    const int n_args = (int)(rng() % 12);
    for (int k = 0; k < n_args; ++k) {
      TArg a{(int)(rng() % 4), 0, 1, 0};
      if (a.kind == 0) a.add = (int64_t)(((uint64_t)rng() << 32) | rng());
      if (a.kind == 1) { a.index = (int)(rng() % n_vars); a.mul = (int64_t)(rng() % 7) - 2; a.add = (int64_t)(rng() % 100) - 50; }
      if (a.kind == 2) { a.index = (int)(rng() % n_ptrs); a.add = (int64_t)(rng() % 64); }
      op.args.push_back(a);
    }
    if (!op.flags) {
      const int groups = (int)(rng() % 3);
      for (int g = 0; g < groups; ++g) {
        const int n_terms = 1 + (int)(rng() % 3);
        for (int k = 0; k < n_terms; ++k) {
          TTerm t{(int)(rng() % 2), (int)(rng() % n_vars), 0, 0, g};
          if (t.kind == 0) { t.lo = (int64_t)(rng() % 200) - 20; t.hi = t.lo + (int64_t)(rng() % 150); }
          else t.lo = (int64_t)(rng() % 512);
          op.terms.push_back(t);
        }
      }
    }
    std::vector<int64_t> a, t;
    for (const TArg& x : op.args) { a.push_back(x.kind); a.push_back(x.index); a.push_back(x.mul); a.push_back(x.add); }
    for (const TTerm& x : op.terms) { t.push_back(x.kind); t.push_back(x.var); t.push_back(x.lo); t.push_back(x.hi); t.push_back(x.group); }
    CHECK(ia_program_add_op(p, (void*)fns[(size_t)i], "stand-in", a.data(), (int)op.args.size(), t.data(),
                            (int)op.terms.size(), op.flags) == 0);
    ops.push_back(op);
  }
  std::vector<int64_t> none;
  CHECK(ia_program_run(p, none.data(), 0, nullptr, 0, nullptr) != 0);          // not finished yet
  CHECK(ia_program_finish(p, n_vars, n_ptrs) == 0);
  CHECK(ia_program_num_ops(p) == n_ops);
  CHECK(ia_program_add_op(p, (void*)fns[0], "late", nullptr, 0, nullptr, 0, 0) != 0);
  char arrays[3][128];
  void* ptrs[3] = {arrays[0], nullptr, arrays[2]};
  for (int step = 0; step < 60; ++step) {
    std::vector<int64_t> vars((size_t)n_vars);
    for (auto& v : vars) v = (int64_t)(rng() % 220) - 10;
    g_unsupported.clear();
    for (int i = 0; i + 1 < n_ops; ++i)
      if (ops[(size_t)i + 1].flags && rng() % 2) g_unsupported.push_back(i);
    // what must run: in order, an operation whose condition holds; a stand-in only behind an unsupported one
    std::vector<int> want;
    bool unsupported = false;
    for (int i = 0; i < n_ops; ++i) {
      const bool ran = ops[(size_t)i].flags ? unsupported : plain_runs(ops[(size_t)i], vars);
      unsupported = false;
      if (!ran) continue;
      want.push_back(i);
      for (int u : g_unsupported) if (u == i) unsupported = true;
    }
    g_seen.clear();
    void* stream = (void*)(uintptr_t)(0x1000 + step);
    const int rc = ia_program_run(p, vars.data(), n_vars, ptrs, n_ptrs, stream);
    if (rc != 0) { std::fprintf(stderr, "seed %u step %d: %s\n", seed, step, ia_program_error(p)); std::exit(1); }
    CHECK(g_seen.size() == want.size());
    CHECK(ia_program_last_launches(p) == (long long)want.size());
    for (size_t k = 0; k < want.size(); ++k) {
      CHECK(g_seen[k].op == want[k]);
      const TOp& op = ops[(size_t)want[k]];
      CHECK(g_seen[k].slots.size() == op.args.size());
      for (size_t j = 0; j < op.args.size(); ++j) {
        const TArg& a = op.args[j];
        uint64_t v = 0;
        if (a.kind == 0) v = (uint64_t)a.add;
        if (a.kind == 1) v = (uint64_t)(a.mul * vars[(size_t)a.index] + a.add);
        if (a.kind == 2) v = ptrs[a.index] ? (uint64_t)(uintptr_t)((char*)ptrs[a.index] + a.add) : 0;
        if (a.kind == 3) v = (uint64_t)(uintptr_t)stream;
        CHECK(g_seen[k].slots[j] == v);
      }
    }
  }
  // what a caller gets wrong is refused, not run
  std::vector<int64_t> vars((size_t)n_vars, 1);
  CHECK(ia_program_run(p, vars.data(), n_vars - 1, ptrs, n_ptrs, nullptr) != 0);
  CHECK(ia_program_run(p, vars.data(), n_vars, ptrs, n_ptrs + 1, nullptr) != 0);
  ia_program_destroy(p);

  // an operation's own error comes back with its name; an operation that names a number no step brings is
  // refused when the program is finished; a stand-in with nothing before it is refused at once
  p = ia_program_create();
  const int64_t arg[4] = {1, 2, 1, 0};
  CHECK(ia_program_add_op(p, (void*)&stand_in<63>, "fails", arg, 1, nullptr, 0, 1) != 0);
  CHECK(ia_program_add_op(p, (void*)&stand_in<63>, "fails", arg, 1, nullptr, 0, 0) == 0);
  CHECK(ia_program_finish(p, 2, 0) != 0);
  CHECK(ia_program_finish(p, 3, 0) == 0);
  const int64_t three[3] = {0, 0, 5};
  CHECK(ia_program_run(p, three, 3, nullptr, 0, nullptr) == 77);
  CHECK(std::strstr(ia_program_error(p), "fails") != nullptr);
  ia_program_destroy(p);
}

int main() {
  for (unsigned seed = 1; seed <= 12; ++seed) cache_under_random_requests(seed);
  for (unsigned seed = 1; seed <= 40; ++seed) interpreter_against_a_plain_evaluation(seed);
  std::printf("host library: ok (%ld stand-in launches)\n", g_calls);
  return 0;
}
