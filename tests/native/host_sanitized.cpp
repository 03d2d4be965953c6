// The host library under AddressSanitizer and UBSan, on the CPU: the cache's bookkeeping under a random order of
// requests (every page free or held once after every operation), and the native program of a step with kernels
// replaced by stand-ins that write every byte the real kernel would write, into an arena of exactly the size the
// program asked for, so that an intermediate planned too small shows as an overflow.
// Built and run by tests/test_host_sanitized.py together with csrc/host_core.cpp and csrc/step_program.cpp.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
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
void* ia_program_create(const int*, int, const void*);
void ia_program_destroy(void*);
const char* ia_program_error(void*);
void ia_program_set_rotation(void*, int);
int ia_program_set_functions(void*, void* const*, int);
int ia_program_add_norm(void*, const void*, int, float, int);
int ia_program_add_attention(void*, const int*, int, float, void* const*, int, const int*);
int ia_program_add_swiglu(void*, const void*, const void*, int, int, int);
int ia_program_set_head(void*, const void*);
size_t ia_program_finish(void*, int);
int ia_program_set_arena(void*, void*, size_t, void*, size_t);
int ia_program_run(void*, const int*, int, void* const*, int, const int*, const int*, const int*, int, float*, void*);
}

#define CHECK(cond)                                                              \
  do {                                                                           \
    if (!(cond)) {                                                               \
      std::fprintf(stderr, "%s:%d: check failed: %s\n", __FILE__, __LINE__, #cond); \
      std::exit(1);                                                              \
    }                                                                            \
  } while (0)

static size_t es(int dtype) { return dtype == 0 ? 4 : 2; }
static long g_calls = 0;

// ---- stand-ins for the kernel launchers: they write what the kernel would write
static int st_embed(const void*, int, const int*, float* out, int N, int H, int, void*) {
  std::memset(out, 0, (size_t)N * H * 4); ++g_calls; return 0;
}
static int st_add_rmsnorm(float* h, const void* delta, int d_dtype, int splits, int d_rows, int act, const void*, int,
                          void* out, const int* rows, int N, int H, float, void*) {
  if (delta) { volatile char c = ((const char*)delta)[(size_t)splits * d_rows * H * es(d_dtype) - 1]; (void)c; }
  if (!rows && delta) std::memset(h, 0, (size_t)d_rows * H * 4);
  std::memset(out, 0, (size_t)N * H * es(act)); ++g_calls; return 0;
}
static int st_rope(const void* src, int src_dtype, int splits, int src_rows, void* q_out, int q_stride, int act,
                   const int*, const int*, const void*, int, void*, void*, int N, int row, int nh, int, int d, int, int,
                   int, int, void*) {
  volatile char c = ((const char*)src)[(size_t)splits * src_rows * row * es(src_dtype) - 1]; (void)c;
  for (int n = 0; n < N; ++n) std::memset((char*)q_out + (size_t)n * q_stride * es(act), 0, (size_t)nh * d * es(act));
  ++g_calls; return 0;
}
static int st_swiglu(const void* gu, void* out, int dt, int N, int I, void*) {
  volatile char c = ((const char*)gu)[(size_t)N * 2 * I * es(dt) - 1]; (void)c;
  std::memset(out, 0, (size_t)N * I * es(dt)); ++g_calls; return 0;
}
static int st_gemm_generic(const void*, const void*, void* C, int, int out_dtype, int M, int N, int, int, int, int, void*) {
  std::memset(C, 0, (size_t)M * N * es(out_dtype)); ++g_calls; return 0;
}
static int st_gemm_mfma(const void*, const void*, void* C, int M, int N, int, int, void*) {
  std::memset(C, 0, (size_t)M * N * 2); ++g_calls; return 0;
}
static int skinny_splits(int N, int K) { return (N < 300 && K >= 512) ? 3 : 1; }
static int st_gemm_skinny(const void*, const void*, void* C, int out_dtype, int M, int N, int K, int epi, float* ws,
                          size_t ws_floats, void*) {
  const int s = skinny_splits(N, K);
  if (s > 1) { CHECK(ws && ws_floats >= (size_t)s * M * N); std::memset(ws, 0, (size_t)s * M * N * 4); }
  if (C) std::memset(C, 0, (size_t)M * (epi ? N / 2 : N) * es(out_dtype));
  ++g_calls; return 0;
}
static int st_gemm_lt(const void*, const void*, void* C, int M, int N, int, int dt, void*, size_t, void*) {
  std::memset(C, 0, (size_t)M * N * es(dt)); ++g_calls; return 0;
}
static int st_attn_generic(const void*, int, const void*, const void*, void* out, int out_stride, int dt, const int*,
                           const int*, const int*, int, int N, int, int, int, int, int, float, int, void*) {
  std::memset(out, 0, (size_t)N * out_stride * es(dt)); ++g_calls; return 0;
}
static int st_attn_decode(const void*, int, const void*, const void*, void* out, int out_stride, float* po, float* pml,
                          const int*, const int*, int, int B, int nh, int, int, int, float, int, int splits, void*) {
  if (splits > 1) { std::memset(po, 0, (size_t)B * nh * splits * (out_stride / nh) * 4); std::memset(pml, 0, (size_t)B * nh * splits * 8); }
  std::memset(out, 0, (size_t)B * out_stride * 2); ++g_calls; return 0;
}
static int st_attn_fused(const void* src, int src_dtype, int splits_in, int rows, int row, const int*, const void*, int,
                         int, void*, void*, void* out, int out_stride, float* po, float* pml, const int*, const int*,
                         int, int B, int nh, int, int, int, float, int, int splits, void*) {
  volatile char c = ((const char*)src)[(size_t)splits_in * rows * row * es(src_dtype) - 1]; (void)c;
  if (splits > 1) { std::memset(po, 0, (size_t)B * nh * splits * (out_stride / nh) * 4); std::memset(pml, 0, (size_t)B * nh * splits * 8); }
  std::memset(out, 0, (size_t)B * out_stride * 2); ++g_calls; return 0;
}
static int st_attn_prefill(const void*, int, const void*, const void*, void*, int, const int*, const int*, const int*,
                           int, const int* tiles, int num_tiles, int, int, int, int, float, int, int, void*) {
  if (num_tiles) { volatile int t = tiles[2 * num_tiles - 1]; (void)t; }
  ++g_calls; return 0;
}

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

static void program_writes_stay_inside_the_arena(int act, int generic, int T) {
  const int H = 96, V = 300, nh = 6, nkv = 2, d = 16, I = 200, ps = 4, pages = 64;
  std::vector<char> weights(1 << 20), pagesbuf(1 << 20);
  const int settings[10] = {act, H, V, generic, 0, 64, 16384, 1, 64, act};
  void* p = ia_program_create(settings, 10, weights.data());
  CHECK(p);
  void* fns[10] = {(void*)st_embed, (void*)st_add_rmsnorm, (void*)st_rope, (void*)st_swiglu, (void*)st_gemm_generic,
                   (void*)st_gemm_mfma, (void*)st_gemm_skinny, (void*)skinny_splits, (void*)st_gemm_lt,
                   (void*)st_attn_generic};
  CHECK(ia_program_set_functions(p, fns, 10) == 0);
  ia_program_set_rotation(p, 1);
  const int masks[3] = {-1, 0, 2};
  for (int layer = 0; layer < 3; ++layer) {
    CHECK(ia_program_add_norm(p, weights.data(), act, 1e-5f, 0) == 0);
    const int use_mfma = (act == 1 && !generic) ? 1 : 0;
    const int ints[11] = {nh, nkv, d, layer == 1 ? 9 : 0, d, 1, layer == 1 ? 1 : 0, layer == 2 ? 0 : 1, use_mfma, ps, pages};
    void* ptrs[8] = {weights.data(), weights.data(), weights.data(), pagesbuf.data(), pagesbuf.data(),
                     (void*)st_attn_decode, (void*)st_attn_fused, (void*)st_attn_prefill};
    CHECK(ia_program_add_attention(p, ints, 11, 0.25f, ptrs, 8, masks) == 0);
    CHECK(ia_program_add_norm(p, weights.data(), act, 1e-5f, 0) == 0);
    CHECK(ia_program_add_swiglu(p, weights.data(), weights.data(), I, -1, 1 << 3) == 0);
  }
  CHECK(ia_program_add_norm(p, weights.data(), act, 1e-5f, 1) == 0);
  CHECK(ia_program_set_head(p, weights.data()) == 0);
  const size_t need = ia_program_finish(p, T);
  CHECK(need > 0);
  char* arena = (char*)std::malloc(need);                 // exactly what was asked for: ASan guards both ends
  CHECK(ia_program_set_arena(p, arena, need, nullptr, 0) == 0);
  std::vector<int> ids((size_t)T, 1), tiles(2 * (size_t)T, 0), bt((size_t)T * 64, 0);
  std::vector<float> logits((size_t)T * V);
  // steps of many shapes: all single tokens (few, many), one long portion, mixed
  const int shapes[][3] = {{1, 1, 1}, {8, 8, 8}, {64, 64, 64}, {T < 100 ? T : 100, 100, 100}, {T, 1, 0}, {T, 5, 3},
                           {70, 3, 0}, {T, T, T}, {130, 2, 1}};
  for (const auto& sh : shapes) {
    const int N = sh[0] <= T ? sh[0] : T, B = sh[1] <= N ? sh[1] : N, nd = sh[2] <= B ? sh[2] : B;
    const int R = B;
    const int ints[7] = {N, B, nd, R, 200, (N + 63) / 64, 2};
    void* ptrs[11] = {ids.data(), ids.data(), ids.data(), ids.data(), ids.data(), ids.data(), tiles.data(),
                      bt.data(), ids.data(), bt.data(), ids.data()};
    // parts of the keys as the host chooses them: several only while the requests are few
    const int parts = nd <= 64 ? 3 : 1;
    const int cols[2] = {64, 64}, splits[3] = {parts, parts, parts}, hpw[3] = {0, 2, 0};
    const int rc = ia_program_run(p, ints, 7, ptrs, 11, cols, splits, hpw, 3, logits.data(), nullptr);
    if (rc != 0) {
      std::fprintf(stderr, "run N=%d B=%d nd=%d: %s\n", N, B, nd, ia_program_error(p));
      std::exit(1);
    }
  }
  // what a caller gets wrong is refused, not run
  const int bad[7] = {T + 1, 1, 1, 1, 10, 1, 2};
  void* ptrs[11] = {ids.data(), ids.data(), ids.data(), ids.data(), ids.data(), ids.data(), tiles.data(), bt.data(),
                    ids.data(), bt.data(), ids.data()};
  const int cols[2] = {64, 64}, one[3] = {1, 1, 1};
  CHECK(ia_program_run(p, bad, 7, ptrs, 11, cols, one, one, 3, logits.data(), nullptr) != 0);
  const int ok[7] = {4, 1, 0, 1, 10, 1, 2};
  CHECK(ia_program_run(p, ok, 7, ptrs, 11, cols, one, one, 2, logits.data(), nullptr) != 0);   // too few attention numbers
  std::free(arena);
  ia_program_destroy(p);
}

int main() {
  for (unsigned seed = 1; seed <= 12; ++seed) cache_under_random_requests(seed);
  for (int act = 0; act < 2; ++act)
    for (int generic = 0; generic < 2; ++generic)
      for (int T : {7, 64, 129, 600}) program_writes_stay_inside_the_arena(act, generic, T);
  std::printf("host library: ok (%ld stand-in launches)\n", g_calls);
  return 0;
}
