// A model's forward pass of one step as a native program: the sequence of kernel launches that the parts of a
// decoder make (embedding, add + RMSNorm, attention over the paged cache, SwiGLU feed-forward, head), run from
// one call instead of one call per launch from Python.
//
// The program is a list of operations over three registers: the fp32 residual stream `h`, the normalised
// activations `x`, and a `pending` delta that the next norm adds to `h` (a tensor, or a stack of fp32 partial
// sums of a matrix product whose inner dimension was split).  Python builds the list from the model's parts
// (every built-in part describes itself as one operation; a model with a part that cannot falls back to the
// parts' own `forward`), gives the entry points of the kernel libraries as function pointers, and an arena for
// the intermediates.  Every choice of a kernel made here (which matrix product for how many rows, rotation inside
// the attention kernel or before it, the plain twins) is the same as in `parts/linear.py` and
// `parts/attention.py`, so that both ways give the same bits; tests compare them.
//
// This file makes no GPU call of its own: it only calls the libraries' launchers.  (The reference runs its
// graph of operations natively too: infernum-cuda/src/inner/cuda_graph_engine.rs.)
#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

namespace {

enum { DT_F32 = 0, DT_BF16 = 1 };
enum { ERR_BAD_ARG = 10001, ERR_UNSUPPORTED = 10002, ERR_ARENA = 10005, ERR_PROGRAM = 10006 };
enum { EPI_NONE = 0, EPI_SWIGLU = 1 };
enum { GEMM_LIBRARY = 0, GEMM_MFMA = 1 };
enum { OP_NORM = 1, OP_ATTENTION = 2, OP_SWIGLU_FF = 3 };
const int SKINNY_MAX_M = 128;

typedef void* stream_t;
typedef int (*fn_embed)(const void*, int, const int*, float*, int, int, int, stream_t);
typedef int (*fn_add_rmsnorm)(float*, const void*, int, int, int, int, const void*, int, void*, const int*, int, int,
                              float, stream_t);
typedef int (*fn_rope_kv_append)(const void*, int, int, int, void*, int, int, const int*, const int*, const void*, int,
                                 void*, void*, int, int, int, int, int, int, int, int, int, stream_t);
typedef int (*fn_swiglu)(const void*, void*, int, int, int, stream_t);
typedef int (*fn_gemm_generic)(const void*, const void*, void*, int, int, int, int, int, int, int, int, stream_t);
typedef int (*fn_gemm_mfma)(const void*, const void*, void*, int, int, int, int, stream_t);
typedef int (*fn_gemm_skinny)(const void*, const void*, void*, int, int, int, int, int, float*, size_t, stream_t);
typedef int (*fn_gemm_skinny_splits)(int, int);
typedef int (*fn_gemm_lt)(const void*, const void*, void*, int, int, int, int, void*, size_t, stream_t);
typedef int (*fn_attention_generic)(const void*, int, const void*, const void*, void*, int, int, const int*,
                                    const int*, const int*, int, int, int, int, int, int, int, float, int, stream_t);
typedef int (*fn_attn_decode)(const void*, int, const void*, const void*, void*, int, float*, float*, const int*,
                              const int*, int, int, int, int, int, int, float, int, int, stream_t);
typedef int (*fn_attn_decode_fused)(const void*, int, int, int, int, const int*, const void*, int, int, void*, void*,
                                    void*, int, float*, float*, const int*, const int*, int, int, int, int, int, int,
                                    float, int, int, stream_t);
typedef int (*fn_attn_prefill)(const void*, int, const void*, const void*, void*, int, const int*, const int*,
                               const int*, int, const int*, int, int, int, int, int, float, int, int, stream_t);

// indices of ia_program_set_functions
enum { FN_EMBED, FN_ADD_RMSNORM, FN_ROPE_KV_APPEND, FN_SWIGLU, FN_GEMM_GENERIC, FN_GEMM_MFMA, FN_GEMM_SKINNY,
       FN_GEMM_SKINNY_SPLITS, FN_GEMM_LT, FN_ATTENTION_GENERIC, FN_COUNT };

struct Weight {          // a matrix [N, K] in the activations' type
  const void* w = nullptr;
  int N = 0, K = 0, splits = 1;      // splits: parts of K in the weight-streaming product (a function of N, K)
  int library_rows = -1;             // measured: bit b set = 16 b + 1 .. 16 b + 16 rows go to the library; -1: the rule
};

struct Op {
  int kind = 0;
  // norm
  const void* norm_w = nullptr;
  int norm_w_dtype = 0;
  float eps = 0.f;
  // attention
  Weight qkv, q_only, o;              // q_only: the first nh*d rows of qkv, for a run that reads another's pages
  int nh = 0, nkv = 0, d = 0, window = 0, rot = 0, freq_f64 = 0, group = 0, writable = 1, use_mfma = 0;
  int page_size = 0, num_pages = 0;
  float scale = 0.f;
  const void* inv_freq = nullptr;
  void* k_pages = nullptr;
  void* v_pages = nullptr;
  fn_attn_decode attn_decode = nullptr;
  fn_attn_decode_fused attn_decode_fused = nullptr;
  fn_attn_prefill attn_prefill = nullptr;
  // feed-forward
  Weight gate_up, down;
};

struct Value {           // a matrix [rows, cols] as a tensor (splits == 0) or as fp32 partial sums [splits, rows, cols]
  void* p = nullptr;
  int splits = 0;
  int dtype = DT_F32;
};

struct Buffers {         // offsets into the arena, in bytes
  size_t h, x, qkv, qrot, aout, part_o, part_ml, mix, gu, act, ff, head_ws, total;
  size_t part_o_floats, part_ml_floats;
};

struct Program {
  int act = DT_BF16;                 // type of activations, matrices and pages
  int H = 0, V = 0;
  int generic = 0;                   // 1: the plain twins for every product and the attention
  int prefill_gemm = GEMM_LIBRARY;
  int skinny_rows_any_width = 64, skinny_wide = 16384, rotate_in_attention = 1, rotate_up_to = 64;
  const void* table = nullptr;
  int table_dtype = 0;
  std::vector<Op> ops;
  Op final_norm;
  bool has_final_norm = false;
  Weight head;
  void* fns[FN_COUNT] = {nullptr};
  int max_tokens = 0;
  Buffers buf{};
  char* arena = nullptr;
  size_t arena_bytes = 0;
  void* lt_workspace = nullptr;
  size_t lt_workspace_bytes = 0;
  std::string error;
};

struct Step {            // what Python passes for one step (see ia_program_run)
  int N, B, num_decode, R, max_total_len, num_tiles;
  const int *token_ids, *positions, *token_seq, *seq_starts, *seq_ctx, *logit_rows, *tiles;
  const int* const* block_tables;    // per group
  const int* bt_cols;                // per group
  const int* const* slots;           // per group
  const int* attn_splits;            // per attention operation, in program order: parts of the keys for the decode rows
  const int* attn_hpw;               // per attention operation: heads per workgroup for the portions of prompts
  stream_t stream;
};

size_t es(int dtype) { return dtype == DT_F32 ? 4 : 2; }
size_t up256(size_t n) { return (n + 255) & ~(size_t)255; }

int fail(Program* p, int code, const std::string& what) {
  p->error = what + ": error " + std::to_string(code);
  return code;
}

bool skinny_supported(int M, int N, int K) { return M > 0 && M <= SKINNY_MAX_M && K % 8 == 0 && K >= 8 && N >= 1; }
bool mfma_supported(int M, int N, int K) {
  return M >= 1 && N >= 1 && K >= 64 && K % 64 == 0 && (double)M * K * 2 < 4294967296.0 && (double)N * K * 2 < 4294967296.0;
}

// y = x W^T.  `out`: where a tensor result goes ([M, N] or [M, N/2] with the SwiGLU epilogue, in out_dtype);
// `scratch`: room for partial sums ([splits, M, N] fp32) or for the product before the activation.  With
// keep_split the result may be the partial sums themselves (then they lie in `out`).
int linear(Program* p, const Step& s, const void* x, int M, const Weight& w, int out_dtype, int epilogue,
           bool keep_split, void* out, void* scratch, Value* result) {
  const int N = w.N, K = w.K;
  const int in_dtype = p->act;
  result->p = out;
  result->splits = 0;
  result->dtype = out_dtype;
  int rc;
  void* y = epilogue == EPI_SWIGLU ? scratch : out;
  if (p->generic || in_dtype == DT_F32) {
    rc = ((fn_gemm_generic)p->fns[FN_GEMM_GENERIC])(x, w.w, y, in_dtype, out_dtype, M, N, K, K, K, N, s.stream);
    if (rc) return fail(p, rc, "gemm_generic");
  } else if (skinny_supported(M, N, K) &&
             (out_dtype != DT_BF16 ||
              (w.library_rows >= 0 ? !((w.library_rows >> ((M - 1) / 16)) & 1)
                                   : (M <= p->skinny_rows_any_width || N < p->skinny_wide)))) {
    fn_gemm_skinny skinny = (fn_gemm_skinny)p->fns[FN_GEMM_SKINNY];
    const size_t ws_floats = w.splits > 1 ? (size_t)w.splits * M * N : 0;
    if (keep_split && epilogue == EPI_NONE && w.splits > 1) {
      rc = skinny(x, w.w, nullptr, 0, M, N, K, 0, (float*)out, ws_floats, s.stream);
      if (rc) return fail(p, rc, "gemm_skinny");
      result->splits = w.splits;
      result->dtype = DT_F32;
      return 0;
    }
    rc = skinny(x, w.w, out, out_dtype, M, N, K, epilogue, w.splits > 1 ? (float*)scratch : nullptr, ws_floats,
                s.stream);
    if (rc) return fail(p, rc, "gemm_skinny");
    return 0;
  } else if (out_dtype == DT_BF16) {
    if (p->prefill_gemm == GEMM_MFMA && mfma_supported(M, N, K)) {
      rc = ((fn_gemm_mfma)p->fns[FN_GEMM_MFMA])(x, w.w, y, M, N, K, 0, s.stream);
      if (rc) return fail(p, rc, "gemm_mfma");
    } else {
      rc = ((fn_gemm_lt)p->fns[FN_GEMM_LT])(x, w.w, y, M, N, K, DT_BF16, p->lt_workspace, p->lt_workspace_bytes,
                                           s.stream);
      if (rc == ERR_UNSUPPORTED) {          // the library has no algorithm for this shape
        if (mfma_supported(M, N, K))
          rc = ((fn_gemm_mfma)p->fns[FN_GEMM_MFMA])(x, w.w, y, M, N, K, 0, s.stream);
        else
          rc = ((fn_gemm_generic)p->fns[FN_GEMM_GENERIC])(x, w.w, y, in_dtype, out_dtype, M, N, K, K, K, N, s.stream);
      }
      if (rc) return fail(p, rc, "gemm_library");
    }
  } else if (skinny_supported(1, N, K)) {
    // fp32 result from bf16 operands, many rows: 128 rows at a time through the weight-streaming product
    fn_gemm_skinny skinny = (fn_gemm_skinny)p->fns[FN_GEMM_SKINNY];
    for (int m0 = 0; m0 < M; m0 += SKINNY_MAX_M) {
      const int m = std::min(SKINNY_MAX_M, M - m0);
      const size_t ws_floats = w.splits > 1 ? (size_t)w.splits * m * N : 0;
      rc = skinny((const char*)x + (size_t)m0 * K * 2, w.w, (char*)y + (size_t)m0 * N * es(out_dtype), out_dtype, m, N,
                  K, 0, w.splits > 1 ? (float*)scratch : nullptr, ws_floats, s.stream);
      if (rc) return fail(p, rc, "gemm_skinny");
    }
    if (epilogue == EPI_SWIGLU) return fail(p, ERR_PROGRAM, "an fp32 product of many rows has no activation here");
  } else {
    rc = ((fn_gemm_generic)p->fns[FN_GEMM_GENERIC])(x, w.w, y, in_dtype, out_dtype, M, N, K, K, K, N, s.stream);
    if (rc) return fail(p, rc, "gemm_generic");
  }
  if (epilogue == EPI_SWIGLU) {
    rc = ((fn_swiglu)p->fns[FN_SWIGLU])(y, out, out_dtype, M, N / 2, s.stream);
    if (rc) return fail(p, rc, "swiglu");
  }
  return 0;
}

// h += pending; out = norm(h) (all rows), or the norm of the chosen rows with h untouched
int add_norm(Program* p, const Step& s, const Op& op, float* h, const Value& pending, void* out, const int* rows,
             int n_out) {
  const void* delta = pending.p;
  int splits = 1, d_code = p->act;
  if (pending.p && pending.splits > 0) {
    splits = pending.splits;
    d_code = DT_F32;
  }
  const int rc = ((fn_add_rmsnorm)p->fns[FN_ADD_RMSNORM])(h, delta, d_code, splits, s.N, p->act, op.norm_w,
                                                          op.norm_w_dtype, out, rows, n_out, p->H, op.eps, s.stream);
  return rc ? fail(p, rc, "add_rmsnorm") : 0;
}

int attention(Program* p, const Step& s, const Op& op, int attn_index, char* a, const void* x, Value* result) {
  const Buffers& b = p->buf;
  const int N = s.N, nh = op.nh, nkv = op.nkv, d = op.d, g = op.group;
  const int* bt = s.block_tables[g];
  const int bt_cols = s.bt_cols[g];
  const int* slots = op.writable ? s.slots[g] : nullptr;
  const Weight& wq = op.writable ? op.qkv : op.q_only;    // another run's keys and values: only queries are made
  const int row = wq.N;
  const int rot = op.inv_freq ? op.rot : 0;
  void* out = a + b.aout;
  int rc;
  Value qkv;
  rc = linear(p, s, x, N, wq, p->act, EPI_NONE, true, a + b.qkv, nullptr, &qkv);
  if (rc) return rc;
  const int splits = s.attn_splits[attn_index];
  float* part_o = splits > 1 ? (float*)(a + b.part_o) : nullptr;
  float* part_ml = splits > 1 ? (float*)(a + b.part_ml) : nullptr;
  if (splits > 1 && ((size_t)s.num_decode * nh * splits * d > b.part_o_floats ||
                     (size_t)s.num_decode * nh * splits * 2 > b.part_ml_floats))
    return fail(p, ERR_ARENA, "attention: the parts of the keys do not fit the arena");
  if (op.use_mfma && p->rotate_in_attention && s.num_decode == N && N > 0 && N <= p->rotate_up_to &&
      op.page_size % 4 == 0) {
    // every request brings one token: rotation, the write to the pages and attention are one launch
    if ((long long)bt_cols * op.page_size < s.max_total_len) return fail(p, ERR_BAD_ARG, "attention: block tables too narrow");
    rc = op.attn_decode_fused(qkv.p, qkv.splits ? DT_F32 : DT_BF16, qkv.splits ? qkv.splits : 1, N, row, slots,
                              op.inv_freq, op.freq_f64, rot, op.k_pages, op.v_pages, out, nh * d, part_o, part_ml,
                              s.positions, bt, bt_cols, N, nh, nkv, op.page_size, op.num_pages, op.scale, op.window,
                              splits, s.stream);
    if (rc) return fail(p, rc, "attention_decode_rotating");
  } else {
    const void* q = qkv.p;
    int q_stride = row;
    void* q_out = qkv.p;
    if (qkv.splits) {                    // partial sums: the rotated queries get a tensor of their own
      q_out = a + b.qrot;
      q = q_out;
      q_stride = nh * d;
    }
    rc = ((fn_rope_kv_append)p->fns[FN_ROPE_KV_APPEND])(
        qkv.p, qkv.splits ? DT_F32 : p->act, qkv.splits ? qkv.splits : 1, N, q_out, q_stride, p->act, s.positions,
        slots, op.inv_freq, op.freq_f64, op.writable ? op.k_pages : nullptr, op.writable ? op.v_pages : nullptr, N, row,
        nh, nkv, d, rot, op.writable ? op.page_size : 0, op.writable ? op.num_pages : 0, op.writable ? 1 : 0, s.stream);
    if (rc) return fail(p, rc, "rope_kv_append");
    if (!op.use_mfma || op.page_size % 4) {
      rc = ((fn_attention_generic)p->fns[FN_ATTENTION_GENERIC])(q, q_stride, op.k_pages, op.v_pages, out, nh * d, p->act,
                                                                s.token_seq, s.positions, bt, bt_cols, N, nh, nkv, d,
                                                                op.page_size, op.num_pages, op.scale, op.window,
                                                                s.stream);
      if (rc) return fail(p, rc, "attention_generic");
    } else {
      if (s.num_decode > 0) {
        if ((long long)bt_cols * op.page_size < s.max_total_len)
          return fail(p, ERR_BAD_ARG, "attention: block tables too narrow");
        rc = op.attn_decode(q, q_stride, op.k_pages, op.v_pages, out, nh * d, part_o, part_ml, s.positions, bt, bt_cols,
                            s.num_decode, nh, nkv, op.page_size, op.num_pages, op.scale, op.window, splits, s.stream);
        if (rc) return fail(p, rc, "attention_decode");
      }
      if (s.B > s.num_decode) {
        rc = op.attn_prefill(q, q_stride, op.k_pages, op.v_pages, out, nh * d, s.seq_starts, s.seq_ctx, bt, bt_cols,
                             s.tiles, s.num_tiles, nh, nkv, op.page_size, op.num_pages, op.scale, op.window,
                             s.attn_hpw[attn_index], s.stream);
        if (rc) return fail(p, rc, "attention_prefill");
      }
    }
  }
  return linear(p, s, out, N, op.o, p->act, EPI_NONE, true, a + b.mix, nullptr, result);
}

int feed_forward(Program* p, const Step& s, const Op& op, char* a, const void* x, Value* result) {
  const Buffers& b = p->buf;
  Value act;
  int rc = linear(p, s, x, s.N, op.gate_up, p->act, EPI_SWIGLU, false, a + b.act, a + b.gu, &act);
  if (rc) return rc;
  return linear(p, s, act.p, s.N, op.down, p->act, EPI_NONE, true, a + b.ff, nullptr, result);
}

size_t value_bytes(const Program* p, const Weight& w, int T, bool with_activation) {
  // the largest of: the tensor [T, N]; the partial sums [splits, min(T, 128), N]
  size_t n = (size_t)T * w.N * es(p->act);
  if (w.splits > 1) n = std::max(n, (size_t)w.splits * std::min(T, SKINNY_MAX_M) * w.N * 4);
  (void)with_activation;
  return n;
}

void plan_buffers(Program* p) {
  const int T = p->max_tokens;
  Buffers& b = p->buf;
  size_t qkv = 0, qrot = 0, aout = 0, mix = 0, gu = 0, act = 0, ff = 0, part = 0, part_ml = 0;
  for (const Op& op : p->ops) {
    if (op.kind == OP_ATTENTION) {
      qkv = std::max(qkv, value_bytes(p, op.qkv, T, false));
      qrot = std::max(qrot, (size_t)T * op.nh * op.d * es(p->act));
      aout = std::max(aout, (size_t)T * op.nh * op.d * es(p->act));
      mix = std::max(mix, value_bytes(p, op.o, T, false));
      // parts of the keys: requests x parts is bounded by what fills the GPU plus the requests themselves
      const size_t recs = (size_t)T + 1024;
      part = std::max(part, recs * op.nh * op.d);
      part_ml = std::max(part_ml, recs * op.nh * 2);
    } else if (op.kind == OP_SWIGLU_FF) {
      gu = std::max(gu, value_bytes(p, op.gate_up, T, true));
      act = std::max(act, (size_t)T * (op.gate_up.N / 2) * es(p->act));
      ff = std::max(ff, value_bytes(p, op.down, T, false));
    }
  }
  size_t at = 0;
  auto take = [&](size_t bytes) { size_t o = at; at += up256(bytes); return o; };
  b.h = take((size_t)T * p->H * 4);
  b.x = take((size_t)T * p->H * es(p->act));
  b.qkv = take(qkv);
  b.qrot = take(qrot);
  b.aout = take(aout);
  b.part_o = take(part * 4);
  b.part_ml = take(part_ml * 4);
  b.part_o_floats = part;
  b.part_ml_floats = part_ml;
  b.mix = take(mix);
  b.gu = take(gu);
  b.act = take(act);
  b.ff = take(ff);
  b.head_ws = take(p->head.splits > 1 ? (size_t)p->head.splits * SKINNY_MAX_M * p->head.N * 4 : 0);
  b.total = at;
}

}  // namespace

extern "C" {

// settings: [activations' type, H, V, generic, prefill gemm, skinny_rows_any_width, skinny_wide,
//            rotate_in_attention, rotate_up_to, table dtype]
void* ia_program_create(const int* settings, int n, const void* table) {
  if (n != 10) return nullptr;
  Program* p = new Program();
  p->act = settings[0];
  p->H = settings[1];
  p->V = settings[2];
  p->generic = settings[3];
  p->prefill_gemm = settings[4];
  p->skinny_rows_any_width = settings[5];
  p->skinny_wide = settings[6];
  p->rotate_in_attention = settings[7];
  p->rotate_up_to = settings[8];
  p->table_dtype = settings[9];
  p->table = table;
  return p;
}

// where steps of single tokens rotate queries and keys: 1 inside the attention kernel, 0 in the kernel before it
void ia_program_set_rotation(void* h, int in_attention) { static_cast<Program*>(h)->rotate_in_attention = in_attention; }

void ia_program_destroy(void* h) { delete static_cast<Program*>(h); }

const char* ia_program_error(void* h) { return static_cast<Program*>(h)->error.c_str(); }

int ia_program_set_functions(void* h, void* const* fns, int n) {
  Program* p = static_cast<Program*>(h);
  if (n != FN_COUNT) return fail(p, ERR_BAD_ARG, "set_functions");
  for (int i = 0; i < n; ++i) {
    if (!fns[i]) return fail(p, ERR_BAD_ARG, "set_functions: entry point " + std::to_string(i) + " is missing");
    p->fns[i] = fns[i];
  }
  return 0;
}

static int set_weight(Program* p, Weight* w, const void* ptr, int N, int K) {
  if (!ptr || N <= 0 || K <= 0) return fail(p, ERR_BAD_ARG, "a weight of the program");
  if (!p->fns[FN_GEMM_SKINNY_SPLITS]) return fail(p, ERR_PROGRAM, "set the functions before the operations");
  w->w = ptr;
  w->N = N;
  w->K = K;
  w->splits = (p->act == DT_BF16 && !p->generic) ? ((fn_gemm_skinny_splits)p->fns[FN_GEMM_SKINNY_SPLITS])(N, K) : 1;
  if (w->splits < 1) w->splits = 1;
  return 0;
}

// a norm: x = norm(h += pending).  final != 0: the norm before the head, on the wanted rows only
int ia_program_add_norm(void* h, const void* weight, int weight_dtype, float eps, int final) {
  Program* p = static_cast<Program*>(h);
  if (!weight || !(eps > 0.f)) return fail(p, ERR_BAD_ARG, "norm");
  Op op;
  op.kind = OP_NORM;
  op.norm_w = weight;
  op.norm_w_dtype = weight_dtype;
  op.eps = eps;
  if (final) {
    p->final_norm = op;
    p->has_final_norm = true;
  } else {
    p->ops.push_back(op);
  }
  return 0;
}

// attention: pending = attention(x).  ints: [nh, nkv, d, window, rot, freq_f64, group, writable, use_mfma,
// page_size, num_pages]; ptrs: [w_qkv, w_o, inv_freq or null, k_pages, v_pages, ia_attn_decode,
// ia_attn_decode_fused, ia_attn_prefill (the three may be null without use_mfma)]
// library_rows: the measured choice of a product for the qkv, the queries-only and the output weight (see Weight)
int ia_program_add_attention(void* h, const int* ints, int n_ints, float scale, void* const* ptrs, int n_ptrs,
                             const int* library_rows) {
  Program* p = static_cast<Program*>(h);
  if (n_ints != 11 || n_ptrs != 8) return fail(p, ERR_BAD_ARG, "attention");
  Op op;
  op.kind = OP_ATTENTION;
  op.nh = ints[0]; op.nkv = ints[1]; op.d = ints[2]; op.window = ints[3]; op.rot = ints[4]; op.freq_f64 = ints[5];
  op.group = ints[6]; op.writable = ints[7]; op.use_mfma = ints[8]; op.page_size = ints[9]; op.num_pages = ints[10];
  op.scale = scale;
  if (op.nh <= 0 || op.nkv <= 0 || op.nh % op.nkv || op.d <= 0 || op.group < 0 || op.page_size <= 0 || op.num_pages <= 0)
    return fail(p, ERR_BAD_ARG, "attention: sizes");
  int rc = set_weight(p, &op.qkv, ptrs[0], (op.nh + 2 * op.nkv) * op.d, p->H);
  if (rc) return rc;
  rc = set_weight(p, &op.q_only, ptrs[0], op.nh * op.d, p->H);
  if (rc) return rc;
  rc = set_weight(p, &op.o, ptrs[1], p->H, op.nh * op.d);
  if (rc) return rc;
  op.qkv.library_rows = library_rows[0];
  op.q_only.library_rows = library_rows[1];
  op.o.library_rows = library_rows[2];
  op.inv_freq = ptrs[2];
  op.k_pages = ptrs[3];
  op.v_pages = ptrs[4];
  if (!op.k_pages || !op.v_pages) return fail(p, ERR_BAD_ARG, "attention: pages");
  op.attn_decode = (fn_attn_decode)ptrs[5];
  op.attn_decode_fused = (fn_attn_decode_fused)ptrs[6];
  op.attn_prefill = (fn_attn_prefill)ptrs[7];
  if (op.use_mfma && (!op.attn_decode || !op.attn_decode_fused || !op.attn_prefill))
    return fail(p, ERR_BAD_ARG, "attention: the MFMA kernels' entry points");
  p->ops.push_back(op);
  return 0;
}

// SwiGLU feed-forward: pending = down(silu(gate(x)) * up(x)); gate and up are one matrix [2 I, H]
int ia_program_add_swiglu(void* h, const void* w_gate_up, const void* w_down, int I, int gate_up_library_rows,
                          int down_library_rows) {
  Program* p = static_cast<Program*>(h);
  Op op;
  op.kind = OP_SWIGLU_FF;
  int rc = set_weight(p, &op.gate_up, w_gate_up, 2 * I, p->H);
  if (rc) return rc;
  rc = set_weight(p, &op.down, w_down, p->H, I);
  if (rc) return rc;
  op.gate_up.library_rows = gate_up_library_rows;
  op.down.library_rows = down_library_rows;
  p->ops.push_back(op);
  return 0;
}

int ia_program_set_head(void* h, const void* weight) {
  Program* p = static_cast<Program*>(h);
  return set_weight(p, &p->head, weight, p->V, p->H);
}

// The program is complete: bytes of the arena that steps of up to max_tokens tokens need (0 on error).
size_t ia_program_finish(void* h, int max_tokens) {
  Program* p = static_cast<Program*>(h);
  if (max_tokens <= 0 || !p->has_final_norm || !p->head.w || !p->table || p->ops.empty()) {
    fail(p, ERR_PROGRAM, "the program needs operations, a final norm, a head and a limit of tokens");
    return 0;
  }
  p->max_tokens = max_tokens;
  plan_buffers(p);
  return p->buf.total;
}

int ia_program_set_arena(void* h, void* arena, size_t bytes, void* lt_workspace, size_t lt_bytes) {
  Program* p = static_cast<Program*>(h);
  if (!arena || bytes < p->buf.total) return fail(p, ERR_ARENA, "the arena is smaller than the program needs");
  p->arena = static_cast<char*>(arena);
  p->arena_bytes = bytes;
  p->lt_workspace = lt_workspace;
  p->lt_workspace_bytes = lt_bytes;
  return 0;
}

// One step.  ints: [N, requests, single-token requests, wanted rows, longest total length, tiles, groups];
// ptrs: [token_ids, positions, token_seq, seq_starts, seq_ctx, logit_rows, tiles], then per group
// [block table, slots]; bt_cols per group; attn_splits and attn_hpw per attention operation; logits: fp32
// [wanted rows, V] of the caller.
int ia_program_run(void* h, const int* ints, int n_ints, void* const* ptrs, int n_ptrs, const int* bt_cols,
                   const int* attn_splits, const int* attn_hpw, int n_attn, float* logits, void* stream) {
  Program* p = static_cast<Program*>(h);
  if (!p->arena) return fail(p, ERR_ARENA, "no arena");
  if (n_ints != 7) return fail(p, ERR_BAD_ARG, "run: ints");
  Step s;
  s.N = ints[0]; s.B = ints[1]; s.num_decode = ints[2]; s.R = ints[3]; s.max_total_len = ints[4]; s.num_tiles = ints[5];
  const int groups = ints[6];
  if (s.N <= 0 || s.N > p->max_tokens || s.B <= 0 || s.num_decode < 0 || s.num_decode > s.B || s.R < 0 || groups < 0 ||
      n_ptrs != 7 + 2 * groups)
    return fail(p, ERR_BAD_ARG, "run: sizes");
  s.token_ids = (const int*)ptrs[0]; s.positions = (const int*)ptrs[1]; s.token_seq = (const int*)ptrs[2];
  s.seq_starts = (const int*)ptrs[3]; s.seq_ctx = (const int*)ptrs[4]; s.logit_rows = (const int*)ptrs[5];
  s.tiles = (const int*)ptrs[6];
  std::vector<const int*> bts((size_t)groups), slots((size_t)groups);
  for (int g = 0; g < groups; ++g) {
    bts[(size_t)g] = (const int*)ptrs[7 + 2 * g];
    slots[(size_t)g] = (const int*)ptrs[8 + 2 * g];
  }
  s.block_tables = bts.data();
  s.slots = slots.data();
  s.bt_cols = bt_cols;
  s.attn_splits = attn_splits;
  s.attn_hpw = attn_hpw;
  s.stream = stream;
  int n_attention = 0;
  for (const Op& op : p->ops) {
    if (op.kind != OP_ATTENTION) continue;
    if (op.group >= groups) return fail(p, ERR_BAD_ARG, "run: an attention's group has no block table");
    ++n_attention;
  }
  if (n_attention != n_attn) return fail(p, ERR_BAD_ARG, "run: one number of parts per attention operation");

  char* a = p->arena;
  const Buffers& b = p->buf;
  float* hres = (float*)(a + b.h);
  void* x = a + b.x;
  int rc = ((fn_embed)p->fns[FN_EMBED])(p->table, p->table_dtype, s.token_ids, hres, s.N, p->H, p->V, s.stream);
  if (rc) return fail(p, rc, "embed");
  Value pending;                         // nothing to add yet
  int attn_index = 0;
  for (const Op& op : p->ops) {
    if (op.kind == OP_NORM) {
      rc = add_norm(p, s, op, hres, pending, x, nullptr, s.N);
      pending = Value();
    } else if (op.kind == OP_ATTENTION) {
      rc = attention(p, s, op, attn_index++, a, x, &pending);
    } else if (op.kind == OP_SWIGLU_FF) {
      rc = feed_forward(p, s, op, a, x, &pending);
    } else {
      rc = fail(p, ERR_PROGRAM, "unknown operation");
    }
    if (rc) return rc;
  }
  if (s.R == 0) return 0;
  if (!logits) return fail(p, ERR_BAD_ARG, "run: logits");
  rc = add_norm(p, s, p->final_norm, hres, pending, x, s.logit_rows, s.R);
  if (rc) return rc;
  Value out;
  return linear(p, s, x, s.R, p->head, DT_F32, EPI_NONE, false, logits, a + b.head_ws, &out);
}

}  // extern "C"
