// A model's forward pass of one step as a program of launches that is data: the interpreter.
//
// An operation is a launcher (a function pointer with the one calling convention of op_call.h), its arguments and
// a condition.  An argument is a constant (an address of a weight, of a page pool or of an intermediate, a size, a
// float), a number of the step (tokens, requests, single-token requests, ... as the caller lists them) put through
// a * x + b, one of the step's arrays (plus a byte offset), or the stream.  The condition says for which steps the
// operation runs: a disjunction of conjunctions of terms "low <= number <= high" and "the block of sixteen that the
// number lies in is one of these" (which product a matrix goes to depends on its rows in such blocks).  An
// operation may be marked as the one to run when the operation before it found its size unsupported.
//
// The parts of a model write the program (each part the operations of its own launches: engine/program.py and the
// parts' `native`); this file knows no part, no kernel and no architecture, makes no GPU call of its own and
// allocates nothing per step.  (The reference walks its graph of operations natively as well:
// infernum-cuda/src/inner/cuda_graph_engine.rs.)
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

namespace {

enum { ERR_BAD_ARG = 10001, ERR_UNSUPPORTED = 10002, ERR_PROGRAM = 10006 };
enum { ARG_CONST = 0, ARG_VAR = 1, ARG_PTR = 2, ARG_STREAM = 3 };
enum { TERM_RANGE = 0, TERM_BLOCKS = 1 };
enum { FLAG_IF_UNSUPPORTED = 1 };
const int MAX_ARGS = 40;

typedef int (*launcher_t)(const uint64_t* slots, int n);

struct Arg {
  int kind = ARG_CONST, index = 0;
  int64_t mul = 1, add = 0;          // CONST: add holds the slot's bits
};

struct Term {
  int kind = TERM_RANGE, var = 0, group = 0;
  int64_t lo = 0, hi = 0;            // BLOCKS: lo is the mask: bit min((x - 1) / 16, 8) for x >= 1
};

struct Op {
  launcher_t fn = nullptr;
  std::string name;
  std::vector<Arg> args;
  std::vector<Term> terms;           // sorted by group
  int flags = 0;
};

struct Program {
  std::vector<Op> ops;
  int n_vars = -1, n_ptrs = -1;      // what a step must bring; set by ia_program_finish
  long long launches = 0;            // operations run by the last step
  std::string error;
};

int fail(Program* p, int code, const std::string& what) {
  p->error = what + ": error " + std::to_string(code);
  return code;
}

bool term_holds(const Term& t, const int64_t* vars) {
  const int64_t x = vars[t.var];
  if (t.kind == TERM_RANGE) return t.lo <= x && x <= t.hi;
  if (x < 1) return false;
  const int64_t block = (x - 1) / 16 < 8 ? (x - 1) / 16 : 8;
  return (t.lo >> block) & 1;
}

bool runs(const Op& op, const int64_t* vars) {
  if (op.terms.empty()) return true;
  size_t i = 0;
  while (i < op.terms.size()) {
    const int group = op.terms[i].group;
    bool all = true;
    for (; i < op.terms.size() && op.terms[i].group == group; ++i) all = all && term_holds(op.terms[i], vars);
    if (all) return true;
  }
  return false;
}

}  // namespace

extern "C" {

void* ia_program_create() { return new Program(); }

void ia_program_destroy(void* h) { delete static_cast<Program*>(h); }

const char* ia_program_error(void* h) { return static_cast<Program*>(h)->error.c_str(); }

int ia_program_num_ops(void* h) { return (int)static_cast<Program*>(h)->ops.size(); }

long long ia_program_last_launches(void* h) { return static_cast<Program*>(h)->launches; }

// args: 4 numbers each [kind, index, mul, add]; terms: 5 numbers each [kind, var, lo, hi, group], groups rising.
int ia_program_add_op(void* h, void* fn, const char* name, const int64_t* args, int n_args, const int64_t* terms,
                      int n_terms, int flags) {
  Program* p = static_cast<Program*>(h);
  if (p->n_vars >= 0) return fail(p, ERR_PROGRAM, "the program is finished");
  const std::string nm = name ? name : "?";
  if (!fn || n_args < 0 || n_args > MAX_ARGS || n_terms < 0 || (n_args && !args) || (n_terms && !terms))
    return fail(p, ERR_BAD_ARG, "operation " + nm);
  Op op;
  op.fn = reinterpret_cast<launcher_t>(fn);
  op.name = nm;
  op.flags = flags;
  for (int i = 0; i < n_args; ++i) {
    Arg a;
    a.kind = (int)args[4 * i];
    a.index = (int)args[4 * i + 1];
    a.mul = args[4 * i + 2];
    a.add = args[4 * i + 3];
    if (a.kind < ARG_CONST || a.kind > ARG_STREAM || a.index < 0) return fail(p, ERR_BAD_ARG, "operation " + nm + ": argument");
    op.args.push_back(a);
  }
  int last_group = -1;
  for (int i = 0; i < n_terms; ++i) {
    Term t;
    t.kind = (int)terms[5 * i];
    t.var = (int)terms[5 * i + 1];
    t.lo = terms[5 * i + 2];
    t.hi = terms[5 * i + 3];
    t.group = (int)terms[5 * i + 4];
    if ((t.kind != TERM_RANGE && t.kind != TERM_BLOCKS) || t.var < 0 || t.group < last_group)
      return fail(p, ERR_BAD_ARG, "operation " + nm + ": condition");
    last_group = t.group;
    op.terms.push_back(t);
  }
  if ((flags & FLAG_IF_UNSUPPORTED) && p->ops.empty()) return fail(p, ERR_PROGRAM, "operation " + nm + " stands in for none");
  p->ops.push_back(op);
  return 0;
}

// The program is complete; a step brings n_vars numbers and n_ptrs arrays.
int ia_program_finish(void* h, int n_vars, int n_ptrs) {
  Program* p = static_cast<Program*>(h);
  if (n_vars < 0 || n_ptrs < 0) return fail(p, ERR_BAD_ARG, "finish");
  for (const Op& op : p->ops) {
    for (const Arg& a : op.args)
      if ((a.kind == ARG_VAR && a.index >= n_vars) || (a.kind == ARG_PTR && a.index >= n_ptrs))
        return fail(p, ERR_PROGRAM, "operation " + op.name + " names a number or an array that no step brings");
    for (const Term& t : op.terms)
      if (t.var >= n_vars) return fail(p, ERR_PROGRAM, "operation " + op.name + ": its condition names a number that no step brings");
  }
  p->n_vars = n_vars;
  p->n_ptrs = n_ptrs;
  return 0;
}

// One step: its numbers, its arrays, the stream.  Operations run in the program's order.
int ia_program_run(void* h, const int64_t* vars, int n_vars, void* const* ptrs, int n_ptrs, void* stream) {
  Program* p = static_cast<Program*>(h);
  if (p->n_vars < 0) return fail(p, ERR_PROGRAM, "the program is not finished");
  if (n_vars != p->n_vars || n_ptrs != p->n_ptrs || (n_vars && !vars) || (n_ptrs && !ptrs)) return fail(p, ERR_BAD_ARG, "run");
  uint64_t slots[MAX_ARGS];
  p->launches = 0;
  bool unsupported = false;          // the operation before this one ran and found its size unsupported
  for (size_t i = 0; i < p->ops.size(); ++i) {
    const Op& op = p->ops[i];
    if (op.flags & FLAG_IF_UNSUPPORTED) {
      if (!unsupported) continue;
    } else if (unsupported) {
      return fail(p, ERR_UNSUPPORTED, "operation #" + std::to_string(i - 1) + " (" + p->ops[i - 1].name + ")");
    } else if (!runs(op, vars)) {
      continue;
    }
    unsupported = false;
    const int n = (int)op.args.size();
    for (int k = 0; k < n; ++k) {
      const Arg& a = op.args[(size_t)k];
      switch (a.kind) {
        case ARG_CONST: slots[k] = (uint64_t)a.add; break;
        case ARG_VAR: slots[k] = (uint64_t)(a.mul * vars[a.index] + a.add); break;
        case ARG_PTR: {
          const char* base = static_cast<const char*>(ptrs[a.index]);
          slots[k] = base ? (uint64_t)(uintptr_t)(base + a.add) : 0;
          break;
        }
        default: slots[k] = (uint64_t)(uintptr_t)stream; break;
      }
    }
    const int rc = op.fn(slots, n);
    ++p->launches;
    if (rc == ERR_UNSUPPORTED && i + 1 < p->ops.size() && (p->ops[i + 1].flags & FLAG_IF_UNSUPPORTED)) {
      unsupported = true;
      continue;
    }
    if (rc) return fail(p, rc, "operation #" + std::to_string(i) + " (" + op.name + ")");
  }
  return 0;
}

}  // extern "C"
