"""The model's forward pass of a step as a program of launches (interpreted by ``csrc/step_program.cpp``).

Every part writes the operations of its own launches into a :class:`StepProgram` (``Part.native``): a launcher
of a kernel library, its arguments, and the steps it runs for.  An argument is a constant (a weight, a page
pool, an intermediate of the program's arena, a size), a number of the step (:class:`Var`: tokens, requests,
single-token requests, wanted rows, ...; ``a * x + b`` of one), one of the step's arrays (:class:`StepPtr`) or
the stream.  A condition (:class:`Guard`) is made of "low <= number <= high" and "the number's block of sixteen
is one of these", joined by ``&``, ``|`` and ``~``.  What one part leaves for the next (the pending delta of the
residual stream: a tensor, or the partial sums of a split matrix product, depending on the step's rows) is a
:class:`Value`: alternatives with a condition each; the consumer writes one operation per alternative.

The interpreter knows no part and no kernel.  A part without launchers of its own is an operation too: a call
back into its ``forward`` (``StepProgram.python``), so a model with parts that the framework has never seen still
runs its step as one program, the stock parts' launches made natively around it.  Intermediates live in one
arena, planned here: buffers are named, and equal names share memory (a layer's scratch is dead when the next
layer of its kind runs).  (The reference's executors walk a graph of operations that its blocks register:
infernum-macros/src/lib.rs:32-106, infernum-cuda/src/inner/cuda_graph_engine.rs.)
"""
from __future__ import annotations

import ctypes
import itertools
import struct
from typing import Any, Callable, Dict, Hashable, List, Optional, Sequence, Tuple, Union

import torch

from ..cache import native
from ..kernels import api as K
from ..parts.base import CacheView, StepContext

_INF = 1 << 62
_ARG_CONST, _ARG_VAR, _ARG_PTR, _ARG_STREAM = 0, 1, 2, 3
_TERM_RANGE, _TERM_BLOCKS = 0, 1
ALL_BLOCKS = 0x1FF          # bits 0..7: 1-16, 17-32, ... 113-128 rows; bit 8: more than 128
PYTHON_FAILED = 10007
_GUARD, _GUARD_BYTE = 256, 0xA5


class ProgramError(K.KernelError):
    pass


class Var:
    """A number of the step (``mul * x + add`` of it as an argument)."""

    __slots__ = ("index", "name", "mul", "add")

    def __init__(self, index: int, name: str, mul: int = 1, add: int = 0):
        self.index, self.name, self.mul, self.add = index, name, int(mul), int(add)

    def __mul__(self, k: int) -> "Var":
        return Var(self.index, self.name, self.mul * int(k), self.add * int(k))

    __rmul__ = __mul__

    def __add__(self, k: int) -> "Var":
        return Var(self.index, self.name, self.mul, self.add + int(k))

    def __repr__(self) -> str:
        return f"Var({self.name})" if (self.mul, self.add) == (1, 0) else f"Var({self.mul}*{self.name}+{self.add})"


class StepPtr:
    """One of the step's arrays (plus a byte offset)."""

    __slots__ = ("index", "name", "offset")

    def __init__(self, index: int, name: str, offset: int = 0):
        self.index, self.name, self.offset = index, name, int(offset)


class _Stream:
    def __repr__(self) -> str:
        return "STREAM"


STREAM = _Stream()


class Buffer:
    """A named intermediate in the program's arena; its address is known once the program is finished."""

    __slots__ = ("key", "nbytes", "offset", "_program")

    def __init__(self, key: str, program: "StepProgram"):
        self.key, self.nbytes, self.offset, self._program = key, 0, -1, program

    @property
    def ptr(self) -> int:
        if self.offset < 0:
            raise ProgramError(f"buffer {self.key!r} has no address before the program is finished")
        return self._program._arena.data_ptr() + self.offset

    def view(self, dtype: torch.dtype, *shape: int) -> torch.Tensor:
        """The first prod(shape) elements as a tensor (for operations written in Python)."""
        n = 1
        for s in shape:
            n *= int(s)
        esz = torch.empty((), dtype=dtype).element_size()
        if n * esz > self.nbytes:
            raise ProgramError(f"buffer {self.key!r} holds {self.nbytes} bytes, {n * esz} asked for")
        return self._program._arena[self.offset:self.offset + n * esz].view(dtype).view(*shape)


def _term_not(t: Tuple) -> List[Tuple]:
    kind, var, lo, hi = t
    if kind == _TERM_RANGE:
        out = []
        if lo > -_INF:
            out.append((_TERM_RANGE, var, -_INF, lo - 1))
        if hi < _INF:
            out.append((_TERM_RANGE, var, hi + 1, _INF))
        return out
    out = [(_TERM_RANGE, var, -_INF, 0)]
    if ~lo & ALL_BLOCKS:
        out.append((_TERM_BLOCKS, var, ~lo & ALL_BLOCKS, 0))
    return out


def _tidy(conj: Sequence[Tuple]) -> Optional[Tuple[Tuple, ...]]:
    """One conjunction with the terms of a number merged; None when nothing can satisfy it."""
    ranges: Dict[int, List[int]] = {}
    blocks: Dict[int, int] = {}
    for kind, var, lo, hi in conj:
        if kind == _TERM_RANGE:
            r = ranges.setdefault(var, [-_INF, _INF])
            r[0], r[1] = max(r[0], lo), min(r[1], hi)
        else:
            blocks[var] = blocks.get(var, ALL_BLOCKS) & lo
    out = []
    for var, (lo, hi) in sorted(ranges.items()):
        if lo > hi:
            return None
        if var in blocks:                                   # a range can rule blocks out
            keep = 0
            for b in range(9):
                first, last = 16 * b + 1, (16 * b + 16 if b < 8 else _INF)
                if last >= lo and first <= hi:
                    keep |= 1 << b
            blocks[var] &= keep
        if (lo, hi) != (-_INF, _INF):
            out.append((_TERM_RANGE, var, lo, hi))
    for var, mask in sorted(blocks.items()):
        if mask == 0:
            return None
        out.append((_TERM_BLOCKS, var, mask, 0))
    return tuple(out)


class Guard:
    """For which steps an operation runs: a disjunction of conjunctions of terms over the step's numbers."""

    __slots__ = ("alts",)

    def __init__(self, alts: Sequence[Sequence[Tuple]]):
        tidy = []
        for c in alts:
            t = _tidy(c)
            if t is not None and t not in tidy:
                tidy.append(t)
        if () in tidy:
            tidy = [()]
        self.alts: Tuple[Tuple[Tuple, ...], ...] = tuple(tidy)

    @staticmethod
    def between(var: Var, lo: Optional[int] = None, hi: Optional[int] = None) -> "Guard":
        _plain(var)
        return Guard([[(_TERM_RANGE, var.index, -_INF if lo is None else int(lo), _INF if hi is None else int(hi))]])

    @staticmethod
    def blocks(var: Var, mask: int) -> "Guard":
        """The number is at least 1 and lies in one of the blocks of sixteen whose bit is set (see ALL_BLOCKS)."""
        _plain(var)
        return Guard([[(_TERM_BLOCKS, var.index, int(mask) & ALL_BLOCKS, 0)]])

    def __and__(self, other: "Guard") -> "Guard":
        return Guard([a + b for a in self.alts for b in other.alts])

    def __or__(self, other: "Guard") -> "Guard":
        return Guard(self.alts + other.alts)

    def __invert__(self) -> "Guard":
        if not self.alts:
            return ALWAYS
        choices = [list(itertools.chain.from_iterable(_term_not(t) for t in conj)) for conj in self.alts]
        return Guard([list(pick) for pick in itertools.product(*choices)])

    @property
    def never(self) -> bool:
        return not self.alts

    def holds(self, numbers: Sequence[int]) -> bool:
        def term(t):
            kind, var, lo, hi = t
            x = numbers[var]
            if kind == _TERM_RANGE:
                return lo <= x <= hi
            return x >= 1 and bool((lo >> min((x - 1) // 16, 8)) & 1)
        return any(all(term(t) for t in conj) for conj in self.alts)

    def __repr__(self) -> str:
        return f"Guard({self.alts})"


def _plain(var: Var) -> None:
    if (var.mul, var.add) != (1, 0):
        raise ProgramError("a condition is about a number of the step itself, not about a multiple of it")


ALWAYS = Guard([[]])
NEVER = Guard([])


class Alt:
    """One form of a :class:`Value`: where it lies, how (``splits`` 0: a tensor [rows, cols] of ``dtype``;
    otherwise fp32 partial sums [splits, rows, cols]), and for which steps."""

    __slots__ = ("when", "where", "splits", "dtype")

    def __init__(self, when: Guard, where: Any, splits: int, dtype: torch.dtype):
        self.when, self.where, self.splits, self.dtype = when, where, int(splits), dtype


class Value:
    """A matrix [rows, cols] that an operation left: one alternative per form it can have."""

    def __init__(self, cols: int, alts: Sequence[Alt]):
        self.cols = int(cols)
        merged: List[Alt] = []
        for a in alts:
            if a.when.never:
                continue
            for m in merged:
                if m.where is a.where and (m.splits, m.dtype) == (a.splits, a.dtype):
                    m.when = m.when | a.when
                    break
            else:
                merged.append(Alt(a.when, a.where, a.splits, a.dtype))
        self.alts = merged

    def tensor(self) -> Any:
        """Where the value lies when it has one form only, a tensor (what a product with an activation leaves)."""
        if len(self.alts) != 1 or self.alts[0].splits:
            raise ProgramError("the value is not one tensor for every step")
        return self.alts[0].where


_CALLBACK = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.POINTER(ctypes.c_uint64), ctypes.c_int)


class StepProgram:
    """Written by the parts (``Part.native``), finished once, then run once per step."""

    def __init__(self, rt, hidden_size: int, logits_cols: int, num_groups: int, max_tokens: int):
        self.rt = rt
        self.T = int(max_tokens)
        self.hidden_size, self.logits_cols = int(hidden_size), int(logits_cols)
        self.act_code = K.DTYPE_CODE[rt.dtype]
        self.act_bytes = 4 if rt.dtype == torch.float32 else 2
        self._lib = native.lib()
        self._h = ctypes.c_void_p(self._lib.ia_program_create())
        self._keep: List[Any] = []
        self._ops: List[tuple] = []
        self._buffers: Dict[str, Buffer] = {}
        self._arena: Optional[torch.Tensor] = None
        self._finished = False
        self._ctx: Optional[StepContext] = None
        self._logits: Optional[torch.Tensor] = None
        self._numbers: List[int] = []
        self._python_error: Optional[BaseException] = None
        # the step's numbers
        self._vars: List[Var] = []
        self._var_fns: List[Callable[[StepContext], int]] = []
        self._scalars: Dict[Hashable, Var] = {}
        self.N = self._var("tokens", lambda c: c.num_tokens)
        self.B = self._var("requests", lambda c: c.num_seqs)
        self.ND = self._var("single-token requests", lambda c: c.num_decode)
        self.R = self._var("wanted rows", lambda c: int(c.logit_rows.numel()))
        self.MAX_LEN = self._var("longest request", lambda c: c.max_total_len)
        self.NP = self._var("requests with a portion", lambda c: c.num_seqs - c.num_decode)
        self.NPT = self._var("tokens of portions", lambda c: c.num_tokens - c.num_decode)
        self._bt_cols = [self._var(f"block-table width {g}", (lambda c, g=g: int(c.block_tables[g].shape[1])))
                         for g in range(num_groups)]
        # the step's arrays
        self._ptrs: List[StepPtr] = []
        self._ptr_fns: List[Callable[[StepContext], Optional[torch.Tensor]]] = []
        self.token_ids = self._ptr("token_ids", lambda c: c.token_ids)
        self.positions = self._ptr("positions", lambda c: c.positions)
        self.token_seq = self._ptr("token_seq", lambda c: c.token_seq)
        self.seq_starts = self._ptr("seq_starts", lambda c: c.seq_starts)
        self.seq_ctx = self._ptr("seq_ctx", lambda c: c.seq_ctx)
        self.state_slots = self._ptr("state_slots", lambda c: c.state_slots)
        self.logit_rows = self._ptr("logit_rows", lambda c: c.logit_rows)
        self.logits = self._ptr("logits", lambda c: self._logits)
        self._block_tables = [self._ptr(f"block_table {g}", (lambda c, g=g: c.block_tables[g])) for g in range(num_groups)]
        self._slots = [self._ptr(f"slots {g}", (lambda c, g=g: c.slots[g])) for g in range(num_groups)]
        self._tiles: Dict[int, Tuple[StepPtr, Var]] = {}
        # the registers that the parts hand on: the fp32 residual stream, the normalised activations, and the
        # delta that the next norm adds to the residual stream
        self.h = self.buffer("h", self.T * self.hidden_size * 4)
        self.x = self.buffer("x", self.T * self.hidden_size * self.act_bytes)
        self.pending: Optional[Value] = None

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.ia_program_destroy(self._h)
            self._h = None

    # ---- numbers and arrays of a step -----------------------------------------------------
    def _var(self, name: str, fn: Callable[[StepContext], int]) -> Var:
        v = Var(len(self._vars), name)
        self._vars.append(v)
        self._var_fns.append(fn)
        return v

    def _ptr(self, name: str, fn: Callable[[StepContext], Optional[torch.Tensor]]) -> StepPtr:
        p = StepPtr(len(self._ptrs), name)
        self._ptrs.append(p)
        self._ptr_fns.append(fn)
        return p

    def bt_cols(self, group: int) -> Var:
        return self._bt_cols[group]

    def block_table(self, group: int) -> StepPtr:
        return self._block_tables[group]

    def slots(self, group: int) -> StepPtr:
        return self._slots[group]

    def scalar(self, key: Hashable, fn: Callable[[StepContext], int]) -> Var:
        """A number that a part works out on the host for every step (``fn(ctx)``); parts that give the same
        key share it, so it is worked out once a step."""
        self._not_finished()
        v = self._scalars.get(key)
        if v is None:
            v = self._scalars[key] = self._var(str(key), fn)
        return v

    def row_tiles(self, rows: int) -> Tuple[StepPtr, Var]:
        """The step's portions of prompts cut into tiles of ``rows`` rows (``StepContext.row_tiles``): the array
        and the number of tiles; made only for steps that have portions."""
        self._not_finished()
        hit = self._tiles.get(rows)
        if hit is None:
            made: Dict[int, Tuple[Optional[torch.Tensor], int]] = {}

            def tiles(c: StepContext, rows=rows):
                if made.get("step") is not c:
                    made["step"], made["tiles"] = c, (c.row_tiles(rows) if c.num_seqs > c.num_decode else (None, 0))
                return made["tiles"]
            hit = self._tiles[rows] = (self._ptr(f"tiles of {rows}", lambda c: tiles(c)[0]),
                                       self._var(f"tiles of {rows}", lambda c: tiles(c)[1]))
        return hit

    # ---- what the parts write ---------------------------------------------------------------
    def _not_finished(self) -> None:
        if self._finished:
            raise ProgramError("the program is finished")

    def keep(self, *objects: Any) -> None:
        """Tensors whose addresses the program holds stay alive with it."""
        self._keep.extend(o for o in objects if o is not None)

    def buffer(self, key: str, nbytes: int) -> Buffer:
        """An intermediate of at least ``nbytes``; the same key gives the same memory (the largest size asked)."""
        self._not_finished()
        b = self._buffers.get(key)
        if b is None:
            b = self._buffers[key] = Buffer(key, self)
        b.nbytes = max(b.nbytes, int(nbytes))
        return b

    def op(self, library: Union[str, ctypes.CDLL], launcher: str, args: Sequence[Any], when: Guard = ALWAYS,
           if_unsupported: bool = False) -> None:
        """``launcher`` (``ia_...`` of a kernel library, by the library's name or handle) with ``args`` in the
        launcher's own order: int, float, None (a null pointer), tensor, Buffer, Var, StepPtr or STREAM.
        ``if_unsupported``: runs in place of the operation before it when that found its size unsupported."""
        self._not_finished()
        if when.never and not if_unsupported:
            return
        lib = K.load_library(library) if isinstance(library, str) else library
        try:
            fn = ctypes.cast(getattr(lib, "ia_op_" + launcher), ctypes.c_void_p)
        except AttributeError:
            raise ProgramError(f"the library has no operation for {launcher}") from None
        self._ops.append((fn, launcher, list(args), when, bool(if_unsupported)))

    def python(self, fn: Callable[[StepContext], None], name: str, when: Guard = ALWAYS) -> None:
        """An operation written in Python: ``fn(ctx)`` is called in the program's order (its torch calls and
        kernel calls go to the step's stream like everything else)."""
        self._not_finished()
        if when.never:
            return

        def call(_slots, _n, fn=fn):
            try:
                fn(self._ctx)
                return 0
            except BaseException as e:          # carried over the native frame, raised again by run()
                self._python_error = e
                return PYTHON_FAILED
        cb = _CALLBACK(call)
        self._keep.append(cb)
        self._ops.append((ctypes.cast(cb, ctypes.c_void_p), "python:" + name, [], when, False))

    # ---- values between Python operations and launches ----------------------------------------
    def read(self, value: Optional[Value], rows: int):
        """(Inside a Python operation.)  The form that ``value`` has in the running step: a tensor, a
        ``SplitSum``, or None."""
        if value is None:
            return None
        for a in value.alts:
            if a.when.holds(self._numbers):
                if a.splits:
                    return K.SplitSum(a.where.view(torch.float32, a.splits, rows, value.cols))
                return a.where.view(a.dtype, rows, value.cols)
        raise ProgramError("a value has no form for this step")

    def store(self, key: str, cols: int, dtype: Optional[torch.dtype] = None) -> Tuple[Buffer, Value]:
        """A buffer [max tokens, cols] for what a Python operation returns, and the Value that stands for it."""
        dtype = dtype or self.rt.dtype
        esz = torch.empty((), dtype=dtype).element_size()
        buf = self.buffer(key, self.T * int(cols) * esz)
        return buf, Value(cols, [Alt(ALWAYS, buf, 0, dtype)])

    # ---- finishing ---------------------------------------------------------------------------
    def finish(self) -> None:
        self._not_finished()
        # buffers one after the other, each followed by a guard of 256 bytes that holds a pattern: a launch that
        # writes past its buffer's end writes into the guard first (``check_guards``; tests look after their steps)
        at = 0
        for b in self._buffers.values():
            b.offset = at
            at += ((b.nbytes + 255) & ~255) + _GUARD
        self.arena_bytes = at
        self._arena = torch.empty(max(at, 256), dtype=torch.uint8, device=self.rt.device)
        for b in self._buffers.values():
            end = b.offset + ((b.nbytes + 255) & ~255)
            self._arena[end:end + _GUARD].fill_(_GUARD_BYTE)
        add = self._lib.ia_program_add_op
        for fn, name, args, when, if_unsupported in self._ops:
            flat: List[int] = []
            for a in args:
                flat += self._slot(a, name)
            terms: List[int] = []
            for group, conj in enumerate(when.alts):
                for kind, var, lo, hi in conj:
                    terms += [kind, var, lo, hi, group]
            if when.alts == ((),):
                terms = []
            A = (ctypes.c_int64 * max(len(flat), 1))(*flat)
            G = (ctypes.c_int64 * max(len(terms), 1))(*terms)
            self._check(add(self._h, fn, name.encode(), A, len(flat) // 4, G, len(terms) // 5, int(if_unsupported)))
        self._check(self._lib.ia_program_finish(self._h, len(self._vars), len(self._ptrs)))
        self.num_ops = len(self._ops)
        self.op_names = [op[1] for op in self._ops]              # the launchers, in the program's order
        self.num_python_ops = sum(1 for op in self._ops if op[1].startswith("python:"))   # parts called back into
        self._ops = []
        self._finished = True
        self._var_array = (ctypes.c_int64 * len(self._vars))()
        self._ptr_array = (ctypes.c_void_p * len(self._ptrs))()

    def _slot(self, a: Any, name: str) -> List[int]:
        if a is None:
            return [_ARG_CONST, 0, 1, 0]
        if a is STREAM:
            return [_ARG_STREAM, 0, 1, 0]
        if isinstance(a, bool):
            return [_ARG_CONST, 0, 1, int(a)]
        if isinstance(a, int):
            return [_ARG_CONST, 0, 1, a]
        if isinstance(a, float):
            return [_ARG_CONST, 0, 1, struct.unpack("<q", struct.pack("<d", a))[0]]
        if isinstance(a, Var):
            return [_ARG_VAR, a.index, a.mul, a.add]
        if isinstance(a, StepPtr):
            return [_ARG_PTR, a.index, 1, a.offset]
        if isinstance(a, Buffer):
            return [_ARG_CONST, 0, 1, a.ptr]
        if isinstance(a, torch.Tensor):
            if a.device != self._arena.device:
                raise ProgramError(f"{name}: an operand is not on the program's device")
            self._keep.append(a)
            return [_ARG_CONST, 0, 1, a.data_ptr()]
        raise ProgramError(f"{name}: an argument of type {type(a).__name__}")

    def _check(self, rc: int) -> None:
        if rc != 0:
            err, self._python_error = self._python_error, None
            if err is not None:
                raise err
            msg = self._lib.ia_program_error(self._h).decode()
            raise (K.KernelUnsupported if rc == 10002 else ProgramError)(msg)

    # ---- one step ------------------------------------------------------------------------------
    def run(self, ctx: StepContext) -> torch.Tensor:
        """The launches of the model's forward pass for this step; fp32 logits [R, V] at ctx.logit_rows."""
        if not self._finished:
            raise ProgramError("the program is not finished")
        if ctx.num_tokens > self.T:
            raise ProgramError(f"a step of {ctx.num_tokens} tokens; the program's intermediates hold {self.T}")
        R = int(ctx.logit_rows.numel())
        self._logits = torch.empty((R, self.logits_cols), dtype=torch.float32, device=self.rt.device)
        self._ctx = ctx
        try:
            numbers = self._numbers = [int(fn(ctx)) for fn in self._var_fns]
            va, pa = self._var_array, self._ptr_array
            for i, x in enumerate(numbers):
                va[i] = x
            for i, fn in enumerate(self._ptr_fns):
                t = fn(ctx)
                pa[i] = t.data_ptr() if t is not None else None
            self._check(self._lib.ia_program_run(self._h, va, len(numbers), pa, len(self._ptr_fns), K._stream()))
            return self._logits
        finally:
            self._ctx = None
            self._logits = None

    def step_logits(self) -> torch.Tensor:
        """(Inside a Python operation.)  The logits [wanted rows, vocabulary] that the running step returns."""
        return self._logits

    def check_guards(self) -> None:
        """Raises when something wrote past the end of one of the program's buffers."""
        for b in self._buffers.values():
            end = b.offset + ((b.nbytes + 255) & ~255)
            if not bool((self._arena[end:end + _GUARD] == _GUARD_BYTE).all()):
                raise ProgramError(f"something wrote past the end of buffer {b.key!r} ({b.nbytes} bytes)")

    def last_launches(self) -> int:
        return int(self._lib.ia_program_last_launches(self._h))


def build(model, views: Sequence[CacheView], num_groups: int, max_tokens: int) -> Optional[StepProgram]:
    """The model's program: every part writes its operations in the order of ``DecoderModel.forward``.  None
    while the parts' kernel calls are being timed one by one (a launch made natively has no call to time)."""
    if K.profiling() or model.rt.device.type != "cuda":
        return None
    spec = model.spec
    program = StepProgram(model.rt, spec.hidden_size, spec.vocab_size, num_groups, max_tokens)
    model.native(program, views)
    program.finish()
    return program
