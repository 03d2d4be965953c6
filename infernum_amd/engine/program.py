"""The model's forward pass of a step as a native program (``csrc/step_program.cpp``).

A model whose parts can all describe themselves as operations of the native program (the built-in embedding,
RMSNorm, attention, SwiGLU feed-forward, linear head, in the pre-norm arrangement) runs a step with one call
into the host library, which makes the kernel launches itself, instead of one Python call per launch.  The
launches, their order and their arguments are those of the parts' own ``forward`` (the same bits; tests
compare the two).  A model with a part that has no native description runs through ``DecoderModel.forward``
as before: ``build`` returns None for it.  (The reference's executors walk their graph of operations natively
as well, infernum-cuda/src/inner/cuda_graph_engine.rs.)
"""
from __future__ import annotations

import ctypes
import importlib
from typing import Any, Dict, List, Optional, Sequence

import torch

from ..cache import native
from ..kernels import api as K
from ..parts.base import CacheView, StepContext

# the modules, not the functions of the same names that the package exports
attention_part = importlib.import_module("infernum_amd.parts.attention")
linear_part = importlib.import_module("infernum_amd.parts.linear")

_FUNCTIONS = ("ia_embed", "ia_add_rmsnorm", "ia_rope_kv_append", "ia_swiglu", "ia_gemm_generic", "ia_gemm_mfma",
              "ia_gemm_skinny", "ia_gemm_skinny_splits")          # of the core library, in the program's order
_GEMMS = {"library": 0, "mfma": 1}


class ProgramError(K.KernelError):
    pass


def _fn(lib: ctypes.CDLL, name: str) -> ctypes.c_void_p:
    return ctypes.cast(getattr(lib, name), ctypes.c_void_p)


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


class StepProgram:
    """Built by the parts (``Part.native``), then run once per step."""

    def __init__(self, model, max_tokens: int):
        rt = model.rt
        self.rt = rt
        self.model = model
        self._lib = native.lib()
        self._keep: List[Any] = []                   # tensors whose addresses the program holds
        self.attentions: List[Dict[str, int]] = []   # per attention operation: what its per-step numbers depend on
        core = K.load_library("core")
        blaslt = K.load_library("blaslt") if rt.dtype == torch.bfloat16 and rt.kernels != "generic" else None
        emb = model.embedding
        table = getattr(emb, "table", None)
        if table is None:
            raise ProgramError("the embedding has no table")
        settings = (ctypes.c_int * 10)(
            K.DTYPE_CODE[rt.dtype], model.spec.hidden_size, model.spec.vocab_size, int(rt.kernels == "generic"),
            _GEMMS[linear_part.prefill_gemm()], linear_part.SKINNY_ROWS_ANY_WIDTH, linear_part.SKINNY_WIDE,
            0, attention_part.ROTATE_IN_ATTENTION_UP_TO, K.DTYPE_CODE[table.dtype])
        self._settings = settings
        self._h = ctypes.c_void_p(self._lib.ia_program_create(settings, 10, _ptr(table)))
        if not self._h:
            raise ProgramError("the native program could not be created")
        self._keep.append(table)
        fns = [_fn(core, n) for n in _FUNCTIONS]
        fns.append(_fn(blaslt, "ia_gemm_lt") if blaslt is not None else _fn(core, "ia_gemm_generic"))   # never called then
        fns.append(_fn(core, "ia_attention_generic"))
        self._check(self._lib.ia_program_set_functions(self._h, (ctypes.c_void_p * len(fns))(*fns), len(fns)))
        self.max_tokens = int(max_tokens)
        self._arena: Optional[torch.Tensor] = None
        self._arena_bytes = 0
        self._finished = False

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.ia_program_destroy(self._h)
            self._h = None

    def _check(self, rc: int) -> None:
        if rc != 0:
            raise ProgramError(self._lib.ia_program_error(self._h).decode())

    # ---- what the parts add ------------------------------------------------------------
    def add_norm(self, weight: torch.Tensor, eps: float, final: bool = False) -> None:
        self._keep.append(weight)
        self._check(self._lib.ia_program_add_norm(self._h, _ptr(weight), K.DTYPE_CODE[weight.dtype],
                                                  ctypes.c_float(eps), int(final)))

    def add_attention(self, part, view: CacheView) -> None:
        """``part``: a parts.attention.Attention; ``view``: what its run sees of the cache."""
        k, v = view.k_pages, view.v_pages
        pos = part.position
        inv_freq = pos.inv_freq
        lib = K._attn(part.d) if part.use_mfma else None
        ints = (ctypes.c_int * 11)(part.nh, part.nkv, part.d, part.window, pos.rotary_dim if inv_freq is not None else 0,
                                   int(inv_freq is not None and inv_freq.dtype == torch.float64), view.group,
                                   int(view.writable), int(part.use_mfma), k.shape[2], k.shape[0])
        ptrs = [_ptr(part.w_qkv), _ptr(part.w_o), _ptr(inv_freq), _ptr(k), _ptr(v)]
        for name in ("ia_attn_decode", "ia_attn_decode_fused", "ia_attn_prefill"):
            ptrs.append(_fn(lib, name) if lib is not None else ctypes.c_void_p(0))
        self._keep += [part.w_qkv, part.w_o, inv_freq, k, v]
        masks = (ctypes.c_int * 3)(self._route(part.w_qkv, None, True),
                                   self._route(part.w_qkv[: part.nh * part.d], None, True),
                                   self._route(part.w_o, None, True))
        self._check(self._lib.ia_program_add_attention(self._h, ints, 11, ctypes.c_float(part.scale),
                                                       (ctypes.c_void_p * 8)(*ptrs), 8, masks))
        self.attentions.append({"nh": part.nh, "nkv": part.nkv, "d": part.d, "window": part.window,
                                "mfma": int(part.use_mfma and k.shape[2] % 4 == 0),
                                "rotates": int(part.rotate_in_attention)})

    @staticmethod
    def _route(w: torch.Tensor, epilogue: Optional[str], keep_split: bool) -> int:
        """The measured choice between the two products for this weight and use (parts/linear.py)."""
        return linear_part.library_rows(w.shape[0], w.shape[1], epilogue, keep_split)

    def add_swiglu(self, w_gate_up: torch.Tensor, w_down: torch.Tensor) -> None:
        self._keep += [w_gate_up, w_down]
        self._check(self._lib.ia_program_add_swiglu(self._h, _ptr(w_gate_up), _ptr(w_down), w_down.shape[1],
                                                    self._route(w_gate_up, "swiglu", False),
                                                    self._route(w_down, None, True)))

    def set_head(self, weight: torch.Tensor) -> None:
        self._keep.append(weight)
        self._check(self._lib.ia_program_set_head(self._h, _ptr(weight)))

    def finish(self) -> None:
        rotates = {a["rotates"] for a in self.attentions}
        if len(rotates) > 1:
            raise ProgramError("attention parts of one program rotate in different places")
        # where steps of single tokens rotate is a setting of the whole program: written now that the parts are known
        self._settings[7] = rotates.pop() if rotates else 0
        self._lib.ia_program_set_rotation(self._h, int(self._settings[7]))
        need = int(self._lib.ia_program_finish(self._h, self.max_tokens))
        if need == 0:
            self._check(10006)
        self._arena_bytes = need
        self._finished = True

    # ---- one step ------------------------------------------------------------------------
    def run(self, ctx: StepContext) -> torch.Tensor:
        """The launches of ``DecoderModel.forward`` for this step; fp32 logits [R, V] at ctx.logit_rows."""
        dev = self.rt.device
        if self._arena is None:             # at the first step: models that are built and never stepped need none
            self._arena = torch.empty(self._arena_bytes, dtype=torch.uint8, device=dev)
            ws = None
            if self.rt.dtype == torch.bfloat16 and self.rt.kernels != "generic":
                ws = K.library_workspace(dev)
            self._check(self._lib.ia_program_set_arena(self._h, _ptr(self._arena), ctypes.c_size_t(self._arena_bytes),
                                                       _ptr(ws), ctypes.c_size_t(ws.numel() if ws is not None else 0)))
        R = int(ctx.logit_rows.numel())
        V = self.model.spec.vocab_size
        logits = torch.empty((R, V), dtype=torch.float32, device=dev)
        G = len(ctx.block_tables)
        nd = ctx.num_decode
        tiles, num_tiles = (None, 0)
        n_attn = len(self.attentions)
        splits = (ctypes.c_int * max(n_attn, 1))()
        hpw = (ctypes.c_int * max(n_attn, 1))()
        memo: Dict[tuple, tuple] = {}
        for i, a in enumerate(self.attentions):
            key = (a["nh"], a["nkv"], a["d"], a["window"], a["mfma"])
            got = memo.get(key)
            if got is None:
                s, w = 1, 0
                if a["mfma"]:
                    if nd > 0:
                        s = K.decode_splits(nd, a["nh"], a["nkv"], ctx.max_total_len)
                    if ctx.num_seqs > nd:
                        w = K.prefill_launch_shape(a["nh"], a["nkv"], a["d"], ctx.q_lens[nd:], ctx.ctx_lens[nd:],
                                                   a["window"], dev)
                        if tiles is None:
                            tiles, num_tiles = ctx.row_tiles(K.PREFILL_TILE_ROWS)
                got = memo[key] = (s, w)
            splits[i], hpw[i] = got
        ints = (ctypes.c_int * 7)(ctx.num_tokens, ctx.num_seqs, nd, R, ctx.max_total_len, num_tiles, G)
        ptrs = [ctx.token_ids, ctx.positions, ctx.token_seq, ctx.seq_starts, ctx.seq_ctx, ctx.logit_rows, tiles]
        cols = (ctypes.c_int * max(G, 1))()
        for g in range(G):
            ptrs += [ctx.block_tables[g], ctx.slots[g]]
            cols[g] = ctx.block_tables[g].shape[1]
        arr = (ctypes.c_void_p * len(ptrs))(*[t.data_ptr() if t is not None else 0 for t in ptrs])
        self._check(self._lib.ia_program_run(self._h, ints, 7, arr, len(ptrs), cols, splits, hpw, n_attn, _ptr(logits),
                                             K._stream()))
        return logits


def build(model, views: Sequence[CacheView], max_tokens: int) -> Optional[StepProgram]:
    """The model's native program, or None when a part has no native description, the many-row products are
    set to go through ``torch.mm``, or the parts' kernel calls are being timed one by one."""
    if linear_part.prefill_gemm() not in _GEMMS or K.profiling() or model.rt.device.type != "cuda":
        return None
    if model.final_norm is None or len(views) != len(model.spec.schedule):
        return None
    program = StepProgram(model, max_tokens)
    if not model.embedding.native(program, None):
        return None
    for e, view in zip(model.spec.schedule, views):
        if not model.blocks[e.layer].native(program, view):
            return None
    if not model.final_norm.native(program, None, final=True) or not model.head.native(program, None):
        return None
    program.finish()
    return program
