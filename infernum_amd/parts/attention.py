"""Grouped-query attention over the paged cache.

q = x Wq^T, k = x Wk^T, v = x Wv^T without bias; heads are consecutive within a
row; q and k are rotated, then k and v are written to the pages at the tokens'
positions; query head h reads key/value head h // (nh / nkv); scores are
scale * <q, k_j> over the keys 0 .. p of the same request (the last ``window``
of them when a window is set), softmax with the maximum subtracted, output
sum_j w_j v_j; then the output projection.  (infernum-llama/src/graph_builder.rs:
456-483 and 819-867; infernum-cuda/kernels/paged_decode_attention.cu:319-430;
kernels/flash_prefill_attention_v2.cu:85-88 for the causal range with a window.)

The three projections are kept as one [ (nh + 2 nkv) d, H ] matrix (row-wise
concatenation, as the reference's optional fused weight,
infernum-cuda/src/inner/weights/generic_impl.rs:153-180).
"""
from __future__ import annotations

import math
from typing import Any, Dict, Mapping, Optional

import torch

from ..kernels import api as K
from .base import (CacheSpec, CacheView, Mixer, PartSpec, Runtime, StepContext, WeightSpec, make_part,
                   register_part)
from .linear import emit_linear, linear, prepare_weights


# Steps of up to this many single tokens rotate inside the attention kernel (8B shape: 1.5 % faster at 1 and 8
# tokens, 0.4 % at 64; at 128 the rotary kernel in front is 1 % faster: every workgroup of the attention starts
# with the rotation, and with many of them that costs more than the one launch it saves).
ROTATE_IN_ATTENTION_UP_TO = 64
DECODE_ROTATIONS = ("attention", "separate")
_decode_rotation = "attention"


def set_decode_rotation(name: str) -> str:
    """Where a step of single tokens rotates queries and keys and writes the pages, for attention parts made
    from now on: inside the attention kernel ("attention") or in the rotary kernel before it ("separate"; the
    same bits).  Returns the previous choice."""
    global _decode_rotation
    if name not in DECODE_ROTATIONS:
        raise ValueError(f"decode rotation {name!r}: one of {DECODE_ROTATIONS}")
    previous, _decode_rotation = _decode_rotation, name
    return previous


class Attention(Mixer):
    graph_safe = True
    def __init__(self, rt: Runtime, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: Optional[Mapping[str, Any]] = None, window: Optional[int] = None,
                 scale: Optional[float] = None, kernels: str = "auto", init_std: float = 0.02,
                 qk_transform: Optional[Mapping[str, Any]] = None):
        super().__init__(rt)
        if num_heads % num_kv_heads:
            raise ValueError(f"num_heads {num_heads} is not a multiple of num_kv_heads {num_kv_heads}")
        if head_dim > 256:
            raise ValueError(f"head size {head_dim} is above 256, the largest the attention kernels take")
        self.hidden_size, self.nh, self.nkv, self.d = int(hidden_size), int(num_heads), int(num_kv_heads), int(head_dim)
        self.window = int(window) if window else 0
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.d)
        if kernels not in ("auto", "generic"):
            raise ValueError("kernels must be 'auto' or 'generic'")
        self.kernels = kernels = "generic" if rt.kernels == "generic" else kernels
        self.init_std = init_std
        pos_spec = PartSpec(**position) if isinstance(position, Mapping) else (position or PartSpec("none"))
        self.position = make_part("position", pos_spec, rt)
        # an optional part of category "qk_transform" that works on the projected heads before the rotation;
        # with one, steps of single tokens take the separate kernels too (the fused one rotates what it projects)
        self.qk_transform = None
        if qk_transform is not None:
            spec = PartSpec(**qk_transform) if isinstance(qk_transform, Mapping) else qk_transform
            self.qk_transform = make_part("qk_transform", spec, rt)
        # recordable into a graph only when the parts inside are
        self.graph_safe = (getattr(self.position, "graph_safe", False)
                           and (self.qk_transform is None or getattr(self.qk_transform, "graph_safe", False)))
        self.w_qkv: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None
        self.rotate_in_attention = _decode_rotation == "attention"
        self.use_mfma = (kernels == "auto" and rt.dtype == torch.bfloat16 and rt.device.type == "cuda"
                         and K.attention_mfma_available(self.d))

    # ---- what it needs ---------------------------------------------------
    def cache_spec(self) -> CacheSpec:
        return CacheSpec("window" if self.window else "full", self.nkv, self.d, self.window)

    def step_needs(self) -> Dict[str, Any]:
        # the MFMA kernel for portions of prompts works on tiles of 64 query rows
        return {"row_tiles": K.PREFILL_TILE_ROWS} if self.use_mfma else {}

    def weights(self) -> Dict[str, WeightSpec]:
        nh, nkv, d, H = self.nh, self.nkv, self.d, self.hidden_size
        init = ("normal", self.init_std)
        own = {
            "q_proj.weight": WeightSpec((nh * d, H), init),
            "k_proj.weight": WeightSpec((nkv * d, H), init),
            "v_proj.weight": WeightSpec((nkv * d, H), init),
            "o_proj.weight": WeightSpec((H, nh * d), init),
        }
        if self.qk_transform is not None:
            extra = self.qk_transform.weights()
            if set(extra) & set(own):
                raise ValueError(f"the qk_transform's tensors {sorted(set(extra) & set(own))} have the attention's names")
            own.update(extra)
        return own

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        wq, wk = tensors["q_proj.weight"], tensors["k_proj.weight"]
        perm = self.position.head_permutation()
        if perm is not None:
            # the position encoding's own order of a head's values (see PositionEncoding.head_permutation)
            perm = perm.to(wq.device).long()
            if sorted(perm.tolist()) != list(range(self.d)):
                raise ValueError("the position encoding's head_permutation is no permutation of a head's values")
            wq = wq.view(self.nh, self.d, -1)[:, perm].reshape(wq.shape)
            wk = wk.view(self.nkv, self.d, -1)[:, perm].reshape(wk.shape)
        self.w_qkv = torch.cat([wq, wk, tensors["v_proj.weight"]], dim=0)
        self.w_qkv = self.w_qkv.contiguous()
        self.w_o = tensors["o_proj.weight"].contiguous()
        prepare_weights(self.rt, [(self.w_qkv, None, True), (self.w_qkv[: self.nh * self.d], None, True),
                                     (self.w_o, None, True)])
        if self.qk_transform is not None:
            self.qk_transform.load({name: tensors[name] for name in self.qk_transform.weights()})

    # ---- one step --------------------------------------------------------
    def forward(self, x: torch.Tensor, ctx: StepContext, cache: CacheView):
        nh, nkv, d = self.nh, self.nkv, self.d
        if cache.k_pages is None:
            raise K.KernelError("attention needs pages of the cache")
        g = cache.group
        if (self.use_mfma and self.rotate_in_attention and 0 < ctx.num_decode == x.shape[0] and self.qk_transform is None
                and x.shape[0] <= ROTATE_IN_ATTENTION_UP_TO and cache.k_pages.shape[2] % 4 == 0):
            # every request brings one token: rotation, the write to the pages and attention are one launch
            w = self.w_qkv if cache.writable else self.w_qkv[: nh * d]
            qkv = linear(x, w, keep_split=True, kernels=self.rt.kernels)
            out = torch.empty((x.shape[0], nh * d), dtype=x.dtype, device=x.device)
            K.attention_decode_rotating(qkv, ctx.positions, self.position.inv_freq, self.position.rotary_dim,
                                        ctx.slots[g] if cache.writable else None, cache.k_pages, cache.v_pages, out,
                                        ctx.block_tables[g], nh, nkv, d, self.scale, self.window, ctx.max_total_len)
            return linear(out, self.w_o, keep_split=True, kernels=self.rt.kernels)
        q_out = None
        if self.qk_transform is not None:
            w = self.w_qkv if cache.writable else self.w_qkv[: nh * d]
            qkv = self.qk_transform.forward(linear(x, w, kernels=self.rt.kernels), nh, nkv if cache.writable else 0, d, ctx)
            if cache.writable:
                q = K.rope_kv_append(qkv, ctx.positions, self.position.inv_freq, nh, nkv, d, self.position.rotary_dim,
                                     ctx.slots[g], cache.k_pages, cache.v_pages)
            else:
                q = K.rope_kv_append(qkv, ctx.positions, self.position.inv_freq, nh, nkv, d, self.position.rotary_dim)
        elif cache.writable:
            qkv = linear(x, self.w_qkv, keep_split=True, kernels=self.rt.kernels)
            if isinstance(qkv, K.SplitSum):
                q_out = torch.empty((x.shape[0], nh * d), dtype=x.dtype, device=x.device)
            q = K.rope_kv_append(qkv, ctx.positions, self.position.inv_freq, nh, nkv, d, self.position.rotary_dim,
                                 ctx.slots[g], cache.k_pages, cache.v_pages, q_out=q_out)
        else:
            # keys and values of another run of a layer: only queries are made here
            qkv = linear(x, self.w_qkv[: nh * d], keep_split=True, kernels=self.rt.kernels)
            if isinstance(qkv, K.SplitSum):
                q_out = torch.empty((x.shape[0], nh * d), dtype=x.dtype, device=x.device)
            q = K.rope_kv_append(qkv, ctx.positions, self.position.inv_freq, nh, nkv, d, self.position.rotary_dim,
                                 q_out=q_out)
        out = torch.empty((x.shape[0], nh * d), dtype=x.dtype, device=x.device)
        self.attend(q, out, ctx, cache)
        return linear(out, self.w_o, keep_split=True, kernels=self.rt.kernels)

    def native(self, program, view: CacheView) -> None:
        """The launches of ``forward`` and ``attend``, each with the steps it is for: steps of up to
        ROTATE_IN_ATTENTION_UP_TO single tokens take the kernel that rotates, writes the pages and attends in one
        launch; all others the rotary kernel, then the kernel for single tokens on the first rows and the one for
        portions of prompts on the rest (or the plain kernel on all rows)."""
        if type(self).forward is not Attention.forward or type(self).attend is not Attention.attend:
            return super().native(program, view)              # a subclass that computes something else
        from ..engine.program import NEVER, STREAM, Guard
        if view is None or view.k_pages is None or view.v_pages is None:
            raise K.KernelError("attention needs pages of the cache")
        nh, nkv, d, window, rt = self.nh, self.nkv, self.d, self.window, self.rt
        k, v, g, writable = view.k_pages, view.v_pages, view.group, view.writable
        ps, num_pages = int(k.shape[2]), int(k.shape[0])
        inv_freq = self.position.inv_freq
        rot = self.position.rotary_dim if inv_freq is not None else 0
        f64 = int(inv_freq is not None and inv_freq.dtype == torch.float64)
        w = self.w_qkv if writable else self.w_qkv[: nh * d]     # another run's keys and values: only queries are made
        row, T, N = int(w.shape[0]), program.T, program.N
        act, scale = program.act_code, float(self.scale)
        mfma = self.use_mfma and ps % 4 == 0
        program.keep(k, v, inv_freq, w)
        bt, bt_cols = program.block_table(g), program.bt_cols(g)
        slots = program.slots(g) if writable else None
        out = program.buffer("attention.out", T * nh * d * program.act_bytes)
        fused = NEVER
        if mfma and self.rotate_in_attention and self.qk_transform is None:
            fused = Guard.between(program.NPT, 0, 0) & Guard.between(N, 1, ROTATE_IN_ATTENTION_UP_TO)
        separate = ~fused
        if mfma:
            lib = K._attn(d)
            records = T + 1024      # requests x parts of their keys: what fills the GPU, or the requests themselves
            part_o = program.buffer("attention.part_o", records * nh * d * 4)
            part_ml = program.buffer("attention.part_ml", records * nh * 2 * 4)
            dev = rt.device

            def parts_of_the_keys(ctx: StepContext) -> int:
                nd = ctx.num_decode
                if nd == 0:
                    return 1
                if ctx.block_tables[g].shape[1] * ps < ctx.max_total_len:
                    raise K.KernelError("attention: the block tables are narrower than the longest request")
                n = K.decode_splits(nd, nh, nkv, ctx.max_total_len, dev, d)
                if nd * n > records:
                    raise K.KernelError("attention: the parts of the keys do not fit the program's arena")
                return n

            def launch_shape(ctx: StepContext) -> int:
                nd = ctx.num_decode
                if ctx.num_seqs == nd:
                    return 0
                return K.prefill_launch_shape(nh, nkv, d, ctx.q_lens[nd:], ctx.ctx_lens[nd:], window, dev)
            splits = program.scalar(("attention: parts of the keys", nh, nkv, g, ps), parts_of_the_keys)
            shape = program.scalar(("attention: launch shape", nh, nkv, d, window), launch_shape)
            tiles, num_tiles = program.row_tiles(K.PREFILL_TILE_ROWS)
        qkv = emit_linear(program, program.x, N, w, rt.dtype, None, self.qk_transform is None, "attention.qkv",
                          "attention.qkv")
        if self.qk_transform is not None:
            where, transform, kv_heads = qkv.tensor(), self.qk_transform, (nkv if writable else 0)

            def between_projection_and_rotation(ctx: StepContext) -> None:
                t = where.view(rt.dtype, ctx.num_tokens, row)
                y = transform.forward(t, nh, kv_heads, d, ctx)
                if y.data_ptr() != t.data_ptr():
                    t.copy_(y)
            program.python(between_projection_and_rotation, type(transform).__name__)
        for alt in qkv.alts:
            src, code, parts = alt.where, (K.DTYPE_CODE[torch.float32] if alt.splits else act), (alt.splits or 1)
            if mfma:
                program.op(lib, "ia_attn_decode_fused",
                           [src, code, parts, N, row, slots, inv_freq, f64, rot, k, v, out, nh * d, part_o, part_ml,
                            program.positions, bt, bt_cols, N, nh, nkv, ps, num_pages, scale, window, splits, STREAM],
                           alt.when & fused)
            q, q_stride = src, row
            if alt.splits:                   # partial sums: the rotated queries get a tensor of their own
                q, q_stride = program.buffer("attention.q", T * nh * d * program.act_bytes), nh * d
            program.op("core", "ia_rope_kv_append",
                       [src, code, parts, N, q, q_stride, act, program.positions, slots, inv_freq, f64,
                        k if writable else None, v if writable else None, N, row, nh, nkv, d, rot,
                        ps if writable else 0, num_pages if writable else 0, int(writable), STREAM], alt.when & separate)
            if not mfma:
                program.op("core", "ia_attention_generic",
                           [q, q_stride, k, v, out, nh * d, act, program.token_seq, program.positions, bt, bt_cols, N, nh,
                            nkv, d, ps, num_pages, scale, window, STREAM], alt.when & separate)
                continue
            program.op(lib, "ia_attn_decode",
                       [q, q_stride, k, v, out, nh * d, part_o, part_ml, program.positions, bt, bt_cols, program.ND, nh,
                        nkv, ps, num_pages, scale, window, splits, STREAM],
                       alt.when & separate & Guard.between(program.ND, 1))
            program.op(lib, "ia_attn_prefill",
                       [q, q_stride, k, v, out, nh * d, program.seq_starts, program.seq_ctx, bt, bt_cols, tiles, num_tiles,
                        nh, nkv, ps, num_pages, scale, window, shape, STREAM],
                       alt.when & separate & Guard.between(program.NP, 1))
        program.pending = emit_linear(program, out, N, self.w_o, rt.dtype, None, True, "attention.mix", "attention.o")

    def attend(self, qkv: torch.Tensor, out: torch.Tensor, ctx: StepContext, cache: CacheView) -> None:
        nh, nkv, d = self.nh, self.nkv, self.d
        bt = ctx.block_tables[cache.group]
        if not self.use_mfma or cache.k_pages.shape[2] % 4:
            K.attention_generic(qkv, cache.k_pages, cache.v_pages, out, ctx.token_seq, ctx.positions, bt, nh, nkv, d,
                                self.scale, self.window)
            return
        nd = ctx.num_decode
        if nd > 0:
            K.attention_decode(qkv[:nd], cache.k_pages, cache.v_pages, out[:nd], ctx.positions[:nd], bt[:nd], nh, nkv,
                               d, self.scale, self.window, ctx.max_total_len)
        if ctx.num_seqs > nd:
            key = ("prefill_launch_shape", nh, nkv, d, self.window)
            hpw = ctx.extras.get(key)
            if hpw is None:             # once per step for all layers of this shape
                hpw = ctx.extras[key] = K.prefill_launch_shape(nh, nkv, d, ctx.q_lens[nd:], ctx.ctx_lens[nd:],
                                                               self.window, qkv.device)
            tiles, num_tiles = ctx.row_tiles(K.PREFILL_TILE_ROWS)
            K.attention_prefill(qkv, cache.k_pages, cache.v_pages, out, ctx.seq_starts, ctx.seq_ctx, bt,
                                tiles, num_tiles, nh, nkv, d, self.scale, self.window, hpw)


register_part("mixer", "attention", Attention)
