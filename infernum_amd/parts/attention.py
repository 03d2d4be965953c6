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
import os
from typing import Any, Dict, Mapping, Optional

import torch

from ..kernels import api as K
from .base import (CacheSpec, CacheView, Mixer, PartSpec, Runtime, StepContext, WeightSpec, make_part,
                   register_part)
from .linear import linear, measure_routes_for


# Steps of up to this many single tokens rotate inside the attention kernel (8B shape: 1.5 % faster at 1 and 8
# tokens, 0.4 % at 64; at 128 the rotary kernel in front is 1 % faster: every workgroup of the attention starts
# with the rotation, and with many of them that costs more than the one launch it saves).
ROTATE_IN_ATTENTION_UP_TO = 64
DECODE_ROTATIONS = ("attention", "separate")
_decode_rotation = os.environ.get("INFERNUM_DECODE_ROTATE", "attention")
if _decode_rotation not in DECODE_ROTATIONS:
    raise ValueError(f"INFERNUM_DECODE_ROTATE={_decode_rotation!r}: one of {DECODE_ROTATIONS}")


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
        self.w_qkv = torch.cat([tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]], dim=0)
        self.w_qkv = self.w_qkv.contiguous()
        self.w_o = tensors["o_proj.weight"].contiguous()
        measure_routes_for(self.rt, [(self.w_qkv, None, True), (self.w_qkv[: self.nh * self.d], None, True),
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

    def native(self, program, view: CacheView) -> bool:
        from . import rope
        if type(self) is not Attention or type(self.position) not in (rope.RotaryEmbedding, rope.NoPositionEncoding):
            return False                      # a subclass may do something else in forward
        if self.qk_transform is not None:
            return False                      # a part of the model's own between projection and rotation
        if view is None or view.k_pages is None or view.v_pages is None:
            return False
        program.add_attention(self, view)
        return True

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
