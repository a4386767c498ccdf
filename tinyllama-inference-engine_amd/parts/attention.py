"""Grouped-query causal attention over the paged cache.

reference (one token at a time, src/model.cpp:140-179; src/cuda/model.cu:412-447): q, k, v
projections of the normed input; rotation of q and k; the rotated key and the value go to the
cache at the token's position; each query head h attends over the cached keys 0..pos of kv head
h // (nq / nkv) with scores scaled by 1/sqrt(d) after the dot product; the output projection
follows.  Here the three projections are one product over the concatenated weight, the rotation
and the cache write are one kernel, and all tokens of a step run together.
"""
from __future__ import annotations

import math
from functools import partial

import torch

from .. import ops
from ..config.spec import PartSpec, TensorSpec
from ..errors import invalid_config
from ..registry import lookup, register
from ..weights.arena import keep_in
from .base import Binding, CacheNeed, Mixer, PositionEncoding
from .linear import Linear


@register("mixer", "attention")
class Attention(Mixer):
    """spec: hidden_size, num_heads, num_kv_heads, head_dim, bias, window (None or a count of
    positions), position (a PartSpec of a position encoding).
    Tensors: `<prefix>{q,k,v,o}_proj.weight` (and `.bias` when bias)."""

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.hidden = int(spec["hidden_size"])
        self.nq = int(spec["num_heads"])
        self.nkv = int(spec["num_kv_heads"])
        self.d = int(spec["head_dim"])
        self.bias = bool(spec.get("bias", False))
        self.window = spec.get("window")
        if self.nq <= 0 or self.nkv <= 0 or self.nq % self.nkv != 0:
            raise invalid_config("attention: num_heads must be a positive multiple of num_kv_heads")
        if not 0 < self.d <= ops.ATTENTION_MAX_HEAD_DIM:
            # said here, where the model is built, not by the first step's launch
            raise invalid_config(f"attention: head_dim {self.d} is beyond what the attention kernels take "
                                 f"(1 to {ops.ATTENTION_MAX_HEAD_DIM})")
        if self.window is not None and int(self.window) <= 0:
            raise invalid_config("attention: a window must be a positive count of positions")
        position = spec.get("position") or PartSpec("none")
        self.position = lookup("position_encoding", position.kind)(position, dtype, device)
        self.scale = 1.0 / math.sqrt(float(self.d))
        self.qkv = self.o = None

    @classmethod
    def tensor_specs(cls, spec, prefix):
        hidden, d = int(spec["hidden_size"]), int(spec["head_dim"])
        qd, kvd = int(spec["num_heads"]) * d, int(spec["num_kv_heads"]) * d
        shapes = (("q_proj", (qd, hidden)), ("k_proj", (kvd, hidden)), ("v_proj", (kvd, hidden)), ("o_proj", (hidden, qd)))
        specs = [TensorSpec(f"{prefix}{name}.weight", shape) for name, shape in shapes]
        if spec.get("bias", False):
            specs += [TensorSpec(f"{prefix}{name}.bias", (shape[0],)) for name, shape in shapes]
        return specs

    def load(self, weights, prefix):
        # The rows of the fused q/k/v weight are stored with the two elements of a rotation pair
        # side by side when the position encoding is a rotation table: the product of few rows then
        # rotates and writes the cache itself; the kernels that read its output know the order.
        table = self.position.rotary_table()
        self.paired = table is not None
        order = ops.paired_rows(self.nq, self.nkv, self.d, table[1]).to(self.device) if self.paired else None

        def cat(suffix):
            joined = torch.cat([weights[f"{prefix}{name}_proj.{suffix}"] for name in "qkv"], dim=0)
            return joined[order].contiguous() if order is not None else joined
        keep = partial(keep_in, weights)
        self.qkv = Linear(cat("weight"), cat("bias") if self.bias else None, self.dtype, keep=keep)
        self.o = Linear(weights[prefix + "o_proj.weight"], weights.get(prefix + "o_proj.bias") if self.bias else None,
                        self.dtype, keep=keep)

    @property
    def graph_safe(self) -> bool:
        # a rotation table (or none) is fused into this part's own kernels; a position encoding applied
        # as tensors (`apply_qk`) may do anything, so it says itself whether its launches may be recorded
        if self.position.rotary_table() is not None or type(self.position).apply_qk is PositionEncoding.apply_qk:
            return True
        return bool(getattr(self.position, "graph_safe", False))

    adds_to_residual = True

    def takes_normed_rows(self, rows: int) -> bool:
        return self.qkv.takes_rows(rows)

    def cache_need(self):
        """A page holds two planes per kv head, [2, nkv, page_size * d]: the rotated keys as
        [position][dim] and the values transposed, [dim][position], which is how the attention
        kernels want them as matrix operands (`ops.rope_cache` writes them so)."""
        return CacheNeed((2, self.nkv), self.d, int(self.window) if self.window is not None else None)

    def forward(self, x, ctx, binding: Binding, into=None):
        pages = ctx.groups[binding.group]
        slot_map = pages.slot_map if binding.writes else ctx.no_slots
        table = self.position.rotary_table()
        inv_freq, rot_dim = table if table is not None else (None, 0)
        other_positions = table is None and type(self.position).apply_qk is not PositionEncoding.apply_qk
        target = None
        if not other_positions:
            target = ops.RopeTarget(ctx.positions, slot_map, inv_freq, rot_dim, binding.cache, self.nq, self.nkv, self.d)
        q = self.qkv(x, rope=target)
        if isinstance(q, ops.Product):              # the product did not rotate: a kernel of its own does
            if other_positions:
                q = self._apply_other_positions(q, ctx)
            q = ops.rope_cache(q, ctx.positions, slot_map, inv_freq, rot_dim, binding.cache, self.nq, self.nkv, self.d,
                               self.dtype, paired=self.paired)
        page_size = binding.cache.shape[3] // self.d
        if ops.attention_mfma_takes(self.dtype, self.d, page_size):
            tiles, col_tiles, nsplit, split_len, waves, shared = ops.attention_plan(ctx, self.nq // self.nkv, self.nkv, self.d)
            attended = ops.attention_mfma(q, binding.cache, pages.block_table, tiles, ctx.positions, self.nq, self.nkv,
                                          self.d, self.window, self.scale, nsplit, split_len, col_tiles, waves, shared)
        else:
            attended = ops.attention_generic(q, binding.cache, pages.block_table, ctx.token_seq, ctx.positions, self.nq,
                                             self.nkv, self.d, self.window, self.scale,
                                             tiled=ops.attention_generic_plan(ctx, self.d), seq_start=ctx.seq_start)
        return self.o(attended, into=into)

    def _apply_other_positions(self, qkv, ctx):
        """A position encoding that is no rotation table: applied to q and k as tensors."""
        dense = qkv.dense(self.dtype)
        qd, kvd = self.nq * self.d, self.nkv * self.d
        q, k = self.position.apply_qk(dense[:, :qd].reshape(-1, self.nq, self.d),
                                      dense[:, qd:qd + kvd].reshape(-1, self.nkv, self.d), ctx.positions)
        joined = torch.cat([q.reshape(-1, qd), k.reshape(-1, kvd), dense[:, qd + kvd:]], dim=1).contiguous()
        return ops.Product(joined, 1)
