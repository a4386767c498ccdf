"""How a layer's parts are arranged.

"pre_norm" is the reference's block (src/model.cpp:132-203): x += mixer(norm(x)), then
x += feed_forward(norm(x)); the residual itself is never normed in place.  The residual is a
float32 array that lives for the whole step.  A block does not add its last result itself: it
hands it on as `pending`, and whoever norms the residual next (the next block's first norm, or
the model's final norm) adds it in the same kernel.
"""
from __future__ import annotations

import torch

from ..config.spec import LayerSpec
from .. import ops
from ..ops import ResidualUpdated, as_product
from ..registry import lookup, register
from .base import ResidualTarget


@register("block", "pre_norm")
class PreNormBlock:
    def __init__(self, layer: LayerSpec, dtype, device):
        self.layer = layer
        self.dtype = dtype
        self.mixer_norm = lookup("norm", layer.mixer_norm.kind)(layer.mixer_norm, dtype, device)
        self.mixer = lookup("mixer", layer.mixer.kind)(layer.mixer, dtype, device)
        self.feed_forward_norm = lookup("norm", layer.feed_forward_norm.kind)(layer.feed_forward_norm, dtype, device)
        self.feed_forward = lookup("feed_forward", layer.feed_forward.kind)(layer.feed_forward, dtype, device)

    _PARTS = ("mixer_norm", "mixer", "feed_forward_norm", "feed_forward")

    @staticmethod
    def _place(layer: LayerSpec, attribute: str) -> str:
        """Where a part's tensors lie: the layer's prefix and the place the layer's spec names."""
        return layer.prefix + getattr(layer, attribute + "_place")

    @classmethod
    def tensor_specs(cls, layer: LayerSpec):
        specs = []
        for attribute in cls._PARTS:
            part_spec = getattr(layer, attribute)
            table = {"mixer_norm": "norm", "feed_forward_norm": "norm"}.get(attribute, attribute)
            specs += lookup(table, part_spec.kind).tensor_specs(part_spec, cls._place(layer, attribute))
        return specs

    def load(self, weights):
        for attribute in self._PARTS:
            getattr(self, attribute).load(weights, self._place(self.layer, attribute))

    def entry_norm(self):
        """The norm that reads the residual first in this block: whoever writes the residual before
        the block (the embedding, the block before) may leave that norm's inputs with it."""
        return self.mixer_norm

    @property
    def graph_safe(self) -> bool:
        return all(getattr(part, "graph_safe", False)
                   for part in (self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward))

    def forward(self, residual, pending, ctx, binding, next_norm=None):
        """`pending`: what the residual still lacks (a product, a `ResidualUpdated`, or None).
        `next_norm`: the norm that reads the residual after this block, if the caller knows it.
        In a step of few rows the parts that offer it fold the norms into their products and add
        their results into the residual themselves; otherwise the norm kernels do both.
        A step that keeps a trace (`ctx.trace`, a dict) leaves there, under `ctx.trace_prefix`, the
        five tensors the reference's ModelTrace keeps per layer
        (src/model.cpp:136-138,176-177,184-185,200-201,204-205), as float32 copies, and takes the route
        on which all five exist; with `ctx.trace_serving_route` a step of few rows takes the route
        it takes without a trace and leaves those that still exist there: "attention_output" and
        "mlp_output" (what the part added into the residual: the residual after it minus the
        residual before) and "output" (the normed inputs are folded away)."""
        trace = getattr(ctx, "trace", None)
        rows = residual.shape[0]
        few = ops.few_rows_route(rows, self.dtype) and (trace is None or getattr(ctx, "trace_serving_route", False))
        if trace is not None and not few:
            return self._forward_traced(residual, pending, ctx, binding)

        def keep(name, tensor):
            trace[ctx.trace_prefix + name] = tensor.float().clone()
        normed = self.mixer_norm.add_forward(residual, pending, lazy=few and self.mixer.takes_normed_rows(rows))
        before = residual.clone() if trace is not None else None
        if few and self.mixer.adds_to_residual:
            mixed = self.mixer.forward(normed, ctx, binding, into=ResidualTarget(residual, self.feed_forward_norm.lazy_params()))
        else:
            mixed = self.mixer.forward(normed, ctx, binding)
        normed = self.feed_forward_norm.add_forward(residual, mixed, lazy=few and self.feed_forward.takes_normed_rows(rows))
        if trace is not None:
            keep("attention_output", residual - before)        # (whoever added it, the residual holds it now)
            before = residual.clone()
        if few and self.feed_forward.adds_to_residual:
            out = self.feed_forward.forward(normed, ctx, into=ResidualTarget(
                residual, next_norm.lazy_params() if next_norm is not None else None))
        else:
            out = self.feed_forward.forward(normed, ctx)
        if trace is not None:
            added = residual - before if isinstance(out, ResidualUpdated) else as_product(out).dense(torch.float32)
            keep("mlp_output", added)
            keep("output", before + added)
        return out

    def _forward_traced(self, residual, pending, ctx, binding):
        def keep(name, tensor):
            ctx.trace[ctx.trace_prefix + name] = tensor.float().clone()

        def dense(result):
            return as_product(result).dense(torch.float32)
        normed = self.mixer_norm.add_forward(residual, pending)
        keep("input_norm", normed)
        mixed = self.mixer.forward(normed, ctx, binding)
        keep("attention_output", dense(mixed))
        normed = self.feed_forward_norm.add_forward(residual, mixed)
        keep("post_attention_norm", normed)
        out = self.feed_forward.forward(normed, ctx)
        keep("mlp_output", dense(out))
        keep("output", residual + dense(out))
        return out
