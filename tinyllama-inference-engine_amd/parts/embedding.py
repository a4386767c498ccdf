"""The two ends of the model: the token embedding and the output head.

reference: the embedding is a row copy, unscaled (src/model.cpp:94-97); the head is a plain
product of the final norm's output with `lm_head.weight`, no bias, no scaling
(src/model.cpp:224-225).  With tied embeddings the head's matrix is the embedding table.
Logits are float32 whatever the activation type."""
from __future__ import annotations

from functools import partial

import torch

from .. import ops
from ..config.spec import PartSpec, TensorSpec
from ..registry import register
from ..weights.arena import keep_in
from .base import Part
from .linear import Linear


@register("embedding", "token_embedding")
class TokenEmbedding(Part):
    graph_safe = True
    NAME = "model.embed_tokens.weight"

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.table = None

    @classmethod
    def tensor_specs(cls, spec, name=""):
        """`name`: the table's full name in the checkpoint (the model's spec gives it; without one,
        the reference's)."""
        return [TensorSpec(name or cls.NAME, (int(spec["vocab_size"]), int(spec["hidden_size"])))]

    def load(self, weights, name=""):
        self.table = keep_in(weights, weights[name or self.NAME].contiguous())

    def forward(self, tokens: torch.Tensor, ctx=None) -> torch.Tensor:
        """The float32 residual [T, H] of the step's tokens.  `ctx` is the step's context: an
        embedding that depends on more than the token (positions learned per place, say) reads it."""
        return ops.embed_gather(tokens, self.table)

    def forward_rows(self, tokens: torch.Tensor, next_norm: tuple):
        """For a step of few rows: the residual and the first norm's inputs in one launch."""
        return ops.embed_rows(tokens, self.table, next_norm)


@register("head", "lm_head")
class LMHead(Part):
    graph_safe = True
    NAME = "lm_head.weight"

    def __init__(self, spec: PartSpec, dtype, device):
        """spec: vocab_size, hidden_size, tied (the head's matrix is the embedding's table), and, when
        tied, optionally tied_to: that table's full name (default: the reference's)."""
        super().__init__(spec, dtype, device)
        self.tied = bool(spec.get("tied", False))
        self.tied_to = spec.get("tied_to") or TokenEmbedding.NAME
        self.linear = None

    @classmethod
    def tensor_specs(cls, spec, name=""):
        shape = (int(spec["vocab_size"]), int(spec["hidden_size"]))
        # a tied model may still carry the head's matrix; it is then not read
        return [TensorSpec(name or cls.NAME, shape, optional=bool(spec.get("tied", False)))]

    def load(self, weights, name=""):
        matrix = weights[self.tied_to] if self.tied else weights[name or self.NAME]
        self.linear = Linear(matrix, None, self.dtype, keep=partial(keep_in, weights))

    def takes_normed_rows(self, rows: int) -> bool:
        return self.linear.takes_rows(rows)

    def forward(self, normed) -> torch.Tensor:
        return self.linear(normed, out_dtype=torch.float32, whole=True).dense(torch.float32)
