"""What a configuration turns into: a description of the model as data.

A `ModelSpec` names, layer by layer, which mixer, feed-forward and norm a block is made of and
with which sizes and constants, and in which order the layers run.  Nothing below this point
reads config.json or knows an architecture's name; a part sees only its own `PartSpec`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping


@dataclass(frozen=True)
class PartSpec:
    """One part: the name it is registered under and its parameters (sizes, constants)."""
    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)

    def __getitem__(self, key: str) -> Any:
        return self.params[key]

    def get(self, key: str, default: Any = None) -> Any:
        return self.params.get(key, default)


@dataclass(frozen=True)
class LayerSpec:
    """One layer's parts, the prefix its tensors are stored under, and under that prefix the place
    of each part's tensors (the defaults are the names of the reference's checkpoints,
    src/model_config.cpp:81-95; an architecture whose files name them otherwise says so here)."""
    prefix: str                 # e.g. "model.layers.3."
    block: str                  # arrangement of the parts, e.g. "pre_norm"
    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec        # the norm in front of the mixer
    feed_forward_norm: PartSpec  # the norm in front of the feed-forward
    mixer_norm_place: str = "input_layernorm."
    mixer_place: str = "self_attn."
    feed_forward_norm_place: str = "post_attention_layernorm."
    feed_forward_place: str = "mlp."


@dataclass(frozen=True)
class Run:
    """One entry of the order in which layers run.

    `layer` indexes `ModelSpec.layers` (a layer may be named by several runs: its weights are
    then shared, each run keeps a cache of its own).  `cache_of` is the index of the run whose
    cache this run's mixer reads; a run that names itself owns a cache and writes to it, a run
    that names an earlier one only reads what that one wrote in the same step and before.
    """
    layer: int
    cache_of: int


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: PartSpec
    layers: tuple[LayerSpec, ...]
    runs: tuple[Run, ...]
    final_norm: PartSpec
    head: PartSpec
    bos_token_id: int = -1
    eos_token_id: int = -1
    # where the checkpoint keeps what stands outside the layers (the reference's names,
    # src/model_config.cpp:79,96-97): the embedding's table, the final norm's prefix, the head's matrix
    embedding_name: str = "model.embed_tokens.weight"
    final_norm_prefix: str = "model.norm."
    head_name: str = "lm_head.weight"
    # tensors that this architecture's files may carry although no part reads them (buffers that
    # some writers store): regular expressions matched against the whole name.  Anything else that
    # the parts do not expect is an error.
    ignored_tensors: tuple[str, ...] = ()

    def validate(self) -> None:
        from ..errors import invalid_config
        if not self.runs:
            raise invalid_config("a model needs at least one layer to run")
        for index, run in enumerate(self.runs):
            if not 0 <= run.layer < len(self.layers):
                raise invalid_config(f"run {index} names layer {run.layer}, which does not exist")
            if not 0 <= run.cache_of <= index:
                raise invalid_config(f"run {index} reads the cache of run {run.cache_of}, which does not run before it")
            if self.runs[run.cache_of].cache_of != run.cache_of:
                raise invalid_config(f"run {index} reads the cache of run {run.cache_of}, which owns none")


@dataclass(frozen=True)
class TensorSpec:
    """A tensor a part expects in the checkpoint: its full name, shape and kind of values."""
    name: str
    shape: tuple[int, ...]
    init: str = "normal"        # how random weights draw it: "normal", "norm" (around 1), "zeros"
    optional: bool = False       # absent is no error, present it is checked and not read (a tied head's matrix that some files still carry)
