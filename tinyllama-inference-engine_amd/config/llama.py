"""The typed configuration of the Llama dense decoder, read from its own config.json keys.

Keys and their meaning follow the reference's ModelConfig (include/tlie/model_config.hpp:17-43,
src/model_config.cpp:25-43).  The reference accepts exactly one checkpoint
(`ValidateFixedTinyLlama`, src/model_config.cpp:54-76); here only the structural checks stay
(:63-65 and the positivity that the operators demand, src/operators.cpp:27,50,54), so that any
Llama of any size loads.  Options the engine does not implement are refused, never ignored.
"""
from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, asdict
from typing import Any, Mapping

from ..errors import EngineError, ErrorCode, invalid_config
from .spec import LayerSpec, ModelSpec, PartSpec, Run

_MISSING = object()


def _take(raw: Mapping[str, Any], key: str, kind, default=_MISSING):
    if key not in raw or raw[key] is None:
        if default is _MISSING:
            raise invalid_config(f"config.json lacks the key '{key}'")
        return default
    value = raw[key]
    if kind is bool:
        if not isinstance(value, bool):
            raise invalid_config(f"'{key}' must be true or false, not {value!r}")
        return value
    if kind is int:
        if isinstance(value, bool) or not isinstance(value, int):
            raise invalid_config(f"'{key}' must be an integer, not {value!r}")
        return value
    if kind is float:
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise invalid_config(f"'{key}' must be a number, not {value!r}")
        return float(value)
    if kind is str:
        if not isinstance(value, str):
            raise invalid_config(f"'{key}' must be a string, not {value!r}")
        return value
    raise AssertionError(kind)


@dataclass(frozen=True)
class LlamaConfig:
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    vocab_size: int
    rms_norm_eps: float
    rope_theta: float
    attention_bias: bool
    tie_word_embeddings: bool
    hidden_act: str
    bos_token_id: int
    eos_token_id: int
    torch_dtype: str
    architecture: str = "LlamaForCausalLM"

    # ---- derived (include/tlie/model_config.hpp:34-38) -------------------------------------
    @property
    def q_dim(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @property
    def query_groups(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    # ---- reading --------------------------------------------------------------------------
    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "LlamaConfig":
        model_type = _take(raw, "model_type", str, "llama")
        if model_type != "llama":
            raise invalid_config(f"model_type must be llama, not '{model_type}'")
        architectures = raw.get("architectures") or ["LlamaForCausalLM"]
        if not isinstance(architectures, list) or not architectures or not isinstance(architectures[0], str):
            raise invalid_config("'architectures' must be a list of names")
        hidden = _take(raw, "hidden_size", int)
        heads = _take(raw, "num_attention_heads", int)
        if heads <= 0:
            raise invalid_config("num_attention_heads must be positive")
        if "head_dim" in raw and raw["head_dim"] is not None:
            head_dim = _take(raw, "head_dim", int)
        else:
            if hidden % heads != 0:
                raise invalid_config(f"hidden_size {hidden} is not a multiple of num_attention_heads {heads}, and no head_dim is given")
            head_dim = hidden // heads
        scaling = raw.get("rope_scaling")
        if scaling is not None:
            raise invalid_config("rope_scaling is not implemented; it must be absent or null")
        if _take(raw, "mlp_bias", bool, False):
            raise invalid_config("mlp_bias is not implemented; it must be absent or false")
        config = cls(
            hidden_size=hidden,
            intermediate_size=_take(raw, "intermediate_size", int),
            num_hidden_layers=_take(raw, "num_hidden_layers", int),
            num_attention_heads=heads,
            num_key_value_heads=_take(raw, "num_key_value_heads", int, heads),
            head_dim=head_dim,
            max_position_embeddings=_take(raw, "max_position_embeddings", int),
            vocab_size=_take(raw, "vocab_size", int),
            rms_norm_eps=_take(raw, "rms_norm_eps", float),
            rope_theta=_take(raw, "rope_theta", float, 10000.0),
            attention_bias=_take(raw, "attention_bias", bool, False),
            tie_word_embeddings=_take(raw, "tie_word_embeddings", bool, False),
            hidden_act=_take(raw, "hidden_act", str, "silu"),
            bos_token_id=_take(raw, "bos_token_id", int, -1),
            eos_token_id=_take(raw, "eos_token_id", int, -1),
            torch_dtype=_take(raw, "torch_dtype", str, "bfloat16"),
            architecture=architectures[0],
        )
        config.validate()
        return config

    @classmethod
    def load(cls, path: str) -> "LlamaConfig":
        return cls.from_dict(read_config_json(path))

    def validate(self) -> None:
        for name in ("hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
                     "num_key_value_heads", "head_dim", "max_position_embeddings", "vocab_size"):
            if getattr(self, name) <= 0:
                raise invalid_config(f"{name} must be positive, not {getattr(self, name)}")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise invalid_config(
                f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2 != 0:
            raise invalid_config(f"head_dim {self.head_dim} must be even for rotary positions")
        if not (self.rms_norm_eps > 0.0) or not math.isfinite(self.rms_norm_eps):
            raise invalid_config("rms_norm_eps must be positive")
        if not (self.rope_theta > 0.0) or not math.isfinite(self.rope_theta):
            raise invalid_config("rope_theta must be positive")
        if self.hidden_act != "silu":
            raise invalid_config(f"hidden_act '{self.hidden_act}' is not implemented; only silu is")

    def to_dict(self) -> dict:
        out = asdict(self)
        out["architectures"] = [out.pop("architecture")]
        out["model_type"] = "llama"
        return out

    # ---- the model as data ----------------------------------------------------------------
    def to_spec(self) -> ModelSpec:
        """Every block is RMSNorm -> rotary GQA attention -> RMSNorm -> SiLU-gated MLP
        (src/model.cpp:132-203), the layers run once each in order, each with its own cache."""
        norm = PartSpec("rms_norm", {"size": self.hidden_size, "eps": self.rms_norm_eps})
        mixer = PartSpec("attention", {
            "hidden_size": self.hidden_size,
            "num_heads": self.num_attention_heads,
            "num_kv_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "bias": self.attention_bias,
            "window": None,
            "position": PartSpec("rotary", {"head_dim": self.head_dim, "theta": self.rope_theta,
                                            "max_positions": self.max_position_embeddings}),
        })
        feed_forward = PartSpec("gated_mlp", {
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "activation": self.hidden_act,
        })
        layers = tuple(
            LayerSpec(prefix=f"model.layers.{index}.", block="pre_norm", mixer=mixer,
                      feed_forward=feed_forward, mixer_norm=norm, feed_forward_norm=norm)
            for index in range(self.num_hidden_layers))
        spec = ModelSpec(
            architecture=self.architecture,
            hidden_size=self.hidden_size,
            vocab_size=self.vocab_size,
            max_positions=self.max_position_embeddings,
            embedding=PartSpec("token_embedding", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size}),
            layers=layers,
            runs=tuple(Run(layer=index, cache_of=index) for index in range(self.num_hidden_layers)),
            final_norm=norm,
            head=PartSpec("lm_head", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
                                      "tied": self.tie_word_embeddings}),
            bos_token_id=self.bos_token_id,
            eos_token_id=self.eos_token_id,
            # some writers of Llama checkpoints store the rotation's frequency table as a buffer
            ignored_tensors=(r".*\.rotary_emb\.inv_freq",),
        )
        spec.validate()
        return spec


def read_config_json(path: str) -> dict:
    """Reads DIR/config.json (or the file itself).  A missing file is `io_error`, anything that
    is not a JSON object `invalid_config` (src/model_config.cpp:18-21,49-51)."""
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    try:
        with open(path, "r", encoding="utf-8") as handle:
            text = handle.read()
    except OSError as error:
        raise EngineError(ErrorCode.IO, f"unable to open model config: {path} ({error.strerror})") from None
    try:
        raw = json.loads(text)
    except json.JSONDecodeError as error:
        raise invalid_config(f"invalid model config JSON: {error}") from None
    if not isinstance(raw, dict):
        raise invalid_config("invalid model config JSON: the top level must be an object")
    return raw
