"""Configuration and registry.  The error cases follow the reference's unit tests of its config
(tests/unit_tests.cpp:92-112: the fixture loads, derived sizes are right, a mutated size is
`invalid_config`), widened to any Llama, since this engine pins no checkpoint."""
import json

import pytest

import tlie_amd
from tlie_amd import EngineError, ErrorCode, LlamaConfig
from tlie_amd.config import read_config_json
from tlie_amd.models import expected_tensors
from tlie_amd.registry import config_from_dict

# tests/fixtures/config.json:1-18 of the reference
FIXTURE = {"attention_bias": False, "bos_token_id": 1, "eos_token_id": 2, "hidden_act": "silu", "hidden_size": 2048,
           "intermediate_size": 5632, "max_position_embeddings": 2048, "model_type": "llama",
           "num_attention_heads": 32, "num_hidden_layers": 22, "num_key_value_heads": 4, "rms_norm_eps": 1e-05,
           "rope_theta": 10000.0, "tie_word_embeddings": False, "torch_dtype": "bfloat16", "vocab_size": 32000}


def code_of(call):
    with pytest.raises(EngineError) as caught:
        call()
    return caught.value.code


def test_fixture_loads_with_derived_sizes():
    config = config_from_dict(FIXTURE)
    assert isinstance(config, LlamaConfig)
    assert (config.head_dim, config.kv_dim, config.q_dim, config.query_groups) == (64, 256, 2048, 8)
    specs = expected_tensors(config.to_spec())
    assert len(specs) == 22 * 9 + 3                      # src/model_config.cpp:80
    shapes = {spec.name: spec.shape for spec in specs}
    assert shapes["model.layers.21.self_attn.k_proj.weight"] == (256, 2048)
    assert shapes["model.layers.0.mlp.down_proj.weight"] == (2048, 5632)
    assert shapes["lm_head.weight"] == (32000, 2048)


def test_defaults_and_optional_keys():
    raw = {"model_type": "llama", "hidden_size": 96, "intermediate_size": 256, "num_hidden_layers": 3,
           "num_attention_heads": 3, "head_dim": 32, "max_position_embeddings": 256, "vocab_size": 512, "rms_norm_eps": 1e-6}
    config = config_from_dict(raw)
    assert config.num_key_value_heads == 3 and config.rope_theta == 10000.0 and not config.attention_bias
    assert config.q_dim == 96 and config.bos_token_id == -1
    tied = config_from_dict(dict(raw, tie_word_embeddings=True, attention_bias=True, num_key_value_heads=1))
    specs = expected_tensors(tied.to_spec())
    names = {spec.name: spec for spec in specs}
    assert names["lm_head.weight"].optional
    assert names["model.layers.2.self_attn.o_proj.bias"].shape == (96,)
    assert names["model.layers.2.self_attn.k_proj.bias"].shape == (32,)
    assert len([s for s in specs if not s.optional]) == 3 * 13 + 2


@pytest.mark.parametrize("change", [
    {"hidden_size": None}, {"rms_norm_eps": None}, {"vocab_size": None},          # a missing key
    {"model_type": "mistral"}, {"hidden_size": 0}, {"hidden_size": 2047},         # 2047 % 32 != 0 and no head_dim
    {"num_key_value_heads": 5}, {"head_dim": 63}, {"rms_norm_eps": 0.0}, {"rope_theta": -1.0},
    {"hidden_act": "gelu"}, {"rope_scaling": {"type": "linear", "factor": 2.0}}, {"mlp_bias": True},
    {"attention_bias": "no"}, {"num_hidden_layers": "22"}, {"vocab_size": 1.5},
])
def test_invalid_config(change):
    raw = dict(FIXTURE)
    for key, value in change.items():
        if value is None:
            raw.pop(key)
        else:
            raw[key] = value
    assert code_of(lambda: config_from_dict(raw)) == ErrorCode.INVALID_CONFIG


def test_registry_chooses_by_architecture():
    assert code_of(lambda: config_from_dict(dict(FIXTURE, architectures=["MambaForCausalLM"]))) == ErrorCode.INVALID_CONFIG
    assert code_of(lambda: config_from_dict({"hidden_size": 4})) == ErrorCode.INVALID_CONFIG
    assert isinstance(config_from_dict(dict(FIXTURE, architectures=["LlamaForCausalLM"])), LlamaConfig)


def test_reading_the_file(tmp_path):
    assert code_of(lambda: read_config_json(str(tmp_path))) == ErrorCode.IO       # src/model_config.cpp:18-21
    (tmp_path / "config.json").write_text("{ not json")
    assert code_of(lambda: read_config_json(str(tmp_path))) == ErrorCode.INVALID_CONFIG
    (tmp_path / "config.json").write_text("[1, 2]")
    assert code_of(lambda: read_config_json(str(tmp_path))) == ErrorCode.INVALID_CONFIG
    (tmp_path / "config.json").write_text(json.dumps(FIXTURE))
    assert config_from_dict(read_config_json(str(tmp_path))).vocab_size == 32000


def test_spec_is_data():
    spec = config_from_dict(FIXTURE).to_spec()
    assert [run.layer for run in spec.runs] == list(range(22)) and all(run.cache_of == i for i, run in enumerate(spec.runs))
    assert spec.layers[0].mixer.kind == "attention" and spec.layers[0].mixer["position"].kind == "rotary"
    assert spec.layers[3].feed_forward["intermediate_size"] == 5632
    # an order that names a layer twice and lets a run read another run's cache is valid data
    from dataclasses import replace
    from tlie_amd.config import Run
    twice = replace(spec, runs=(Run(0, 0), Run(1, 1), Run(0, 2), Run(1, 1)))
    twice.validate()
    with pytest.raises(EngineError):
        replace(spec, runs=(Run(0, 1), Run(1, 1))).validate()     # reads a cache that runs later
    with pytest.raises(EngineError):
        replace(spec, runs=(Run(0, 0), Run(1, 0), Run(1, 1))).validate()   # run 2 reads run 1, which owns none


def test_a_head_size_the_kernels_do_not_take_is_refused_where_the_part_is_built():
    """Not by the first step's launch: building the attention part (as the engine does when it
    builds the model) refuses a head size beyond the kernels', with the limit in the message."""
    import torch
    from tlie_amd.config import PartSpec
    from tlie_amd.parts.attention import Attention

    def build(head_dim, heads=2, kv_heads=1):
        position = PartSpec("rotary", {"head_dim": head_dim, "theta": 1e4})
        return Attention(PartSpec("attention", {"hidden_size": 64, "num_heads": heads, "num_kv_heads": kv_heads, "head_dim": head_dim,
                                                "position": position}), torch.bfloat16, "cpu")
    assert build(256).d == 256
    with pytest.raises(EngineError) as caught:
        build(272)
    assert caught.value.code == ErrorCode.INVALID_CONFIG and "272" in caught.value.message and "256" in caught.value.message
    assert code_of(lambda: build(64, heads=3, kv_heads=2)) == ErrorCode.INVALID_CONFIG
    # the model built from a configuration goes the same way
    from tlie_amd.models.builder import DecoderModel
    wide = config_from_dict(dict(FIXTURE, head_dim=320, num_hidden_layers=1))
    assert code_of(lambda: DecoderModel(wide.to_spec(), torch.bfloat16, "cpu")) == ErrorCode.INVALID_CONFIG


def test_error_json_shape():
    error = tlie_amd.EngineError(ErrorCode.OUT_OF_BOUNDS, "x")
    assert json.loads(error.to_json()) == {"error": {"code": "out_of_bounds", "message": "x"}}
    names = {code.value for code in ErrorCode}
    assert {"io_error", "invalid_format", "checksum_mismatch", "invalid_config", "invalid_shape", "invalid_dtype",
            "out_of_memory", "out_of_bounds", "tokenizer_error", "numerical_error", "invalid_argument"} <= names


def test_the_device_allocators_refusal_is_out_of_memory():
    """reference: a failed device allocation is `out_of_memory` (src/cuda/weight_store.cpp:273-274)."""
    import torch
    from tlie_amd.errors import EngineError, device_memory_errors
    with pytest.raises(EngineError) as caught:
        with device_memory_errors("the cache pools"):
            raise torch.cuda.OutOfMemoryError("tried to allocate 1 TiB")
    assert caught.value.code.value == "out_of_memory" and "cache pools" in caught.value.message
    with pytest.raises(KeyError):                      # anything else passes through
        with device_memory_errors("the weights"):
            raise KeyError("x")
