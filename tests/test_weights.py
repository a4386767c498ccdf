"""The weight store.  Cases follow the reference's unit tests of its store
(tests/unit_tests.cpp:114-171: valid file, missing tensor, shape mismatch, wrong byte count,
truncated file), on safetensors files instead of its own format."""
import json
import os
import pathlib
import struct

import pytest
import torch
from safetensors.torch import load_file, save_file

from tlie_amd import EngineError, ErrorCode, LlamaConfig, write_random_model
from tlie_amd.models import expected_tensors
from tlie_amd.weights import SafetensorsFile, WeightStore, random_tensors, to_kept_precision, write_safetensors

TINY = dict(model_type="llama", hidden_size=32, intermediate_size=48, num_hidden_layers=2, num_attention_heads=4,
            num_key_value_heads=2, max_position_embeddings=64, vocab_size=40, rms_norm_eps=1e-5)


def code_of(call):
    with pytest.raises(EngineError) as caught:
        call()
    return caught.value


def test_round_trip_against_the_library(tmp_path):
    tensors = {"a": torch.randn(3, 5), "b.c": torch.randn(7).bfloat16(), "ids": torch.arange(6, dtype=torch.int64).view(2, 3),
               "empty": torch.zeros(0, 4)}
    mine = str(tmp_path / "mine.safetensors")
    write_safetensors(mine, tensors, {"k": "v"})
    theirs = load_file(mine)
    for name, tensor in tensors.items():
        assert torch.equal(theirs[name], tensor)
    lib = str(tmp_path / "lib.safetensors")
    save_file(tensors, lib)
    file = SafetensorsFile(lib)
    for name, tensor in tensors.items():
        assert torch.equal(file.tensor(name), tensor) and file.tensor(name).dtype == tensor.dtype


def test_random_model_loads_and_is_seeded(tmp_path):
    config = LlamaConfig.from_dict(TINY)
    one, two, other = (str(tmp_path / name) for name in ("one", "two", "other"))
    write_random_model(one, config, seed=3)
    write_random_model(two, config, seed=3)
    write_random_model(other, config, seed=4)
    specs = expected_tensors(config.to_spec())
    a = WeightStore(one).load(specs, torch.bfloat16, "cpu")
    b = WeightStore(two).load(specs, torch.bfloat16, "cpu")
    c = WeightStore(other).load(specs, torch.bfloat16, "cpu")
    assert set(a) == {spec.name for spec in specs}
    assert all(torch.equal(a[name], b[name]) for name in a)
    assert not torch.equal(a["lm_head.weight"], c["lm_head.weight"])
    assert json.loads(pathlib.Path(one, "config.json").read_text())["hidden_size"] == 32
    # a tensor's values depend on (seed, name) only, not on which other tensors are drawn
    alone = random_tensors([s for s in specs if s.name == "model.norm.weight"], seed=3)
    assert torch.equal(alone["model.norm.weight"], a["model.norm.weight"])
    assert abs(a["model.norm.weight"].float().mean().item() - 1.0) < 0.05           # norms are drawn around 1
    assert abs(a["lm_head.weight"].float().std().item() - 0.02) < 0.005


def test_kept_precision():
    assert to_kept_precision(torch.ones(2, dtype=torch.float16), torch.bfloat16).dtype == torch.bfloat16
    assert to_kept_precision(torch.ones(2, dtype=torch.bfloat16), torch.bfloat16).dtype == torch.bfloat16
    assert to_kept_precision(torch.ones(2, dtype=torch.float32), torch.bfloat16).dtype == torch.float32   # 32-bit stays
    assert to_kept_precision(torch.ones(2, dtype=torch.int64), torch.bfloat16).dtype == torch.int32        # integer tables
    assert to_kept_precision(torch.ones(2, dtype=torch.bfloat16), torch.float32).dtype == torch.float32
    assert code_of(lambda: to_kept_precision(torch.ones(2), torch.float16)).code == ErrorCode.INVALID_DTYPE


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    config = LlamaConfig.from_dict(TINY)
    specs = expected_tensors(config.to_spec())
    tensors = random_tensors(specs, seed=0)
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(32, 31).bfloat16()
    tensors["model.layers.0.extra.weight"] = torch.zeros(2).bfloat16()
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(4)         # a stored buffer: ignored
    write_safetensors(str(tmp_path / "model.safetensors"), tensors)
    ignored = config.to_spec().ignored_tensors
    error = code_of(lambda: WeightStore(str(tmp_path)).load(specs, torch.bfloat16, "cpu", ignored))
    assert error.code == ErrorCode.INVALID_SHAPE
    for piece in ("2 missing", "model.layers.1.mlp.up_proj.weight", "model.norm.weight", "1 unexpected",
                  "model.layers.0.extra.weight", "1 with a wrong shape", "stored [32, 31], expected [32, 32]"):
        assert piece in error.message, piece
    assert "inv_freq" not in error.message
    # which names may be carried unread is the architecture's: the store itself knows none
    error = code_of(lambda: WeightStore(str(tmp_path)).load(specs, torch.bfloat16, "cpu"))
    assert "2 unexpected" in error.message and "rotary_emb.inv_freq" in error.message


def test_tied_model_may_carry_its_head(tmp_path):
    config = LlamaConfig.from_dict(dict(TINY, tie_word_embeddings=True))
    specs = expected_tensors(config.to_spec())
    tensors = random_tensors(specs, seed=0)
    assert "lm_head.weight" not in tensors
    write_safetensors(str(tmp_path / "model.safetensors"), tensors)
    WeightStore(str(tmp_path)).validate(specs)
    tensors["lm_head.weight"] = torch.zeros(40, 32).bfloat16()
    write_safetensors(str(tmp_path / "model.safetensors"), tensors)
    WeightStore(str(tmp_path)).validate(specs)
    # it is checked and not uploaded: the head reads the embedding's table
    loaded = WeightStore(str(tmp_path)).load(specs, torch.bfloat16, "cpu")
    assert "lm_head.weight" not in loaded and "model.embed_tokens.weight" in loaded
    tensors["lm_head.weight"] = torch.zeros(41, 32).bfloat16()
    write_safetensors(str(tmp_path / "model.safetensors"), tensors)
    assert code_of(lambda: WeightStore(str(tmp_path)).validate(specs)).code == ErrorCode.INVALID_SHAPE


def test_matrices_stored_in_32_bit_stay_so_and_say_so(tmp_path):
    """A tensor stored in 32-bit is kept in 32-bit also when the model runs in bfloat16 (its products
    then take the true 32-bit kernel); the loader says so once, since nothing else would show it."""
    import warnings
    config = LlamaConfig.from_dict(TINY)
    specs = expected_tensors(config.to_spec())
    tensors = random_tensors(specs, seed=2)
    name = "model.layers.0.mlp.down_proj.weight"
    tensors[name] = tensors[name].float()
    tensors["model.norm.weight"] = tensors["model.norm.weight"].float()          # a vector: kept wide without a word
    write_safetensors(str(tmp_path / "model.safetensors"), tensors)
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        loaded = WeightStore(str(tmp_path)).load(specs, torch.bfloat16, "cpu")
    assert loaded[name].dtype == torch.float32 and loaded["model.norm.weight"].dtype == torch.float32
    assert loaded["model.layers.0.mlp.up_proj.weight"].dtype == torch.bfloat16
    said = [str(warning.message) for warning in caught if "stored in 32-bit" in str(warning.message)]
    assert len(said) == 1 and "1 matrices" in said[0] and name in said[0], [str(warning.message) for warning in caught]
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        WeightStore(str(tmp_path)).load(specs, torch.float32, "cpu")
    assert not [warning for warning in caught if "stored in 32-bit" in str(warning.message)]


def test_broken_files(tmp_path):
    assert code_of(lambda: WeightStore(str(tmp_path))).code == ErrorCode.IO
    path = str(tmp_path / "model.safetensors")
    write_safetensors(path, {"w": torch.randn(4, 4)})
    raw = pathlib.Path(path).read_bytes()
    pathlib.Path(path).write_bytes(raw[:-5])                                   # truncated (tests/unit_tests.cpp:166-170)
    assert code_of(lambda: WeightStore(str(tmp_path))).code == ErrorCode.INVALID_FORMAT
    pathlib.Path(path).write_bytes(raw + b"\0\0\0\0")                          # trailing bytes
    assert code_of(lambda: WeightStore(str(tmp_path))).code == ErrorCode.INVALID_FORMAT
    pathlib.Path(path).write_bytes(raw[:4])
    assert code_of(lambda: WeightStore(str(tmp_path))).code == ErrorCode.INVALID_FORMAT

    def with_header(header, payload=b"\0" * 64):
        text = json.dumps(header).encode()
        pathlib.Path(path).write_bytes(struct.pack("<Q", len(text)) + text + payload)
    with_header({"w": {"dtype": "F32", "shape": [4, 4], "data_offsets": [0, 60]}})          # bytes do not fit the shape
    assert code_of(lambda: WeightStore(str(tmp_path))).code == ErrorCode.INVALID_SHAPE
    with_header({"w": {"dtype": "F8_E4M3", "shape": [64], "data_offsets": [0, 64]}})
    assert code_of(lambda: WeightStore(str(tmp_path))).code == ErrorCode.INVALID_DTYPE
    with_header({"w": {"dtype": "F32", "shape": [8], "data_offsets": [0, 32]}, "v": {"dtype": "F32", "shape": [8], "data_offsets": [16, 48]}})
    assert code_of(lambda: WeightStore(str(tmp_path))).code == ErrorCode.INVALID_FORMAT     # overlap
    text = b'{"w": {"dtype": "F32", "shape": [8], "data_offsets": [0, 32]}, "w": {"dtype": "F32", "shape": [8], "data_offsets": [32, 64]}}'
    pathlib.Path(path).write_bytes(struct.pack("<Q", len(text)) + text + b"\0" * 64)
    assert code_of(lambda: WeightStore(str(tmp_path))).code == ErrorCode.INVALID_FORMAT     # duplicate name
    pathlib.Path(path).write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    assert code_of(lambda: WeightStore(str(tmp_path))).code == ErrorCode.INVALID_FORMAT


def test_sharded_folder(tmp_path):
    config = LlamaConfig.from_dict(TINY)
    specs = expected_tensors(config.to_spec())
    tensors = random_tensors(specs, seed=1)
    names = sorted(tensors)
    half = len(names) // 2
    write_safetensors(str(tmp_path / "model-00001-of-00002.safetensors"), {n: tensors[n] for n in names[:half]})
    write_safetensors(str(tmp_path / "model-00002-of-00002.safetensors"), {n: tensors[n] for n in names[half:]})
    weight_map = {n: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors") for i, n in enumerate(names)}
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map}))
    loaded = WeightStore(str(tmp_path)).load(specs, torch.float32, "cpu")
    assert all(torch.equal(loaded[n], tensors[n].float()) for n in names)


def test_checksum_of_the_weight_file(tmp_path):
    """The reference checks its weights against a pinned digest (`checksum_mismatch`,
    tests/unit_tests.cpp:150-160); here the digest is the caller's to name."""
    import hashlib
    from tlie_amd import EngineError, LlamaConfig, write_random_model
    from tlie_amd.weights import WeightStore
    raw = dict(model_type="llama", hidden_size=32, intermediate_size=48, num_hidden_layers=1, num_attention_heads=2,
               num_key_value_heads=1, max_position_embeddings=32, vocab_size=40, rms_norm_eps=1e-5)
    write_random_model(str(tmp_path), LlamaConfig.from_dict(raw), seed=1)
    with open(tmp_path / "model.safetensors", "rb") as handle:
        digest = hashlib.sha256(handle.read()).hexdigest()
    store = WeightStore(str(tmp_path))
    assert store.sha256() == digest
    store.expect_sha256(digest.upper() + "\n")
    with pytest.raises(EngineError) as caught:
        store.expect_sha256("0" * 64)
    assert caught.value.code.value == "checksum_mismatch"


def test_a_byte_budget_refuses_the_weight_files_before_mapping(tmp_path):
    """src/weight_store.cpp:134-138: a file beyond the configured budget is out_of_memory."""
    import os
    config = LlamaConfig.from_dict(TINY)
    specs = expected_tensors(config.to_spec())
    write_safetensors(str(tmp_path / "model.safetensors"), random_tensors(specs, seed=3))
    size = os.path.getsize(tmp_path / "model.safetensors")
    WeightStore(str(tmp_path), max_file_bytes=size).validate(specs)
    error = code_of(lambda: WeightStore(str(tmp_path), max_file_bytes=size - 1))
    assert error.code == ErrorCode.OUT_OF_MEMORY and "budget" in error.message


def test_the_arena_hands_out_aligned_places_and_says_when_it_is_full():
    from tlie_amd.weights import WeightArena
    arena = WeightArena(1000, "cpu")
    assert arena.capacity == 1024
    a = arena.place(torch.arange(10, dtype=torch.float32))                  # 40 bytes: one place of 256
    b = arena.place(torch.arange(190, dtype=torch.int32).view(10, 19))      # 760 bytes: three more, the arena is full
    assert a.data_ptr() % 256 == 0 and b.data_ptr() == a.data_ptr() + 256 and arena.used == 1024
    assert torch.equal(a, torch.arange(10, dtype=torch.float32)) and torch.equal(b, torch.arange(190, dtype=torch.int32).view(10, 19))
    assert arena.holds(a) and arena.holds(b[3:]) and arena.place(b) is b and arena.used == 1024
    late = torch.ones(3)
    assert arena.place(late) is late and not arena.holds(late) and arena.outside == 12     # it stays where it is, and is counted


def test_resident_weights_bring_a_tensor_when_asked_and_remember_what_was_kept_whole():
    from tlie_amd.weights import ResidentWeights, keep_in
    calls = []

    def make(name, values):
        def fetch():
            calls.append(name)
            return torch.tensor(values, dtype=torch.float32)
        return fetch
    weights = ResidentWeights({"a": make("a", [1.0, 2.0]), "b": make("b", [3.0]), "c": make("c", [4.0, 5.0, 6.0])},
                              {"a": 8, "b": 4, "c": 12}, "cpu")
    assert weights.arena.capacity == 3 * 256 and set(weights) == {"a", "b", "c"} and "a" in weights and "z" not in weights
    assert calls == []                                                     # nothing is brought before it is asked for
    assert weights["a"] is weights["a"] and calls == ["a"]                 # and once while the part loads
    fused = weights.keep(torch.cat([weights["a"], weights["b"]]))          # a part fuses two and keeps the result
    assert weights.arena.holds(fused) and fused.tolist() == [1.0, 2.0, 3.0]
    whole = weights.keep(weights["c"])                                     # another keeps one as it came
    weights.release()
    assert weights["c"] is whole and calls == ["a", "b", "c"]              # that one is known by its name from then on
    assert weights["a"].tolist() == [1.0, 2.0] and calls == ["a", "b", "c", "a"]      # a fused one is brought again
    assert weights.get("z") is None and code_of(lambda: weights["z"]).code == ErrorCode.INVALID_SHAPE
    plain = {"a": torch.ones(2)}
    assert keep_in(plain, plain["a"]) is plain["a"] and keep_in(weights, whole) is whole


def test_a_model_loaded_through_resident_weights_lies_in_one_allocation(tmp_path):
    """On the CPU (loading launches no kernel): every matrix and norm weight of the model has its place
    in the arena, a tied head shares the table's, each stored tensor is read once, and the values are
    those of a model loaded from a dict."""
    from tlie_amd.models import build_model
    raw = dict(TINY, tie_word_embeddings=True, attention_bias=True)
    config = LlamaConfig.from_dict(raw)
    write_random_model(str(tmp_path), config, seed=9)
    spec = config.to_spec()
    store = WeightStore(str(tmp_path))
    reads = []
    get = store.get
    store.get = lambda name: (reads.append(name), get(name))[1]
    weights = store.resident(expected_tensors(spec), torch.bfloat16, "cpu")
    model = build_model(spec, weights, torch.bfloat16, "cpu")
    arena = weights.arena
    kept = [model.embedding.table, model.final_norm.weight, model.head.linear.weight]
    for block in model.blocks:
        kept += [block.mixer.qkv.weight, block.mixer.qkv.bias, block.mixer.o.weight, block.mixer.o.bias,
                 block.feed_forward.gate_up.weight, block.feed_forward.down.weight, block.mixer_norm.weight, block.feed_forward_norm.weight]
    assert all(arena.holds(tensor) and tensor.data_ptr() % 256 == 0 for tensor in kept) and arena.outside == 0
    assert model.head.linear.weight.data_ptr() == model.embedding.table.data_ptr()
    assert sorted(reads) == sorted(spec.name for spec in expected_tensors(spec) if not spec.optional)     # each once
    assert arena.used <= arena.capacity and not weights._fresh
    eager = build_model(spec, WeightStore(str(tmp_path)).load(expected_tensors(spec), torch.bfloat16, "cpu"), torch.bfloat16, "cpu")
    for mine, theirs in zip(model.blocks, eager.blocks):
        assert torch.equal(mine.mixer.qkv.weight, theirs.mixer.qkv.weight) and torch.equal(mine.feed_forward.gate_up.weight, theirs.feed_forward.gate_up.weight)
        assert torch.equal(mine.mixer.qkv.bias, theirs.mixer.qkv.bias) and torch.equal(mine.feed_forward.down.weight, theirs.feed_forward.down.weight)
    assert torch.equal(model.embedding.table, eager.embedding.table)
