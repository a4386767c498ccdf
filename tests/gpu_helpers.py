"""What the GPU tests share: the two tiny configurations, model folders of random weights in a
temporary place, the plain implementation's logits for a token list, and tolerances."""
import json
import os
import random

import torch
from safetensors.torch import load_file

from plain_llama import plain_forward

# Two tiny configurations that differ in every size and option: layers, width, heads and groups
# (4 on 2, 3 on 1), head size (16, 32), feed-forward width (176 is no multiple of 64), vocabulary,
# theta, eps, positions, tied or not, bias or not.
CONFIG_A = dict(model_type="llama", architectures=["LlamaForCausalLM"], hidden_size=64, intermediate_size=176,
                num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=128,
                vocab_size=256, rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=False, attention_bias=False,
                hidden_act="silu", bos_token_id=1, eos_token_id=2)
CONFIG_B = dict(model_type="llama", architectures=["LlamaForCausalLM"], hidden_size=96, intermediate_size=256,
                num_hidden_layers=3, num_attention_heads=3, num_key_value_heads=1, head_dim=32,
                max_position_embeddings=256, vocab_size=512, rms_norm_eps=1e-6, rope_theta=500000.0,
                tie_word_embeddings=True, attention_bias=True, hidden_act="silu", bos_token_id=1, eos_token_id=2)
CONFIGS = {"A": CONFIG_A, "B": CONFIG_B}
DTYPES = ["float32", "bfloat16"]

# Differences from the plain implementation (float64 on the same stored weights), row by row: a
# row's largest error relative to the row's largest value (a row of small logits is held to its
# own size, not to the largest logit of the whole comparison).  float32: rounding of 32-bit sums
# over at most a few hundred terms.  bfloat16: activations between kernels are rounded to 8 bits of
# mantissa (2^-9 relative each); a few dozen such roundings per token pile up to about a percent.
TOLERANCE = {"float32": 2e-5, "bfloat16": 1.5e-2}
# Two ways of cutting the same request through the same engine differ by less: float32 sums run
# in the same order whatever the cut; bfloat16 may take another kernel for one token than for many
# (and a step that is replayed from a recording must equal the same step launched kernel by kernel
# bit for bit: the tests that compare those two use torch.equal, not a tolerance).  Two bfloat16
# results that each lie within 1.5e-2 of the truth lie within twice that of each other; measured: 1.6e-2.
CUT_TOLERANCE = {"float32": 1e-6, "bfloat16": 2.5e-2}


def make_model(folder, raw_config, seed, dtype_name, std=0.08, norm_std=0.1):
    from tlie_amd import write_random_model
    from tlie_amd.registry import config_from_dict
    config = config_from_dict(raw_config)
    stored = torch.float32 if dtype_name == "float32" else torch.bfloat16
    write_random_model(str(folder), config, seed, std=std, norm_std=norm_std, dtype=stored)
    return str(folder)


def load_plain(folder):
    """The folder as the plain implementation reads it: config dict and float64 weights, through
    the safetensors library (not the engine's reader)."""
    with open(os.path.join(folder, "config.json"), "r", encoding="utf-8") as handle:
        raw = json.load(handle)
    weights = {name: tensor.double() for name, tensor in load_file(os.path.join(folder, "model.safetensors")).items()}
    return raw, weights


def random_tokens(seed, count, vocab):
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(count)]


def _row_errors(got, want):
    """Per row (everything but the last dimension): the largest error and the largest wanted value."""
    got, want = got.double().cpu(), want.double().cpu()
    assert got.shape == want.shape, (got.shape, want.shape)
    if got.dim() < 2:
        got, want = got.reshape(1, -1), want.reshape(1, -1)
    got, want = got.reshape(-1, got.shape[-1]), want.reshape(-1, want.shape[-1])
    return (got - want).abs().amax(dim=-1), want.abs().amax(dim=-1)


def close(got, want, tolerance):
    """Every row: max |got - want| <= tolerance * max |want| of that row; returns (ok, the worst
    row's error, that row's scale)."""
    errors, scales = _row_errors(got, want)
    excess = errors - tolerance * scales
    worst = int(excess.argmax())
    return bool((excess <= 0).all()), errors[worst].item(), scales[worst].item()


def assert_close(got, want, tolerance, what=""):
    ok, error, scale = close(got, want, tolerance)
    assert ok, f"{what}: a row's max error {error:.3e} against its scale {scale:.3e} exceeds {tolerance:.1e} relative"


def first_bad_row(got, want, tolerance):
    """Index of the first row whose error exceeds the tolerance (relative to that row's largest
    wanted value), for messages."""
    errors, scales = _row_errors(got, want)
    rows = (errors > tolerance * scales).nonzero().flatten().tolist()
    return rows[0] if rows else None


class Replayer:
    """Drives an engine as the replay program does and keeps every wanted row by
    (request, position)."""

    def __init__(self, engine):
        self.engine = engine
        self.rows = {}

    def step(self, items, end=()):
        from tlie_amd import StepEntry
        entries = []
        for request, tokens, want in items:
            if not self.engine.cache.is_live(request):
                self.engine.admit(request)
            entries.append((request, self.engine.cache.length(request), StepEntry(request, tokens, want)))
        logits = self.engine.step([entry for _, _, entry in entries]).float().cpu()
        cursor = 0
        for request, start, entry in entries:
            for place in entry.want:
                self.rows[(request, start + place)] = logits[cursor]
                cursor += 1
        assert cursor == logits.shape[0]
        for request in end:
            self.engine.finish(request)
        self.engine.cache.check()

    def logits_of(self, request, positions):
        return torch.stack([self.rows[(request, position)] for position in positions])
