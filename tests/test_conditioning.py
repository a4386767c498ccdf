"""Why the random configurations of the GPU tests scale their weights with the width.

A drawn configuration of width 1920 (15 heads on 3 key heads, head size 128, three layers) with
weights of standard deviation 0.08 once made a bfloat16 engine sample a token whose plain logit lay
7.2% of the row's scale below the best.  This test shows on the CPU, with the plain implementation
alone, that such a model's own float64 logits move by more than that when every weight moves by
half a bfloat16 step (what one rounding does), and that the same configuration with weights scaled
as real checkpoints' are (0.5 / sqrt(width)) does not: the draw was ill-conditioned, the engine's
deviation there was no fault of its kernels, and the scaled draws are a fair test.
"""
import random

import torch

from plain_llama import plain_forward
from tlie_amd.models.builder import expected_tensors
from tlie_amd.registry import config_from_dict
from tlie_amd.weights import random_tensors

WIDE_DRAW = dict(model_type="llama", architectures=["LlamaForCausalLM"], hidden_size=1920, intermediate_size=256,
                 num_hidden_layers=3, num_attention_heads=15, num_key_value_heads=3, head_dim=128, max_position_embeddings=96,
                 vocab_size=1000, rms_norm_eps=1e-6, rope_theta=500000.0, tie_word_embeddings=False, attention_bias=False,
                 hidden_act="silu", bos_token_id=1, eos_token_id=2)
ENGINE_DEVIATION = 0.072      # of the row's scale: what the bfloat16 engine showed on this draw with std 0.08


def moved_by_half_a_step(weights, generator):
    """Every weight moved up or down, at random, by half the distance to its bfloat16 neighbour."""
    out = {}
    for name, tensor in weights.items():
        step = torch.pow(2.0, torch.floor(torch.log2(tensor.abs().clamp(min=1e-30))) - 7)
        sign = (torch.randint(0, 2, tensor.shape, generator=generator) * 2 - 1).double()
        out[name] = tensor + 0.5 * sign * step
    return out


def logit_movement(std):
    specs = expected_tensors(config_from_dict(WIDE_DRAW).to_spec())
    weights = {name: tensor.double() for name, tensor in random_tensors(specs, 68, std=std, norm_std=0.1, dtype=torch.bfloat16).items()}
    rng = random.Random(5)
    tokens = [rng.randrange(WIDE_DRAW["vocab_size"]) for _ in range(48)]
    want = plain_forward(WIDE_DRAW, weights, tokens)
    got = plain_forward(WIDE_DRAW, moved_by_half_a_step(weights, torch.Generator().manual_seed(1)), tokens)
    moved = (got - want).abs().amax(dim=-1) / want.abs().amax(dim=-1)
    return float(moved.median()), float(moved.max()), int((got.argmax(-1) != want.argmax(-1)).sum())


def test_the_wide_draw_with_large_weights_is_ill_conditioned_and_the_scaled_one_is_not():
    median, worst, flipped = logit_movement(0.08)
    assert median > ENGINE_DEVIATION and worst > 2 * ENGINE_DEVIATION, (median, worst)
    assert flipped >= 5                               # the best token itself changes on many rows
    median, worst, flipped = logit_movement(0.5 / 1920 ** 0.5)
    assert worst < 1e-2 and flipped == 0, (median, worst, flipped)
