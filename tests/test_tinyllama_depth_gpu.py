"""TinyLlama 1.1B at its own sizes and all of its 22 layers, random weights: the logits of a request
do not depend on how its tokens are cut into steps or on what else is in the batch, in 32-bit and
in bfloat16, and they are the plain implementation's.

reference: its integration test runs the real checkpoint through the whole model and compares
with stored logits (tests/m1_integration_tests.cpp:106-152, scripts/export_golden.py:73-107); the
checkpoint is not here, so the weights are random (standard deviation 0.02, stored in bfloat16, so
that both precisions and the plain implementation read the same values) and the stored logits are
the float64 plain implementation's.  What the tiny configurations cannot show is here: the growth
of rounding over 22 layers, 22 cache pools behind one block table, recordings of more than a
hundred kernels.

Tolerances.  32-bit: those of the tiny configurations (2e-5 against the plain implementation, 1e-6
between two cuts).  bfloat16: the tiny configurations' 1.5e-2 is what two or three layers of 16-bit
storage cost; what 22 layers cost is measured here, not guessed: the plain implementation is run
once more with every activation that a 16-bit path keeps in memory rounded to bfloat16
(`stored_as`), all sums still float64, and its distance from the unrounded logits (on this model
2.2e-2 of a row's scale at worst, 1.7e-2 at the median row) is the yardstick: the engine may be a
quarter worse than that, at the worst row and at the median row, and two cuts may differ by twice
the yardstick.
"""
import json
import os

import pytest
import torch

from gpu_helpers import CUT_TOLERANCE, TOLERANCE, Replayer, _row_errors, assert_close, random_tokens
from plain_llama import plain_forward, stored_as

pytestmark = pytest.mark.gpu

TINYLLAMA = dict(model_type="llama", architectures=["LlamaForCausalLM"], hidden_size=2048, intermediate_size=5632,
                 num_hidden_layers=22, num_attention_heads=32, num_key_value_heads=4, max_position_embeddings=2048,
                 vocab_size=32000, rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=False, attention_bias=False,
                 hidden_act="silu", bos_token_id=1, eos_token_id=2)
LONG, SHORT = 128, 48


class StoredWeights:
    """The folder's tensors as the plain implementation reads them, widened to float64 one at a
    time (all 1.1e9 values at once would be 9 GB)."""

    def __init__(self, path):
        from safetensors import safe_open
        self.file = safe_open(path, "pt")
        self.names = set(self.file.keys())

    def __getitem__(self, name):
        return self.file.get_tensor(name).double()

    def __contains__(self, name):
        return name in self.names

    def get(self, name, default=None):
        return self[name] if name in self.names else default


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    from tlie_amd import write_random_model
    from tlie_amd.registry import config_from_dict
    folder = str(tmp_path_factory.mktemp("tinyllama_22_layers"))
    print("writing 1.1e9 random weights ...", flush=True)
    write_random_model(folder, config_from_dict(TINYLLAMA), seed=22, std=0.02, norm_std=0.1, dtype=torch.bfloat16)
    with open(os.path.join(folder, "config.json"), "r", encoding="utf-8") as handle:
        raw = json.load(handle)
    weights = StoredWeights(os.path.join(folder, "model.safetensors"))
    streams = {"long": random_tokens(1, LONG, 32000), "short": random_tokens(2, SHORT, 32000)}
    print("the plain implementation, 22 layers in float64 ...", flush=True)
    want = {name: plain_forward(raw, weights, tokens) for name, tokens in streams.items()}
    print("and once more with activations stored in bfloat16 ...", flush=True)
    errors, scales = _row_errors(plain_forward(raw, weights, streams["long"], stored=stored_as(torch.bfloat16)), want["long"])
    yardstick = {"worst": float((errors / scales).max()), "median": float((errors / scales).median())}
    print(f"16-bit storage alone: {yardstick}", flush=True)
    assert 5e-3 < yardstick["median"] < yardstick["worst"] < 4e-2, yardstick
    return folder, streams, want, yardstick


def assert_within_yardstick(got, want, yardstick, what):
    errors, scales = _row_errors(got, want)
    relative = errors / scales
    worst, median = float(relative.max()), float(relative.median())
    assert worst <= 1.25 * yardstick["worst"] and median <= 1.25 * yardstick["median"], \
        f"{what}: worst row {worst:.3e}, median row {median:.3e}; 16-bit storage alone costs {yardstick}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_all_22_layers_under_every_cut(model, dtype):
    from tlie_amd import Engine
    folder, streams, want, yardstick = model
    long, short = streams["long"], streams["short"]
    cut_tolerance = CUT_TOLERANCE[dtype] if dtype == "float32" else 2 * yardstick["worst"]

    def against_plain(got, wanted, what):
        if dtype == "float32":
            assert_close(got, wanted, TOLERANCE[dtype], what)
        else:
            assert_within_yardstick(got, wanted, yardstick, what)
    # 13 pages of 16 positions: the long request's 8 and one short request's 3 fit, a second short one
    # only on pages that another has given back
    engine = Engine(folder, dtype=dtype, max_tokens=LONG + SHORT + 32, page_size=16, max_requests=4)
    assert len(engine.cache.bindings) == 22 and len(engine.cache.groups) == 1 and engine.cache.num_pages == 13
    replay = Replayer(engine)
    every = list(range(LONG))
    print(f"{dtype}: whole", flush=True)
    replay.step([("whole", long, every)], end=["whole"])
    whole = replay.logits_of("whole", every)
    against_plain(whole, want["long"], "whole, against the plain implementation")

    print(f"{dtype}: the last 32 one by one", flush=True)
    replay.step([("tail", long[:LONG - 32], list(range(LONG - 32)))])
    for place in range(LONG - 32, LONG):
        replay.step([("tail", long[place:place + 1], [0])])
    engine.finish("tail")
    assert_close(replay.logits_of("tail", every), whole, cut_tolerance, "the last 32 one by one, against whole")

    print(f"{dtype}: portions of changing size", flush=True)
    cursor = 0
    for size in (2, 31, 5, 48, 3, 17, 2, 4, 16):
        replay.step([("cut", long[cursor:cursor + size], list(range(size)))])
        cursor += size
    assert cursor == LONG
    engine.finish("cut")
    assert_close(replay.logits_of("cut", every), whole, cut_tolerance, "portions of changing size, against whole")

    print(f"{dtype}: mixed with other requests on pages that are used again", flush=True)
    pages_seen = {}

    def note(request):
        pages_seen[request] = set(engine.cache.page_list(request, 0))
    replay.step([("m", long[:20], list(range(20))), ("s1", short[:30], list(range(30)))])
    replay.step([("m", long[20:22], [0, 1]), ("s1", short[30:31], [0])])
    replay.step([("s1", short[31:], list(range(SHORT - 31))), ("m", long[22:23], [0])])
    note("s1")
    engine.finish("s1")
    replay.step([("m", long[23:60], list(range(37))), ("s2", short[:2], [0, 1])])
    for place in range(2, 12):                                      # two requests decode beside a third's portions
        items = [("s2", short[place:place + 1], [0]), ("m", long[58 + place:59 + place], [0])]
        if place == 4:
            items.append(("s3", short[:9], list(range(9))))
        replay.step(items)
    replay.step([("s3", short[9:], list(range(SHORT - 9))), ("s2", short[12:], list(range(SHORT - 12))),
                 ("m", long[70:72], [0, 1])])
    note("s2")
    note("s3")
    engine.finish("s2")
    engine.finish("s3")
    replay.step([("m", long[72:], list(range(LONG - 72))), ("s4", short, list(range(SHORT)))])
    note("m")
    note("s4")
    engine.finish("m")
    engine.finish("s4")
    # the five requests held 20 pages between them, the pool has 13: some were used again
    assert sum(len(pages) for pages in pages_seen.values()) == 20 > engine.cache.num_pages
    assert_close(replay.logits_of("m", every), whole, cut_tolerance, "mixed, against whole")
    against_plain(replay.logits_of("m", every), want["long"], "mixed, against the plain implementation")
    for request in ("s1", "s2", "s3", "s4"):
        against_plain(replay.logits_of(request, range(SHORT)), want["short"], f"{request}, against the plain implementation")
    assert engine.cache.free_pages() == [13]
