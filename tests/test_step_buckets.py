"""Which steps a recording serves, and at which padded sizes: decided on the host, tested without a GPU."""
from types import SimpleNamespace

import torch

from tlie_amd.engine.step import DecodeGraph, ModelRunner, PortionGraph, StepEntry


def runner():
    model = SimpleNamespace(device="cpu", spec=SimpleNamespace(vocab_size=100), graph_safe=True, dtype=torch.bfloat16)
    made = ModelRunner(model, cache=None)
    assert not made.use_graphs              # no recordings without a GPU
    made.use_graphs = True                  # (the decisions below do not touch the device)
    return made


def entries(counts, wants=None):
    wants = wants or [[count - 1] for count in counts]
    return [StepEntry(index, [1] * count, want) for index, (count, want) in enumerate(zip(counts, wants))]


def test_single_tokens_with_every_logit_wanted_replay_a_decode_recording():
    made = runner()
    assert made.replays(entries([1] * 5)) and made.replays(entries([1] * DecodeGraph.MAX_BATCH))
    assert not made.replays(entries([1] * (DecodeGraph.MAX_BATCH + 1)))
    assert not made.replays(entries([1, 2, 1])) and not made.replays(entries([1, 1], [[0], []]))
    assert [DecodeGraph.bucket_of(count) for count in (1, 2, 3, 9, 64, 65, 200)] == [1, 2, 4, 16, 64, 128, 256]


def test_portions_are_padded_to_the_recordings_sizes():
    made = runner()
    assert made.records(entries([5, 3])) == (16, 8)
    assert made.records(entries([16, 1])) == (32, 8)
    assert made.records(entries([33])) == (64, 8)
    assert made.records(entries([64, 1])) == (128, 8)
    assert made.records(entries([500, 12])) == (512, 8)
    assert made.records(entries([2] * 9)) == (32, 32)            # more than 8 sequences: up to 64, and no more than tokens
    assert made.records(entries([30] * 9)) == (320, 64)
    assert made.records(entries([1, 1], [[0], []])) == (16, 8)   # single tokens of which one is not wanted


def test_what_no_recording_serves():
    made = runner()
    assert made.records(entries([PortionGraph.MAX_TOKENS + 1])) is None
    assert made.records(entries([1] * (PortionGraph.MAX_SEQS + 1), [[] for _ in range(PortionGraph.MAX_SEQS + 1)])) is None
    assert made.records(entries([20], [list(range(20))])) is None               # more wanted rows than sequences
    assert made.records(entries([20, 20], [list(range(8)), [0]])) is None
    assert made.records(entries([20], [list(range(8))])) == (32, 8)
    assert made.records([StepEntry(0, [0], [0], source=3), StepEntry(1, [1, 2], [1])]) is None
    made.use_graphs = False
    assert made.records(entries([5, 3])) is None and not made.replays(entries([1]))
