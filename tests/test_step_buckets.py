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


def test_the_skinny_products_launch_shape_is_one_the_kernel_takes():
    """Decided on the host from the sizes alone: every plan is within what the kernel takes, covers
    the inner size exactly, and for matrices that the policy balances the workgroups are no more
    than the compute units (one round) unless a round more is cheaper than more splits."""
    from tlie_amd import ops
    for rows in (1, 16, 17, 32, 33, 64):
        for out_features, in_features in ((2560, 2048), (2048, 2048), (11264, 2048), (2048, 5632), (32000, 2048), (100, 520),
                                          (515, 1000), (64, 5632), (12288, 4096), (28672, 4096), (4096, 14336), (7, 8)):
            for units in (256, 304, 64):
                split_len, waves, strips = ops.skinny_plan(rows, out_features, in_features, units)
                assert split_len > 0 and split_len % 64 == 0 and 4 <= waves <= 16 and strips in (1, 2)
                assert strips == 1 or (rows > 32 and waves <= 8)
                nsplit = -(-in_features // split_len)
                assert (nsplit - 1) * split_len < in_features <= nsplit * split_len
                assert ops.skinny_plan(rows, out_features, in_features, units) == (split_len, waves, strips)    # (kept)
    # TinyLlama's four matrices at 64 rows on 256 compute units: one round of workgroups
    for out_features, in_features in ((2560, 2048), (2048, 2048), (11264, 2048), (2048, 5632)):
        split_len, waves, strips = ops.skinny_plan(64, out_features, in_features, 256)
        workgroups = -(-out_features // (16 * waves * strips)) * -(-in_features // split_len)
        assert 128 < workgroups <= 256, (out_features, in_features, split_len, waves, strips)


def test_the_few_rows_products_launch_shape_is_one_the_kernel_takes():
    """Decided on the host from the sizes alone: waves 4, 8 or 16; an even number of rows of W a
    workgroup up to 16, or 32 with at most 8 waves; the gated product never an odd pairing."""
    from tlie_amd import ops
    for rows in (1, 2, 7, 8, 16):
        for out_features, in_features in ((2560, 2048), (2048, 2048), (11264, 2048), (2048, 5632), (32000, 2048), (6144, 4096),
                                          (28672, 4096), (4096, 14336), (128256, 4096), (100, 520), (30, 64), (2112, 2048)):
            for epilogue in ("store", "rope", "silu", "residual"):
                for units in (256, 304, 64):
                    waves, rows_per_block = ops.gemm_rows_shape(out_features, in_features, epilogue, units, rows)
                    assert waves in (4, 8, 16)
                    assert (rows_per_block % 2 == 0 and 2 <= rows_per_block <= 16) or (rows_per_block == 32 and waves <= 8)
    assert ops.gemm_rows_shape(2560, 2048, "rope", 256, 8) == (16, 10)          # 256 workgroups, one a compute unit
    assert ops.gemm_rows_shape(2048, 2048, "residual", 256, 8) == (16, 16)      # a norm's sums follow: strips of 16
    assert ops.gemm_rows_shape(128256, 4096, "store", 256, 1) == (4, 16) and ops.gemm_rows_shape(128256, 4096, "store", 256, 8) == (4, 32)
