"""The sampling kernel against the plain sampler's distribution."""
import pytest
import torch

from plain_llama import plain_greedy, plain_top_p_distribution

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_greedy_first_maximum_and_non_finite():
    from tlie_amd import ops
    logits = torch.tensor([[1.0, 3.0, 3.0, 2.0]], device=DEV)            # tests/unit_tests.cpp:198-207 -> 1
    assert ops.sample(logits).tolist() == [1]
    torch.manual_seed(0)
    big = torch.randn(5, 32003)
    big[2, 31999] = big[2, 77] = 9.0
    big[3, 5] = float("nan")
    big[4, 9] = float("inf")
    got = ops.sample(big.to(DEV)).tolist()
    assert got[:3] == [plain_greedy(big[i]) for i in range(3)] and got[2] == 77
    assert got[3] == -1 and got[4] == -1                                  # src/operators.cpp:170-172: NaN or Inf is an error


def test_sampler_raises_on_non_finite():
    from tlie_amd import EngineError, ErrorCode
    from tlie_amd.engine import SamplingParams
    from tlie_amd.sampling import Sampler
    logits = torch.tensor([[0.0, float("nan")]], device=DEV)
    with pytest.raises(EngineError) as caught:
        Sampler(DEV).sample(logits, [SamplingParams()], [0])
    assert caught.value.code == ErrorCode.NUMERICAL


@pytest.mark.parametrize("vocab,temperature,top_p", [(50, 1.0, 1.0), (1000, 0.8, 0.9), (517, 1.5, 0.5), (32000, 0.7, 0.95)])
def test_draws_follow_the_plain_distribution(vocab, temperature, top_p):
    """The token drawn for (seed, counter) is the one the plain distribution gives for the same
    uniform number when the kept tokens are walked in index order; and over many counters the
    frequencies follow the distribution."""
    from tlie_amd import ops
    from tlie_amd.sampling import uniform01
    torch.manual_seed(vocab)
    logits = torch.randn(vocab) * 2.0
    distribution = plain_top_p_distribution(logits, temperature, top_p)
    cumulative = torch.cumsum(distribution, 0)
    draws = 400
    rows = logits.to(DEV).repeat(draws, 1).contiguous()
    got = ops.sample(rows, torch.full((draws,), temperature, device=DEV), torch.full((draws,), top_p, device=DEV),
                     torch.full((draws,), 1234, dtype=torch.int64, device=DEV),
                     torch.arange(draws, dtype=torch.int64, device=DEV)).tolist()
    mismatches = 0
    for counter, token in enumerate(got):
        assert distribution[token] > 0, f"token {token} is outside the kept set"
        u = uniform01(1234, counter)
        want = int(torch.searchsorted(cumulative, torch.tensor(u, dtype=torch.float64)).item())
        want = min(want, vocab - 1)
        if token != want:
            # float32 sums on the device against float64 here: only a draw within rounding of a boundary may differ
            edge = min(abs(u - cumulative[token].item()), abs(u - (cumulative[token] - distribution[token]).item()))
            assert edge < 1e-4, f"counter {counter}: drew {token}, the plain walk gives {want}"
            mismatches += 1
    assert mismatches <= 4
    # same (seed, counter) -> same token, whatever else is in the batch
    again = ops.sample(rows[:7].contiguous(), torch.full((7,), temperature, device=DEV), torch.full((7,), top_p, device=DEV),
                       torch.full((7,), 1234, dtype=torch.int64, device=DEV),
                       torch.tensor([5, 0, 399, 17, 17, 3, 1], dtype=torch.int64, device=DEV)).tolist()
    assert again == [got[5], got[0], got[399], got[17], got[17], got[3], got[1]]
    other_seed = ops.sample(rows, torch.full((draws,), temperature, device=DEV), torch.full((draws,), top_p, device=DEV),
                            torch.full((draws,), 99, dtype=torch.int64, device=DEV),
                            torch.arange(draws, dtype=torch.int64, device=DEV)).tolist()
    assert other_seed != got


def test_limits_of_temperature_and_top_p():
    from tlie_amd import ops
    torch.manual_seed(2)
    logits = torch.randn(64, 300).to(DEV)
    greedy = ops.sample(logits).tolist()
    n = logits.shape[0]
    seeds = torch.arange(n, dtype=torch.int64, device=DEV)
    cold = ops.sample(logits, torch.full((n,), 1e-3, device=DEV), torch.ones(n, device=DEV), seeds, seeds).tolist()
    assert cold == greedy                                                # T -> 0+ is greedy
    narrow = ops.sample(logits, torch.ones(n, device=DEV), torch.full((n,), 1e-6, device=DEV), seeds, seeds).tolist()
    assert narrow == greedy                                              # a tiny top_p keeps the best token only
    zero_t = ops.sample(logits, torch.zeros(n, device=DEV), torch.full((n,), 0.5, device=DEV), seeds, seeds).tolist()
    assert zero_t == greedy                                              # temperature <= 0 is greedy (app/server.cpp:238-241)
    mixed_t = torch.ones(n, device=DEV)
    mixed_t[::2] = 0.0
    mixed = ops.sample(logits, mixed_t, torch.ones(n, device=DEV), seeds, seeds).tolist()
    assert mixed[::2] == greedy[::2]
