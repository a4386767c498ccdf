"""The engine on the GPU against the plain implementation: every way of cutting the work, in
32-bit and in bfloat16, for both tiny configurations."""
import json
import os
import random
import subprocess
import sys

import pytest
import torch

from gpu_helpers import (CONFIGS, CUT_TOLERANCE, DTYPES, TOLERANCE, Replayer, _row_errors, assert_close, first_bad_row, load_plain,
                         make_model, random_tokens)
from plain_llama import plain_forward, plain_generate_greedy, stored_as
from tlie_amd import ops

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CASES = [(name, dtype) for name in CONFIGS for dtype in DTYPES]


@pytest.fixture(scope="module")
def setups(tmp_path_factory):
    """Per (configuration, dtype): model folder, plain config and weights, and a cache of plain logits."""
    made = {}

    def get(name, dtype):
        if (name, dtype) not in made:
            folder = make_model(tmp_path_factory.mktemp(f"model_{name}_{dtype}"), CONFIGS[name], seed=11, dtype_name=dtype)
            raw, weights = load_plain(folder)
            made[(name, dtype)] = {"folder": folder, "raw": raw, "weights": weights, "plain": {}}
        return made[(name, dtype)]
    return get


def plain_logits(setup, tokens):
    key = tuple(tokens)
    if key not in setup["plain"]:
        setup["plain"][key] = plain_forward(setup["raw"], setup["weights"], list(tokens))
    return setup["plain"][key]


def new_engine(setup, dtype, max_tokens=512, page_size=16, max_requests=4, use_graphs=True, capture_graphs=True):
    from tlie_amd import Engine
    return Engine(setup["folder"], dtype=dtype, max_tokens=max_tokens, page_size=page_size, max_requests=max_requests,
                  use_graphs=use_graphs, capture_graphs=capture_graphs)


def assert_same_bits(replayed, launched, what):
    """A step replayed from a recording runs the same kernels on the same arrays as the same step,
    padded alike, launched kernel by kernel: the logits must be equal bit for bit (a tolerance
    would let a stale row of a block table or a padding row that leaks pass)."""
    assert set(replayed.rows) == set(launched.rows)
    for key in sorted(replayed.rows, key=str):
        assert torch.equal(replayed.rows[key], launched.rows[key]), f"{what}: the replayed row {key} differs in bits from the launched one"


def request_tokens(name, index, length):
    return random_tokens(1000 * index + length, length, CONFIGS[name]["vocab_size"])


@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_and_alone(setups, name, dtype):
    setup = setups(name, dtype)
    engine = new_engine(setup, dtype)
    for index, length in enumerate((1, 2, 17, 100 if name == "A" else 150)):
        tokens = request_tokens(name, index, length)
        replay = Replayer(engine)
        replay.step([("r", tokens, list(range(length)))], end=["r"])
        got = replay.logits_of("r", range(length))
        want = plain_logits(setup, tokens)
        bad = first_bad_row(got, want, TOLERANCE[dtype])
        assert bad is None, f"{name} {dtype} length {length}: first wrong position {bad}"


@pytest.mark.parametrize("name,dtype", CASES)
def test_named_intermediate_tensors_layer_by_layer(setups, name, dtype):
    """The reference compares its model with a golden layer by layer through a trace of named
    tensors (ModelTrace: src/model.cpp:98-231, tests/m1_integration_tests.cpp:92-128).  A step that
    is given a dict leaves the same names there; each is compared with the plain implementation's,
    so that a fault shows in the first tensor it touches.  A prompt in two portions: the second
    portion's rows are the sequence's later positions."""
    setup = setups(name, dtype)
    engine = new_engine(setup, dtype)
    tokens = request_tokens(name, 3, 45)
    plain = {}
    plain_forward(setup["raw"], setup["weights"], tokens, trace=plain)
    layers = CONFIGS[name]["num_hidden_layers"]
    assert len(plain) == 5 * layers + 3
    from tlie_amd import StepEntry
    engine.admit("t")
    first, second = {}, {}
    engine.step([StepEntry("t", tokens[:28], list(range(28)))], trace=first)
    engine.step([StepEntry("t", tokens[28:], list(range(17)))], trace=second)     # (17: more than the route of few rows takes)
    engine.finish("t")
    assert sorted(first) == sorted(plain) == sorted(second)
    order = ["embedding"] + [f"layer{layer}.{part}" for layer in range(layers)
                             for part in ("input_norm", "attention_output", "post_attention_norm", "mlp_output", "output")] \
        + ["final_norm", "logits"]
    for key in order:
        got = torch.cat([first[key], second[key]]).cpu()
        assert got.dtype == torch.float32 and got.shape == plain[key].shape, key
        assert_close(got, plain[key], TOLERANCE[dtype], key)
    # a step without a dict is not slowed or changed by all this: the same logits
    engine.admit("u")
    again = engine.step([StepEntry("u", tokens, list(range(45)))]).cpu()
    engine.finish("u")
    assert_close(again, torch.cat([first["logits"], second["logits"]]).cpu().double(), CUT_TOLERANCE[dtype], "without a trace")


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_named_intermediate_tensors_on_the_route_of_few_rows(setups, name):
    """A bfloat16 step of at most 16 tokens (what decoding runs) folds the norms into its products
    and lets the products add into the residual themselves; a trace that asks for the serving route
    takes that same route and leaves what still exists there as a tensor: per layer what the mixer and
    the feed-forward added and the layer's output, the embedding and the logits.  Steps of 9, 5, 1 and
    1 tokens after a prompt portion, each name against the plain implementation's rows at those
    positions.  Without that request the same steps leave every name of the reference's trace, and the
    two routes' logits agree within the tolerance of two cuts."""
    setup = setups(name, "bfloat16")
    engine = new_engine(setup, "bfloat16")
    tokens = request_tokens(name, 4, 45)
    plain = {}
    plain_forward(setup["raw"], setup["weights"], tokens, trace=plain)
    # What a tensor in the middle of the model may differ by: the tolerance of the logits, or, where 16-bit
    # storage alone costs more than that, a quarter more than it costs: the plain implementation once more
    # with every stored activation rounded to bfloat16 and all sums still float64 is the yardstick (what the
    # last layer's feed-forward adds is a small difference of large numbers: 1.7e-2 of its rows' scale on
    # configuration B, where the logits' 1.5e-2 had been passed by luck).
    rounded = {}
    plain_forward(setup["raw"], setup["weights"], tokens, trace=rounded, stored=stored_as(torch.bfloat16))

    def allowed(key):
        errors, scales = _row_errors(rounded[key][29:], plain[key][29:])
        return max(TOLERANCE["bfloat16"], 1.25 * float((errors / scales).max()))
    layers = CONFIGS[name]["num_hidden_layers"]
    from tlie_amd import StepEntry
    engine.admit("t")
    engine.step([StepEntry("t", tokens[:29], [])])
    start, traces = 29, []
    for count in (9, 5, 1, 1):
        traces.append({})
        engine.step([StepEntry("t", tokens[start:start + count], list(range(count)))], trace=traces[-1], trace_serving_route=True)
        start += count
    engine.finish("t")
    # by default a traced step of few rows leaves all the names, like any other step
    engine.admit("f")
    engine.step([StepEntry("f", tokens[:29], [])])
    full, start = [], 29
    for count in (9, 5, 1, 1):
        full.append({})
        engine.step([StepEntry("f", tokens[start:start + count], list(range(count)))], trace=full[-1])
        start += count
    engine.finish("f")
    for trace in full:
        assert sorted(trace) == sorted(plain)
    for key in plain:
        assert_close(torch.cat([trace[key] for trace in full]).cpu(), plain[key][29:], allowed(key), "every name: " + key)
    assert_close(torch.cat([trace["logits"] for trace in full]).cpu(), torch.cat([trace["logits"] for trace in traces]).cpu().double(),
                 CUT_TOLERANCE["bfloat16"], "the two routes' logits")
    names = ["embedding"] + [f"layer{layer}.{part}" for layer in range(layers) for part in ("attention_output", "mlp_output", "output")] \
        + ["logits"]
    for trace in traces:
        assert sorted(trace) == sorted(names)          # the normed inputs do not exist on this route
    for key in names:
        got = torch.cat([trace[key] for trace in traces]).cpu()
        assert got.dtype == torch.float32 and got.shape == plain[key][29:].shape, key
        assert_close(got, plain[key][29:], allowed(key), key)
    # the same steps without a trace (replayed from recordings): the same logits up to the cut's tolerance
    engine.admit("u")
    engine.step([StepEntry("u", tokens[:29], [])])
    again, start = [], 29
    for count in (9, 5, 1, 1):
        again.append(engine.step([StepEntry("u", tokens[start:start + count], list(range(count)))]).cpu())
        start += count
    engine.finish("u")
    assert_close(torch.cat(again), torch.cat([trace["logits"] for trace in traces]).cpu().double(), CUT_TOLERANCE["bfloat16"], "without a trace")


@pytest.mark.parametrize("name,dtype", CASES)
def test_most_in_one_step_then_the_last_32_one_by_one(setups, name, dtype):
    setup = setups(name, dtype)
    engine = new_engine(setup, dtype)
    length = 90 if name == "A" else 131
    tokens = request_tokens(name, 7, length)
    whole = Replayer(engine)
    whole.step([("w", tokens, list(range(length)))], end=["w"])
    cut = Replayer(engine)
    cut.step([("c", tokens[:length - 32], list(range(length - 32)))])
    for position in range(length - 32, length):
        cut.step([("c", [tokens[position]], [0])])
    engine.finish("c")
    got = cut.logits_of("c", range(length))
    assert first_bad_row(got, plain_logits(setup, tokens), TOLERANCE[dtype]) is None
    bad = first_bad_row(got, whole.logits_of("w", range(length)), CUT_TOLERANCE[dtype])
    assert bad is None, f"decoded position {bad} differs from the whole prompt's"


@pytest.mark.parametrize("name,dtype", CASES)
def test_portions_of_changing_size(setups, name, dtype):
    setup = setups(name, dtype)
    engine = new_engine(setup, dtype)
    length = 101 if name == "A" else 160
    tokens = request_tokens(name, 3, length)
    sizes = [16, 7, 2, 5, 3, 2, 1, 17, 2, 31, 2, 2, 1, 1, 9]
    replay = Replayer(engine)
    cursor, turn = 0, 0
    while cursor < length:
        size = min(sizes[turn % len(sizes)], length - cursor)
        replay.step([("p", tokens[cursor:cursor + size], list(range(size)))])
        cursor += size
        turn += 1
    engine.finish("p")
    got = replay.logits_of("p", range(length))
    bad = first_bad_row(got, plain_logits(setup, tokens), TOLERANCE[dtype])
    assert bad is None, f"first wrong position {bad} (page size 16; portions {sizes})"


def mixed_trace(name, seed, requests=7, live_limit=4):
    """A seeded trace: up to four live requests, portions of some beside single decoded tokens of
    others, requests ending and new ones starting mid-trace.  Returns (steps, token lists, the
    most 64-rounded positions live at once)."""
    rng = random.Random(seed)
    limit = CONFIGS[name]["max_position_embeddings"]
    lengths = [rng.randint(34, min(limit, 120)) for _ in range(requests)]
    tokens = {f"r{i}": request_tokens(name, 50 + i, lengths[i]) for i in range(requests)}
    waiting = list(tokens)
    live, done_at, steps, most = {}, {}, [], 0
    while waiting or live:
        while waiting and len(live) < live_limit and (not live or rng.random() < 0.6):
            live[waiting.pop(0)] = 0
        items, ending = [], []
        for request in list(live):
            if rng.random() < 0.2 and len(live) > 1:
                continue                                   # left out of this step, goes on later
            at, total = live[request], len(tokens[request])
            decode_from = total - 12
            size = 1 if at >= decode_from else min(rng.choice([2, 3, 5, 8, 16, 23]), decode_from - at)
            items.append((request, tokens[request][at:at + size], list(range(size))))
            live[request] = at + size
            if live[request] == total:
                ending.append(request)
        most = max(most, sum(-(-max(at, 1) // 64) * 64 for at in live.values()))
        if items:
            steps.append((items, ending))
        for request in ending:
            del live[request]
    return steps, tokens, most


@pytest.mark.parametrize("name,dtype", CASES)
def test_mixed_requests_with_pages_used_again(setups, name, dtype):
    setup = setups(name, dtype)
    steps, tokens, most = mixed_trace(name, seed=5)
    engine = new_engine(setup, dtype, max_tokens=most, page_size=16, max_requests=4)
    pages_seen = {}
    replay = Replayer(engine)
    for items, ending in steps:
        replay.step(items, end=())
        for request, _, _ in items:
            pages_seen.setdefault(request, set()).update(engine.cache.page_list(request, 0))
        for request in ending:
            engine.finish(request)
    owners = {}
    for request, pages in pages_seen.items():
        for page in pages:
            owners.setdefault(page, set()).add(request)
    assert any(len(users) > 1 for users in owners.values()), "the trace never used a page again"
    for request, sequence in tokens.items():
        got = replay.logits_of(request, range(len(sequence)))
        bad = first_bad_row(got, plain_logits(setup, sequence), TOLERANCE[dtype])
        assert bad is None, f"{request}: first wrong position {bad} of {len(sequence)}"
    assert engine.cache.free_pages() == [engine.cache.num_pages] and engine.cache.free_slots == 4


@pytest.mark.parametrize("name,dtype", CASES)
def test_long_decoding_and_first_tokens(setups, name, dtype):
    setup = setups(name, dtype)
    engine = new_engine(setup, dtype)
    length = CONFIGS[name]["max_position_embeddings"]
    tokens = request_tokens(name, 9, length)
    replay = Replayer(engine)
    for position in range(length):                      # every token of the sequence decoded one by one, from the first
        replay.step([("d", [tokens[position]], [0])])
    engine.finish("d")
    got = replay.logits_of("d", range(length))
    want = plain_logits(setup, tokens)
    assert_close(got[:4], want[:4], TOLERANCE[dtype], "the first tokens of a sequence")
    bad = first_bad_row(got, want, TOLERANCE[dtype])
    assert bad is None, f"first wrong position {bad} of {length}"
    from tlie_amd import EngineError, StepEntry
    engine.admit("over")
    with pytest.raises(EngineError):
        engine.step([StepEntry("over", tokens + [1], [])])          # past the model's positions
    with pytest.raises(EngineError):
        engine.step([StepEntry("over", [CONFIGS[name]["vocab_size"]], [0])])   # token outside the vocabulary
    with pytest.raises(EngineError):
        engine.step([StepEntry("over", [1], [0]), StepEntry("over", [2], [0])])  # a request twice in a step
    engine.finish("over")


@pytest.mark.parametrize("name,dtype", CASES)
def test_greedy_generation_through_the_entry_point(setups, name, dtype):
    setup = setups(name, dtype)
    engine = new_engine(setup, dtype)
    prompts = [request_tokens(name, 20 + i, n) for i, n in enumerate((16, 5, 37))]
    got = engine.generate(prompts, max_tokens=16, chunk_size=16, max_tokens_per_step=24)
    for prompt, tokens in zip(prompts, got):
        want = plain_generate_greedy(setup["raw"], setup["weights"], prompt, 16)
        if dtype == "float32":
            assert tokens == want
        else:
            # bfloat16 may pick another token where the two best logits are closer than its rounding;
            # up to the first such place the tokens are the same, and that place must be a near tie
            same = next((i for i, (a, b) in enumerate(zip(tokens, want)) if a != b), len(want))
            if same < len(want):
                logits = plain_forward(setup["raw"], setup["weights"], prompt + want[:same])[-1]
                gap = (logits[want[same]] - logits[tokens[same]]).item()
                assert 0 <= gap <= 2 * TOLERANCE[dtype] * logits.abs().max().item(), f"token {same} differs without a near tie"
    assert engine.cache.free_pages() == [engine.cache.num_pages]
    # the loop launched decode steps before it had read the tokens of the step before
    assert engine.stats["steps_ahead"] >= 10 and engine.stats["steps_ahead"] <= engine.stats["steps"]


def test_greedy_generation_of_a_hundred_requests_at_once(setups):
    """A hundred requests through the engine's loop in 32-bit: the decode steps are replays of the
    recording for up to 128 requests, fed with the tokens that sampling left on the device; the
    token budget admits the prompts over several steps, so requests start and end at different
    steps.  The tokens of every seventh request are compared with the plain implementation's."""
    setup = setups("B", "float32")
    engine = new_engine(setup, "float32", max_tokens=100 * 64, max_requests=100)
    prompts = [request_tokens("B", 500 + i, 2 + (5 * i) % 19) for i in range(100)]
    got = engine.generate(prompts, max_tokens=11, max_tokens_per_step=160)
    assert (128, 256) in engine.runner._graphs
    for index in range(0, 100, 7):
        want = plain_generate_greedy(setup["raw"], setup["weights"], prompts[index], 11)
        assert got[index] == want, f"request {index}"
    assert engine.cache.free_pages() == [engine.cache.num_pages]


@pytest.mark.parametrize("name,dtype", CASES)
def test_recorded_portion_steps_replay_like_eager_ones(setups, name, dtype):
    """Steps of prompt portions (beside single tokens) of up to some hundred tokens are recorded
    too, per (tokens, sequences, longest sequence) padded up, with the attention kernel's work list
    at a fixed size.  The same recording is replayed with the step cut in other ways each time
    (other portions, other sequences, fewer tokens than it holds, pages in another order), with
    eager steps (all rows wanted: never recorded) and synchronisations in between, and every
    replay is checked against an engine that launches one kernel at a time."""
    setup = setups(name, dtype)
    recorded, eager = new_engine(setup, dtype, max_tokens=1024, max_requests=8), \
        new_engine(setup, dtype, max_tokens=1024, max_requests=8, use_graphs=False)
    padded = new_engine(setup, dtype, max_tokens=1024, max_requests=8, capture_graphs=False)
    rng = random.Random(5)
    streams = {f"p{i}": request_tokens(name, 40 + i, n) for i, n in enumerate((97, 64, 31, 120))}
    done = {request: 0 for request in streams}
    a, b, c = Replayer(recorded), Replayer(eager), Replayer(padded)
    turn = 0
    while any(done[request] < len(tokens) for request, tokens in streams.items()):
        items = []
        for request, tokens in streams.items():
            left = len(tokens) - done[request]
            if left == 0 or (turn % 3 == 1 and request == "p1"):        # a request may sit a step out
                continue
            count = min(left, rng.choice([1, 1, 2, 3, 5, 16, 17, 30]))
            items.append((request, tokens[done[request]:done[request] + count], [count - 1] if rng.random() < 0.8 else []))
            done[request] += count
        if not items:
            turn += 1
            continue
        for replay in (a, b, c):
            replay.step(items)
        if turn % 4 == 2:
            torch.cuda.synchronize()
            extra = request_tokens(name, 300 + turn, 9)
            for replay in (a, b, c):                      # an eager step in between: every row wanted
                replay.step([(f"x{turn}", extra, list(range(9)))], end=[f"x{turn}"])
        turn += 1
    graphs = recorded.runner._portion_graphs
    assert len(graphs) >= 2 and all(graph.graph is not None for graph in graphs.values()) and not eager.runner._portion_graphs
    assert padded.runner._portion_graphs and all(graph.graph is None for graph in padded.runner._portion_graphs.values())
    assert_same_bits(a, c, "steps of prompt portions")
    assert set(a.rows) == set(b.rows) and len(a.rows) > 30
    keys = sorted(a.rows, key=str)
    got, want = torch.stack([a.rows[key] for key in keys]), torch.stack([b.rows[key] for key in keys])
    bad = first_bad_row(got, want, CUT_TOLERANCE[dtype])
    assert bad is None, f"replayed step differs from the eager one at {keys[bad]}"
    # and against the plain implementation
    for request, tokens in streams.items():
        places = [key[1] for key in keys if key[0] == request]
        rows = torch.stack([a.rows[(request, place)] for place in places])
        assert first_bad_row(rows, plain_logits(setup, tokens)[places], TOLERANCE[dtype]) is None


@pytest.mark.parametrize("name,dtype", CASES)
def test_recorded_decode_steps_replay_like_eager_ones(setups, name, dtype):
    """Decode steps are recorded once per batch-size bucket into a HIP graph and replayed.  Every
    replay is checked against an engine that launches the same steps one kernel at a time, with
    prompt steps (never recorded) and synchronisations in between, batches that do not fill their
    bucket, and a request that ends mid-way so that rows of the bucket become padding."""
    setup = setups(name, dtype)
    recorded, eager = new_engine(setup, dtype, max_tokens=1024, max_requests=8), \
        new_engine(setup, dtype, max_tokens=1024, max_requests=8, use_graphs=False)
    padded = new_engine(setup, dtype, max_tokens=1024, max_requests=8, capture_graphs=False)
    assert recorded.runner.use_graphs and not eager.runner.use_graphs
    prompts = {f"g{i}": request_tokens(name, 70 + i, n) for i, n in enumerate((9, 33, 20))}
    follow = {request: request_tokens(name, 80 + i, 40) for i, request in enumerate(prompts)}
    a, b, c = Replayer(recorded), Replayer(eager), Replayer(padded)
    for replay in (a, b, c):
        replay.step([(request, tokens, [len(tokens) - 1]) for request, tokens in prompts.items()])
    live = list(prompts)
    for turn in range(24):
        if turn == 9:
            for replay in (a, b, c):                      # a prompt step between replays
                replay.step([("late", follow["g0"][:13], [12])])
            live.append("late")
            follow["late"] = request_tokens(name, 90, 40)
        if turn == 15:
            for replay in (a, b, c):
                replay.engine.finish("g1")
            live.remove("g1")
        if turn == 19:
            # a request ends and one of the same name, shorter, takes the same row of the recorded step:
            # nothing of the first one's block table may serve the second
            for replay in (a, b, c):
                replay.engine.finish("late")
                for key in [key for key in replay.rows if key[0] == "late"]:
                    replay.rows[("late before", key[1])] = replay.rows.pop(key)
                replay.step([("late", follow["g2"][:3], [2])])
            follow["late"] = request_tokens(name, 91, 40)
        items = [(request, [follow[request][turn]], [0]) for request in live]
        a.step(items)
        b.step(items)
        c.step(items)
        torch.cuda.synchronize()
    assert recorded.runner._graphs and all(graph.graph is not None for graph in recorded.runner._graphs.values())
    assert padded.runner._graphs and all(graph.graph is None for graph in padded.runner._graphs.values())
    assert_same_bits(a, c, "decode steps")
    assert set(a.rows) == set(b.rows)
    keys = sorted(a.rows, key=str)
    got, want = torch.stack([a.rows[key] for key in keys]), torch.stack([b.rows[key] for key in keys])
    bad = first_bad_row(got, want, CUT_TOLERANCE[dtype])
    assert bad is None, f"replayed step differs from the eager one at {keys[bad]}"


def error_code(stderr):
    """The error line is the last line of standard error (the GPU's driver may print before it)."""
    return json.loads(stderr.strip().splitlines()[-1])["error"]["code"]


def test_replay_program_and_command_line(setups, tmp_path):
    """bin/trace_run and bin/tinyllama_amd as a user runs them: separate processes."""
    setup = setups("A", "float32")
    tokens = request_tokens("A", 1, 40)
    other = request_tokens("A", 2, 21)
    lines = [
        {"step": 0, "entries": [{"id": "a", "tokens": tokens[:30], "want": [0, 29]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": tokens[30:32], "want": []}, {"id": "b", "tokens": other, "want": [20]}], "end": ["b"]},
        {"step": 2, "entries": [{"id": "a", "tokens": tokens[32:], "want": [7]}], "end": ["a"]},
    ]
    out = tmp_path / "logits"
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", setup["folder"], "--dtype", "float32",
                          "--out", str(out), "--max-tokens", "128"], input="\n".join(json.dumps(line) for line in lines) + "\n",
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    assert run.stdout.split() == ["done", "0", "done", "1", "done", "2"]
    import numpy
    vocab = CONFIGS["A"]["vocab_size"]
    step0 = torch.from_numpy(numpy.fromfile(out / "0.f32", dtype="<f4").reshape(-1, vocab))
    step1 = torch.from_numpy(numpy.fromfile(out / "1.f32", dtype="<f4").reshape(-1, vocab))
    step2 = torch.from_numpy(numpy.fromfile(out / "2.f32", dtype="<f4").reshape(-1, vocab))
    want = plain_logits(setup, tokens)
    assert_close(step0, want[[0, 29]], TOLERANCE["float32"], "step 0")
    assert_close(step1, plain_logits(setup, other)[[20]], TOLERANCE["float32"], "step 1")
    assert_close(step2, want[[39]], TOLERANCE["float32"], "step 2")

    # what is no step, or ends a request that is not live, is an error line and exit status 1; the steps before it stand
    for bad_line, code in (('{"step": 7, "entries": [{"id": "a", "tokens": "x"}]}', "invalid_argument"), ("not json", "invalid_argument"),
                           ('{"step": 7, "entries": [], "end": ["nobody"]}', "invalid_argument"),
                           ('{"step": 7, "entries": [{"id": "a", "tokens": [999999], "want": [0]}]}', "out_of_bounds")):
        run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", setup["folder"], "--dtype", "float32",
                              "--out", str(tmp_path / "bad"), "--max-tokens", "128"], input=json.dumps(lines[0]) + "\n" + bad_line + "\n",
                             capture_output=True, text=True, timeout=300)
        assert run.returncode == 1 and run.stdout.split() == ["done", "0"] and error_code(run.stderr) == code, (bad_line, run.stderr)

    prompt = "ids:" + ",".join(str(token) for token in tokens[:9])
    cli = [sys.executable, os.path.join(ROOT, "bin", "tinyllama_amd")]
    run = subprocess.run(cli + ["generate", setup["folder"], prompt, "6", "--dtype", "float32"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    result = json.loads(run.stdout)
    assert result["prompt_tokens"] == 9
    assert result["generated_tokens"] == plain_generate_greedy(setup["raw"], setup["weights"], tokens[:9], 6)
    # the step times that the reference's generate reports (app/cuda_reference.cu:216-224)
    assert all(result[key] > 0 for key in ("prefill_compute_ms", "prefill_transfer_ms", "decode_compute_ms", "decode_transfer_ms"))
    assert result["prefill_compute_ms"] + result["decode_compute_ms"] < result["wall_ms"]
    run = subprocess.run(cli + ["logits", setup["folder"], prompt, "--dtype", "float32"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    assert_close(torch.tensor(json.loads(run.stdout)["logits"]), plain_logits(setup, tokens[:9])[-1], TOLERANCE["float32"], "logits")
    run = subprocess.run(cli + ["generate", setup["folder"], prompt, "many"], capture_output=True, text=True, timeout=300)
    assert run.returncode != 0 and error_code(run.stderr) == "invalid_argument"     # tests/expect_cli_failure.cmake
    run = subprocess.run(cli + ["generate", setup["folder"], "some text", "4"], capture_output=True, text=True, timeout=300)
    assert run.returncode != 0 and error_code(run.stderr) == "tokenizer_error"
    run = subprocess.run(cli + ["generate", setup["folder"], prompt, "200"], capture_output=True, text=True, timeout=300)
    assert run.returncode != 0 and error_code(run.stderr) == "out_of_bounds"         # app/reference_cli.cpp:72-75
    # benchmark MODEL_DIR CONTEXT OUTPUT_TOKENS WARMUP SAMPLES, with the reference's keys (app/cuda_reference.cu:435-469)
    run = subprocess.run(cli + ["benchmark", setup["folder"], "20", "5", "1", "2", "--dtype", "float32"], capture_output=True, text=True,
                         timeout=300)
    assert run.returncode == 0, run.stderr
    result = json.loads(run.stdout)
    assert result["schema_version"] == 1 and result["context"] == 20 and result["output_tokens"] == 5 and result["sample_count"] == 2
    assert len(result["samples"]) == 2 and all(row["ttft_ms"] > 0 and row["tpot_ms"] > 0 for row in result["samples"])
    assert len(result["generated_tokens"]) == 5 and result["sampling"] == "greedy" and result["batch"] == 1
    assert 0 < result["kv_cache_bytes"] < result["engine_peak_device_bytes"] <= result["vram_bytes"] and result["model_device_bytes"] > 0
    assert result["device_segments_after_workload"] >= result["device_segments_before_workload"] > 0
    # the digest of the weight file, when the caller names one
    run = subprocess.run(cli + ["logits", setup["folder"], prompt, "--expect-sha256", "ab" * 32], capture_output=True, text=True, timeout=300)
    assert run.returncode != 0 and error_code(run.stderr) == "checksum_mismatch"


# The layer sizes that the benchmark runs (width 2048, 32 heads on 4 groups of size 64, feed-forward
# 5632, vocabulary 32000), with two layers: the kernels' variants for these sizes (row products of 16
# rows at 2048 and 5632 columns, 8 query heads a key head, split keys, recorded steps) are the ones a
# served model runs, and the tiny configurations reach other variants.
BENCH_SHAPE = dict(model_type="llama", architectures=["LlamaForCausalLM"], hidden_size=2048, intermediate_size=5632,
                   num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=4, max_position_embeddings=2048,
                   vocab_size=32000, rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=False,
                   attention_bias=False, hidden_act="silu", bos_token_id=1, eos_token_id=2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_benchmark_layer_sizes_cut_three_ways(tmp_path, dtype):
    folder = make_model(tmp_path / "model", BENCH_SHAPE, seed=5, dtype_name=dtype, std=0.02, norm_std=0.1)
    raw, weights = load_plain(folder)
    length = 300
    tokens = random_tokens(77, length, BENCH_SHAPE["vocab_size"])
    want = plain_forward(raw, weights, tokens)
    del weights
    from tlie_amd import Engine
    engine = Engine(folder, dtype=dtype, max_tokens=1024, page_size=16, max_requests=4)
    whole = Replayer(engine)
    whole.step([("w", tokens, list(range(length)))], end=["w"])
    bad = first_bad_row(whole.logits_of("w", range(length)), want, TOLERANCE[dtype])
    assert bad is None, f"whole prompt: first wrong position {bad}"
    # most in one step, the last 32 one by one, beside a second request that decodes the same tokens
    cut = Replayer(engine)
    cut.step([("a", tokens[:length - 32], []), ("b", tokens[:length - 32], [])])
    for position in range(length - 32, length):
        cut.step([("a", [tokens[position]], [0]), ("b", [tokens[position]], [0])])
    engine.finish("a")
    engine.finish("b")
    for request in "ab":
        got = cut.logits_of(request, range(length - 32, length))
        bad = first_bad_row(got, want[length - 32:], TOLERANCE[dtype])
        assert bad is None, f"decoded position {length - 32 + bad} of {request} is wrong"
    # portions of changing size, down to two tokens
    portions = Replayer(engine)
    sizes, cursor, turn = [100, 2, 16, 3, 64, 17, 5, 1, 33], 0, 0
    while cursor < length:
        size = min(sizes[turn % len(sizes)], length - cursor)
        portions.step([("p", tokens[cursor:cursor + size], list(range(size)))])
        cursor += size
        turn += 1
    engine.finish("p")
    bad = first_bad_row(portions.logits_of("p", range(length)), want, TOLERANCE[dtype])
    assert bad is None, f"portions {sizes}: first wrong position {bad}"
    # steps that recordings serve (few wanted rows, at most some hundred tokens): two requests cut at
    # different places, so that a recording is replayed with other portions, with the library's
    # products at these sizes inside it
    few = Replayer(engine)
    cuts = {"q": [100, 78, 12, 110], "r": [90, 90, 1, 119]}
    starts = {"q": 0, "r": 0}
    for turn in range(4):
        items = []
        for request, sizes in cuts.items():
            first, size = starts[request], sizes[turn]
            items.append((request, tokens[first:first + size], [0, size - 1] if size > 1 else [0]))
            starts[request] += size
        few.step(items)
        torch.cuda.synchronize()
    engine.finish("q")
    engine.finish("r")
    graphs = engine.runner._portion_graphs
    assert (192, 8, 256) in graphs and (16, 8, 256) in graphs and all(graph.graph is not None for graph in graphs.values())
    for request in cuts:
        places = sorted(place for name, place in few.rows if name == request)
        assert len(places) >= 7
        bad = first_bad_row(few.logits_of(request, places), want[places], TOLERANCE[dtype])
        assert bad is None, f"recorded portions of {request}: position {places[bad]} is wrong"


# The layer sizes of the two larger shapes that bench.py offers (width 4096, head size 128; one with
# as many key heads as query heads and a feed-forward of 11008, one with 4 query heads a key head, a
# feed-forward of 14336 and rope_theta 500000), one layer each and a small vocabulary: other
# variants of the attention kernels (8 x 16 dims a head, one or four columns a tile in decode
# steps) and products whose sizes are no multiples of 512.
LARGER_SHAPES = {
    "mha_11008": dict(hidden_size=4096, intermediate_size=11008, num_attention_heads=32, num_key_value_heads=32, rope_theta=10000.0),
    "gqa_14336": dict(hidden_size=4096, intermediate_size=14336, num_attention_heads=32, num_key_value_heads=8, rope_theta=500000.0),
}


@pytest.mark.parametrize("shape", sorted(LARGER_SHAPES))
def test_larger_layer_sizes_in_bfloat16(tmp_path, shape):
    raw = dict(BENCH_SHAPE, num_hidden_layers=1, vocab_size=1000, max_position_embeddings=4096, **LARGER_SHAPES[shape])
    folder = make_model(tmp_path / "model", raw, seed=6, dtype_name="bfloat16", std=0.02, norm_std=0.1)
    stored, weights = load_plain(folder)
    length = 150
    tokens = random_tokens(91, length, 1000)
    want = plain_forward(stored, weights, tokens)
    del weights
    from tlie_amd import Engine
    engine = Engine(folder, dtype="bfloat16", max_tokens=1024, page_size=16, max_requests=4)
    whole = Replayer(engine)
    whole.step([("w", tokens, list(range(length)))], end=["w"])
    # (a recorded exception to the rows' bound of 1.5e-2: one layer of width 4096 with a feed-forward of
    # up to 14336 and a vocabulary of 1000 leaves rows whose largest logit is small against the noise of
    # sums over that many rounded products; a row of the widest shape reaches 1.6e-2)
    tolerance = 2e-2
    bad = first_bad_row(whole.logits_of("w", range(length)), want, tolerance)
    assert bad is None, f"whole prompt: first wrong position {bad}"
    # a recorded portion, then single tokens beside a second request (recorded decode steps of 2), then portions again
    cut = Replayer(engine)
    cut.step([("a", tokens[:97], [96]), ("b", tokens[:97], [0, 96])])
    for position in range(97, 120):
        cut.step([("a", [tokens[position]], [0]), ("b", [tokens[position]], [0])])
    cut.step([("a", tokens[120:], [0, 29]), ("b", tokens[120:137], [16])])
    cut.step([("b", tokens[137:], [12])], end=["a", "b"])
    assert engine.runner._graphs and engine.runner._portion_graphs
    for request in "ab":
        places = sorted(place for name, place in cut.rows if name == request)
        bad = first_bad_row(cut.logits_of(request, places), want[places], tolerance)
        assert bad is None, f"{shape}: position {places[bad]} of {request} is wrong"


def plain_sampled_continuation(setup, prompt, generated, temperature, top_p, seed, tolerance):
    """Checks a sampled continuation against the plain implementation token by token: token i must be
    what the plain distribution at that place gives for the uniform number of (seed, i) when the
    kept tokens are walked in index order, unless that number falls within rounding of a boundary
    between two tokens.  Returns the number of such near-boundary differences."""
    from tlie_amd.sampling import uniform01
    from plain_llama import plain_top_p_distribution
    near = 0
    for index, token in enumerate(generated):
        logits = plain_forward(setup["raw"], setup["weights"], prompt + generated[:index])[-1]
        distribution = plain_top_p_distribution(logits, temperature, top_p)
        cumulative = torch.cumsum(distribution, 0)
        u = uniform01(seed, index)
        want = min(int(torch.searchsorted(cumulative, torch.tensor(u, dtype=torch.float64)).item()), len(distribution) - 1)
        if token != want:
            assert distribution[token] > 0, f"token {index} = {token} is outside the kept set"
            edge = min(abs(u - cumulative[token].item()), abs(u - (cumulative[token] - distribution[token]).item()))
            assert edge < tolerance, f"token {index}: drew {token}, the plain walk gives {want} (distance to the boundary {edge:.2e})"
            near += 1
    return near


@pytest.mark.parametrize("dtype", DTYPES)
def test_seeded_sampling_is_the_same_under_every_cut_and_under_preemption(setups, dtype):
    """Three requests (prompts of 5, 37 and 64 tokens), temperature 0.8, seeded: together with
    prompts cut into portions of 16 beside decoded tokens; each alone and whole; and with so few
    pages that the scheduler has to preempt and recompute.  In 32-bit all three give the same
    tokens, which are the plain implementation's draws; bfloat16 is checked against the plain draws
    up to its first near tie."""
    from tlie_amd import Engine
    from tlie_amd.engine import Request, SamplingParams, Scheduler
    name = "B"
    setup = setups(name, dtype)
    prompts = [request_tokens(name, 40 + i, n) for i, n in enumerate((5, 37, 64))]
    new_tokens, temperature, top_p, seed = 24, 0.8, 0.95, 321
    together = new_engine(setup, dtype).generate(prompts, max_tokens=new_tokens, temperature=temperature, top_p=top_p,
                                                 seed=seed, chunk_size=16, max_tokens_per_step=24)
    alone = []
    for index, prompt in enumerate(prompts):
        alone += new_engine(setup, dtype).generate([prompt], max_tokens=new_tokens, temperature=temperature, top_p=top_p,
                                                   seed=seed + index)
    # 8 pages of 16 positions: the three requests need 2 + 4 + 6 at their ends, so they cannot all stay
    tight = Engine(setup["folder"], dtype=dtype, max_tokens=128, page_size=16, max_requests=4)
    assert tight.cache.num_pages == 8
    # (admitted as soon as a first portion fits, so that all three are in at once and the last must give way)
    scheduler = Scheduler(tight.cache, max_tokens_per_step=24, max_seqs_per_step=4, chunk_size=16, admit_partial=True,
                          max_positions=tight.spec.max_positions, eos_token_id=tight.spec.eos_token_id)
    requests = [Request(id=("tight", i), prompt=list(prompt),
                        params=SamplingParams(max_tokens=new_tokens, temperature=temperature, top_p=top_p, seed=seed + i))
                for i, prompt in enumerate(prompts)]
    for request in requests:
        scheduler.add(request)
    tight.run(scheduler)
    assert scheduler.stats["preemptions"] > 0, "the pool was meant to be too small for all three"
    assert tight.cache.free_pages() == [8]
    squeezed = [request.generated for request in requests]
    assert all(len(tokens) == new_tokens for tokens in together + alone + squeezed)
    if dtype == "float32":
        assert together == alone, "cutting and batching changed a seeded draw"
        assert squeezed == alone, "preemption and recomputation changed a seeded draw"
        for index, prompt in enumerate(prompts):
            assert plain_sampled_continuation(setup, prompt, alone[index], temperature, top_p, seed + index, 1e-4) <= 1
    else:
        for index, prompt in enumerate(prompts):
            for tokens in (together[index], alone[index], squeezed[index]):
                same = next((i for i, (a, b) in enumerate(zip(tokens, alone[index])) if a != b), new_tokens)
                # up to where two cuts part ways (a near tie for bfloat16), the draws are the plain ones
                plain_sampled_continuation(setup, prompt, tokens[:same], temperature, top_p, seed + index, 5e-2)


def test_step_timings(setups):
    """A step that is asked for its times waits for the device and reports compute, transfer and
    wall time, for a prompt step and for a recorded decode step alike; the logits are the same."""
    from tlie_amd import StepEntry
    from tlie_amd.engine import StepTimings
    setup = setups("A", "bfloat16")
    timed, plain = new_engine(setup, "bfloat16"), new_engine(setup, "bfloat16")
    tokens = request_tokens("A", 5, 30)
    for engine in (timed, plain):
        engine.admit("t")
    measured = StepTimings()
    a = timed.step([StepEntry("t", tokens[:20], [19])], measured)
    b = plain.step([StepEntry("t", tokens[:20], [19])])
    assert torch.equal(a, b) and 0 < measured.compute_ms < measured.wall_ms and measured.transfer_ms > 0
    for position in range(20, 30):
        measured = StepTimings()
        a = timed.step([StepEntry("t", [tokens[position]], [0])], measured)
        b = plain.step([StepEntry("t", [tokens[position]], [0])])
        assert torch.equal(a, b), position
        assert 0 < measured.compute_ms < measured.wall_ms and measured.transfer_ms > 0


def test_a_request_that_stops_at_a_token_beside_one_that_does_not(setups):
    """Stopping at the end-of-sequence token needs the token on the host before the next plan:
    such a request keeps the loop from running ahead, and ends where the token first appears;
    the request beside it is not disturbed, and the loop runs ahead again once it is alone."""
    from tlie_amd.engine import Request, SamplingParams, Scheduler
    setup = setups("A", "float32")
    prompt, other_prompt = request_tokens("A", 61, 12), request_tokens("A", 62, 20)
    free = new_engine(setup, "float32").generate([prompt, other_prompt], max_tokens=14)
    stop_token = free[0][5]
    want = free[0][:free[0].index(stop_token) + 1]
    engine = new_engine(setup, "float32")
    scheduler = Scheduler(engine.cache, max_positions=engine.spec.max_positions, eos_token_id=stop_token)
    stopper = Request("s", list(prompt), SamplingParams(max_tokens=14, stop_on_eos=True))
    other = Request("o", list(other_prompt), SamplingParams(max_tokens=14))
    scheduler.add(stopper)
    scheduler.add(other)
    engine.run(scheduler)
    assert stopper.generated == want and stopper.finish_reason == "eos"
    assert other.generated == free[1] and other.finish_reason == "length"
    assert 0 < engine.stats["steps_ahead"] <= engine.stats["steps"] - len(want)
    assert engine.cache.free_pages() == [engine.cache.num_pages]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("many", [24, 80])
def test_recorded_steps_of_many_requests_replay_like_eager_ones(setups, dtype, many):
    """The same check for steps of 17 to 24 requests, which take other kernels than small steps do
    (products that leave partial sums to their consumers), and of 70 to 80 (the library's products
    inside the recording): every replay of the recording against the same step launched kernel by
    kernel, requests ending mid-way."""
    setup = setups("B", dtype)
    recorded, eager = new_engine(setup, dtype, max_tokens=4096, max_requests=many), \
        new_engine(setup, dtype, max_tokens=4096, max_requests=many, use_graphs=False)
    padded = new_engine(setup, dtype, max_tokens=4096, max_requests=many, capture_graphs=False)
    prompts = {f"m{i}": request_tokens("B", 300 + i, 3 + (7 * i) % 23) for i in range(many)}
    follow = {request: request_tokens("B", 400 + i, 12) for i, request in enumerate(prompts)}
    a, b, c = Replayer(recorded), Replayer(eager), Replayer(padded)
    for replay in (a, b, c):
        replay.step([(request, tokens, [len(tokens) - 1]) for request, tokens in prompts.items()])
    live = list(prompts)
    for turn in range(12):
        if turn in (4, 8):
            for request in live[5:8]:
                for replay in (a, b, c):
                    replay.engine.finish(request)
            del live[5:8]
        items = [(request, [follow[request][turn]], [0]) for request in live]
        a.step(items)
        b.step(items)
        c.step(items)
        torch.cuda.synchronize()
    bucket = 32 if many == 24 else 128
    assert (bucket, 256) in recorded.runner._graphs and recorded.runner._graphs[(bucket, 256)].graph is not None
    assert_same_bits(a, c, f"decode steps of up to {many} requests")
    keys = sorted(a.rows, key=str)
    assert keys == sorted(b.rows, key=str)
    got, want = torch.stack([a.rows[key] for key in keys]), torch.stack([b.rows[key] for key in keys])
    bad = first_bad_row(got, want, CUT_TOLERANCE[dtype])
    assert bad is None, f"replayed step differs from the eager one at {keys[bad]}"
    plain = plain_logits(setup, prompts["m3"] + follow["m3"])
    mine = torch.stack([a.rows[("m3", position)] for position in range(len(prompts["m3"]) - 1, len(prompts["m3"]) + 12)])
    assert first_bad_row(mine, plain[len(prompts["m3"]) - 1:], TOLERANCE[dtype]) is None


def test_a_dropped_engine_frees_its_recordings_at_once(setups):
    """An engine and its recorded steps must not be cyclic garbage: the cycle collector would free
    them at a moment of its choosing, and inside another recording's capture the graph's destructor
    ends the process.  Dropping the last reference frees them, with the collector switched off."""
    import gc
    import weakref
    from tlie_amd import StepEntry
    setup = setups("A", "bfloat16")
    gc.collect()
    gc.disable()
    try:
        engine = new_engine(setup, "bfloat16")
        engine.admit("r")
        engine.step([StepEntry("r", [1, 2, 3], [])])
        for token in (4, 5, 6):
            engine.step([StepEntry("r", [token], [0])])
        recording = engine.runner._graphs[(1, 128)]
        assert recording.graph is not None
        watched = [weakref.ref(engine), weakref.ref(engine.runner), weakref.ref(recording), weakref.ref(recording.graph)]
        del recording
        del engine
        assert [watch() for watch in watched] == [None, None, None, None]
    finally:
        gc.enable()


def test_long_prompts_take_the_walk_through_lds(tmp_path):
    """A sequence long enough (1536 positions and more) that prompt portions are attended with
    the keys brought through LDS once for four waves: the whole prompt, and the same in two
    portions beside another request, against the plain implementation."""
    raw = dict(CONFIGS["A"], max_position_embeddings=2048, num_hidden_layers=1)
    folder = make_model(tmp_path / "model", raw, seed=21, dtype_name="bfloat16")
    stored, weights = load_plain(folder)
    length = 1800
    tokens = random_tokens(5, length, raw["vocab_size"])
    want = plain_forward(stored, weights, tokens)
    from tlie_amd import Engine, StepEntry
    engine = Engine(folder, dtype="bfloat16", max_tokens=4096, page_size=16, max_requests=4)
    replay = Replayer(engine)
    replay.step([("w", tokens, list(range(0, length, 7)) + [length - 1])], end=["w"])
    places = list(range(0, length, 7)) + [length - 1]
    bad = first_bad_row(replay.logits_of("w", places), want[places], TOLERANCE["bfloat16"])
    assert bad is None, f"whole: first wrong position {places[bad]}"
    other = random_tokens(6, 40, raw["vocab_size"])
    replay.step([("p", tokens[:1000], []), ("o", other, [39])])
    replay.step([("o", [3], [0]), ("p", tokens[1000:], list(range(800)))], end=["o", "p"])
    bad = first_bad_row(replay.logits_of("p", range(1000, length)), want[1000:], TOLERANCE["bfloat16"])
    assert bad is None, f"second portion: first wrong position {1000 + bad}"
    # the step's policy did choose that walk
    engine.admit("check")
    engine.cache.reserve("check", 1700)
    policy = ops.attention_plan(engine.runner.build_context([StepEntry("check", tokens[:1700], [])]), 2, 2, 16)
    assert policy[5] is True and policy[4] == 4
    engine.finish("check")


def test_twenty_thousand_positions_cut_two_ways_and_in_both_precisions(tmp_path):
    """A sequence of 20000 positions (1250 pages behind one block table; the plain implementation's
    20000 x 20000 scores are out of reach, what the kernels find among so many keys is
    tests/test_kernels_gpu.py's): the prompt in portions of 4096 and of 1000, then eight tokens one by one
    from recordings made for 32768 positions; the logits of the last positions must not depend on the cut,
    and bfloat16 must agree with the 32-bit path, which the plain implementation holds at shorter lengths."""
    from tlie_amd import Engine
    raw = dict(CONFIGS["A"], max_position_embeddings=32768, num_hidden_layers=1)
    length, tail = 20000, 8
    tokens = random_tokens(12, length, raw["vocab_size"])
    places = list(range(length - tail - 4, length))
    rows = {}
    for dtype in DTYPES:
        folder = make_model(tmp_path / dtype, raw, seed=41, dtype_name="bfloat16")      # (the same stored values for both)
        engine = Engine(folder, dtype=dtype, max_tokens=2 * length + 64, page_size=16, max_requests=2)
        replay = Replayer(engine)
        for name, portion in (("wide", 4096), ("narrow", 1000)):
            cursor = 0
            while cursor < length - tail:
                size = min(portion, length - tail - cursor)
                wanted = [place - cursor for place in places if cursor <= place < cursor + size]
                replay.step([(name, tokens[cursor:cursor + size], wanted)])
                cursor += size
            for position in range(length - tail, length):
                replay.step([(name, [tokens[position]], [0])])
            assert len(engine.cache.page_list(name, 0)) == length // 16
        assert any(key[1] == 32768 for key in engine.runner._graphs), sorted(engine.runner._graphs)
        engine.finish("wide")
        engine.finish("narrow")
        rows[dtype] = replay.logits_of("wide", places)
        assert_close(replay.logits_of("narrow", places), rows[dtype], CUT_TOLERANCE[dtype], f"{dtype}: portions of 1000 against portions of 4096")
    assert_close(rows["bfloat16"], rows["float32"].double(), TOLERANCE["bfloat16"], "bfloat16 against the 32-bit path")


@pytest.mark.parametrize("dtype", DTYPES)
def test_decoding_across_the_lengths_that_recordings_are_made_for(tmp_path, dtype):
    """A recording of decode steps is made for sequences up to a power of two of positions (its
    attention cuts the keys for that length).  A request that decodes from position 240 to 530
    passes from the recording for 256 to the one for 512 and on to the one for the model's 600."""
    raw = dict(CONFIGS["B"], max_position_embeddings=600, num_hidden_layers=1)
    folder = make_model(tmp_path / "model", raw, seed=31, dtype_name=dtype)
    stored, weights = load_plain(folder)
    tokens = random_tokens(8, 531, raw["vocab_size"])
    want = plain_forward(stored, weights, tokens)
    from tlie_amd import Engine
    engine = Engine(folder, dtype=dtype, max_tokens=1024, page_size=16, max_requests=2)
    replay = Replayer(engine)
    replay.step([("r", tokens[:240], [239])])
    for position in range(240, 531):
        replay.step([("r", [tokens[position]], [0])])
    engine.finish("r")
    assert sorted(engine.runner._graphs) == [(1, 256), (1, 512), (1, 600)]
    bad = first_bad_row(replay.logits_of("r", range(239, 531)), want[239:], TOLERANCE[dtype])
    assert bad is None, f"first wrong position {239 + bad}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_logits_that_are_not_finite_end_generation_and_leave_the_engine_usable(tmp_path, dtype):
    """A model whose final norm's weight is so large that the logits overflow: sampling marks the
    row (-1), the decode step that is launched before the host has read that mark takes token 0 and
    not a row before the embedding table, `generate` raises numerical_error, and everything the
    call's requests held has come back: the same engine takes the next call (which fails the same
    way, not with "already live"), and a step with the finiteness check raises too."""
    from safetensors.torch import load_file, save_file
    from tlie_amd import Engine, EngineError, ErrorCode, StepEntry
    folder = make_model(tmp_path / "inf", CONFIGS["A"], seed=3, dtype_name="float32")
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    tensors["model.norm.weight"] = torch.full_like(tensors["model.norm.weight"], 3.0e38)
    save_file(tensors, path)
    engine = Engine(folder, dtype=dtype, max_tokens=256, page_size=16, max_requests=4)
    for _ in range(2):
        with pytest.raises(EngineError) as caught:
            engine.generate([[1, 2, 3], [4, 5, 6, 7]], max_tokens=6)
        assert caught.value.code == ErrorCode.NUMERICAL
        engine.cache.check()
        assert engine.cache.live_requests() == [] and engine.cache.free_pages() == [engine.cache.num_pages]
    engine.admit("s")
    logits = engine.step([StepEntry("s", [1, 2, 3], [2])])
    assert not torch.isfinite(logits).all()
    with pytest.raises(EngineError) as caught:
        engine.step([StepEntry("s", [4], [0])], check_finite=True)
    assert caught.value.code == ErrorCode.NUMERICAL
    engine.finish("s")
    engine.cache.check()


def test_a_step_that_fails_after_reserving_gives_its_pages_back(setups):
    """A step whose launch raises after its pages were reserved (here: a token that is still on
    the device offered to a step that no recording serves) leaves the cache as it found it, and the
    next steps of the same requests get right logits."""
    from tlie_amd import EngineError, StepEntry
    setup = setups("A", "bfloat16")
    engine = new_engine(setup, "bfloat16", max_tokens=256)
    tokens = request_tokens("A", 5, 40)
    replay = Replayer(engine)
    replay.step([("r", tokens[:15], [14])])
    replay.step([("r", tokens[15:16], [0])])                 # a recorded decode step: its rows remember the page list
    free = engine.cache.free_pages()
    pages = list(engine.cache.page_list("r", 0))
    with pytest.raises(EngineError):
        engine.step([StepEntry("r", tokens[16:17], [], source=0)])     # position 16 lies on a second page: reserved, then refused
    assert engine.cache.free_pages() == free and engine.cache.page_list("r", 0) == pages and engine.cache.length("r") == 16
    engine.cache.check()
    engine.admit("other")                                    # takes the page the failed step had reserved first
    engine.step([StepEntry("other", tokens[:20], [])])
    for position in range(16, 40):
        replay.step([("r", tokens[position:position + 1], [0])])
    engine.finish("other")
    engine.finish("r")
    got = replay.logits_of("r", [14] + list(range(15, 40)))
    assert first_bad_row(got, plain_logits(setup, tokens)[14:], TOLERANCE["bfloat16"]) is None


def run_trace(setup, dtype, out, lines, max_tokens, extra=()):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", setup["folder"], "--dtype", dtype,
                           "--out", str(out), "--max-tokens", str(max_tokens), *extra],
                          input="\n".join(json.dumps(line) for line in lines) + "\n", capture_output=True, text=True, timeout=300)


def run_compare(a, b, *options):
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_compare"), str(a), str(b), *options],
                         capture_output=True, text=True, timeout=120)
    return run.returncode, json.loads(run.stdout.strip().splitlines()[-1])


@pytest.mark.parametrize("dtype", DTYPES)
def test_two_replays_cut_differently_agree_through_the_comparison_program(setups, tmp_path, dtype):
    """The same three streams through `bin/trace_run` twice, as processes: once each request whole
    and alone, once in portions down to two tokens beside the other requests' decoded tokens in a pool
    so small that pages are used again.  `bin/trace_compare` joins the two output folders on
    (request, position) through their index files and gates every row as the reference's comparison
    script gates its logits (scripts/compare_logits.py:35-36,126-135); a folder in which one request
    ran on other tokens fails the same gate."""
    setup = setups("B", dtype)
    streams = {name: request_tokens("B", 500 + index, length) for index, (name, length) in enumerate((("a", 70), ("b", 41), ("c", 90)))}
    whole = [{"step": index, "entries": [{"id": name, "tokens": tokens, "want": list(range(len(tokens)))}], "end": [name]}
             for index, (name, tokens) in enumerate(streams.items())]
    rng = random.Random(9)
    done, cut, step = {name: 0 for name in streams}, [], 0
    order = ["a", "b", "c"]
    live = ["a", "b"]                                  # "c" starts when "b" has ended: its pages are b's
    while live:
        entries, ended = [], []
        for name in list(live):
            left = len(streams[name]) - done[name]
            count = min(left, rng.choice([1, 1, 2, 3, 7, 16, 20]))
            entries.append({"id": name, "tokens": streams[name][done[name]:done[name] + count], "want": list(range(count))})
            done[name] += count
            if done[name] == len(streams[name]):
                ended.append(name)
                live.remove(name)
                if name == "b":
                    live.append("c")
        cut.append({"step": step, "entries": entries, "end": ended})
        step += 1
    assert run_trace(setup, dtype, tmp_path / "whole", whole, 256).returncode == 0
    # 12 pages of 16: "a" and "b" take 5 + 3, then "a" and "c" 5 + 6, three of them the pages "b" gave back
    run = run_trace(setup, dtype, tmp_path / "cut", cut, 192, ["--check-finite"])
    assert run.returncode == 0, run.stderr
    index = [json.loads(line) for line in (tmp_path / "cut" / "index.jsonl").read_text().splitlines()]
    assert len(index) == sum(len(tokens) for tokens in streams.values())
    assert {(row["id"], row["position"]) for row in index} == {(name, place) for name, tokens in streams.items() for place in range(len(tokens))}
    gate = ["--atol", "1e-5", "--rtol", "1e-5"] if dtype == "float32" else ["--atol", "0.15", "--rtol", "0.03"]
    code, report = run_compare(tmp_path / "cut", tmp_path / "whole", *gate, "--require-all")
    assert code == 0 and report["status"] == "passed" and report["compared_rows"] == len(index) and report["failed_rows"] == 0, report
    assert report["rows_only_in_a"] == 0 and report["rows_only_in_b"] == 0 and report["logits_max_abs_error"] >= 0.0
    # the relative gate of a row as a whole
    code, report = run_compare(tmp_path / "cut", tmp_path / "whole", "--row-rtol", str(CUT_TOLERANCE[dtype] if dtype == "bfloat16" else 1e-5))
    assert code == 0, report
    # one request on other tokens from its position 30 on: the rows before it pass, those after fail
    other = [dict(line) for line in whole]
    changed = list(streams["a"])
    changed[30] = (changed[30] + 1) % CONFIGS["B"]["vocab_size"]
    other[0] = {"step": 0, "entries": [{"id": "a", "tokens": changed, "want": list(range(70))}], "end": ["a"]}
    assert run_trace(setup, dtype, tmp_path / "other", other, 256).returncode == 0
    code, report = run_compare(tmp_path / "other", tmp_path / "whole", *gate)
    assert code == 1 and report["status"] == "failed" and 1 <= report["failed_rows"] <= 40, report
    assert report["worst"]["id"] == "a" and report["worst"]["position"] >= 30
    # a folder that lacks rows of the other one fails only when all are required
    code, report = run_compare(tmp_path / "whole", tmp_path / "other", *gate, "--require-all")
    assert code == 1
    code, report = run_compare(tmp_path / "nowhere", tmp_path / "whole")
    assert code == 2 and report["status"] == "error"


def test_several_prompts_from_the_command_line_batched_in_portions_with_preemption(setups, tmp_path):
    """`tinyllama_amd generate` with three prompts at once, prompt portions of 16 tokens, a token
    budget of 24 a step and a page pool so small that a request is preempted and recomputed: every
    prompt gets the plain implementation's greedy tokens, which are also what it gets alone (the
    reference gates its batch benchmark on the same equality, app/batch_benchmark.cu:163-177).  And
    the `batch` command: the same prompt once and four times at once."""
    setup = setups("A", "float32")
    prompts = [request_tokens("A", 600 + index, length) for index, length in enumerate((20, 18, 22))]
    want = [plain_generate_greedy(setup["raw"], setup["weights"], prompt, 28) for prompt in prompts]
    cli = [sys.executable, os.path.join(ROOT, "bin", "tinyllama_amd")]
    text = ";".join("ids:" + ",".join(str(token) for token in prompt) for prompt in prompts[:2])
    listed = tmp_path / "prompts.txt"
    listed.write_text("ids:" + " ".join(str(token) for token in prompts[2]) + "\n")
    # the prompts take 2 pages of 16 each; with 28 more positions each grows into a third (and a fourth):
    # 7 pages hold the three prompts, and not what they grow to (all three are admitted at once:
    # --admit-partial; by default the third would wait until the pool has room for all of it)
    run = subprocess.run(cli + ["generate", setup["folder"], text, "28", "--dtype", "float32", "--prompts-file", str(listed),
                                "--page-size", "16", "--max-cache-tokens", "112", "--chunk-size", "16", "--max-tokens-per-step", "24",
                                "--max-requests", "3", "--admit-partial"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    result = json.loads(run.stdout)
    assert [row["generated_tokens"] for row in result["requests"]] == want
    assert [row["prompt_tokens"] for row in result["requests"]] == [20, 18, 22]
    assert result["generated_tokens"] == want[0] and result["preemptions"] >= 1 and result["steps"] > 28
    # alone, with room: the same tokens, no preemption
    run = subprocess.run(cli + ["generate", setup["folder"], "-", "28", "--dtype", "float32", "--prompts-file", str(listed)],
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    result = json.loads(run.stdout)
    assert result["generated_tokens"] == want[2] and result["preemptions"] == 0 and "requests" not in result
    # a prompt that can never fit the pool is refused, as an error line
    run = subprocess.run(cli + ["generate", setup["folder"], text, "12", "--dtype", "float32", "--max-cache-tokens", "16"],
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 1 and error_code(run.stderr) == "out_of_memory"
    run = subprocess.run(cli + ["generate", setup["folder"], "ids:1,2;some text", "4"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 1 and error_code(run.stderr) == "invalid_argument"
    run = subprocess.run(cli + ["batch", setup["folder"], "20", "6", "0", "1", "--dtype", "float32", "--batch", "4"],
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    result = json.loads(run.stdout)
    assert result["tokens_match"] and result["passed"] and result["batch"] == 4 and len(result["generated_tokens"]) == 6
    assert result["batch_4_over_batch_1"] > 0 and result["batch_1_total_tokens_per_second"] > 0
    run = subprocess.run(cli + ["batch", setup["folder"], "20", "6", "0", "1", "--dtype", "float32", "--min-ratio", "1000"],
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 1 and json.loads(run.stdout)["passed"] is False


def test_pool_sized_by_a_share_of_free_memory_and_byte_budgets(setups):
    """Without a count of positions the pools take a share of the device memory that is free after
    the weights; budgets in bytes refuse a folder or a pool with out_of_memory before anything is
    mapped or allocated (src/weight_store.cpp:134-138, src/kv_cache.cpp:40-43)."""
    from tlie_amd import Engine, EngineError, ErrorCode
    setup = setups("A", "bfloat16")
    free, _ = torch.cuda.mem_get_info()
    engine = Engine(setup["folder"], dtype="bfloat16", max_tokens=None, cache_fraction=1e-4, max_requests=2)
    per_page = engine.cache.page_bytes(engine.model.run_needs(), 16, torch.bfloat16)
    assert per_page == 2 * (2 * 2 * 16 * 16 * 2)                       # two layers: keys and values of 2 heads of 16, 16 rows
    assert 0.5e-4 * free / per_page < engine.cache.num_pages <= 1e-4 * free / per_page
    assert engine.generate([[1, 2, 3]], max_tokens=4)[0] == new_engine(setup, "bfloat16").generate([[1, 2, 3]], max_tokens=4)[0]
    for arguments in (dict(max_tokens=4096, max_cache_bytes=255 * per_page), dict(max_tokens=64, max_weight_file_bytes=1000)):
        with pytest.raises(EngineError) as caught:
            Engine(setup["folder"], dtype="bfloat16", **arguments)
        assert caught.value.code == ErrorCode.OUT_OF_MEMORY and "budget" in caught.value.message
    with pytest.raises(EngineError):
        Engine(setup["folder"], dtype="bfloat16", max_tokens=None)


def test_the_weights_lie_in_one_allocation_and_load_part_by_part(tmp_path):
    """What the parts keep lies in the engine's one weight allocation, each tensor at a multiple of 256
    bytes, a tied head on the table's place; and while a model loads, the device never holds much more than
    that allocation: stored tensors come when a part asks and go when it has loaded (a load that brought
    all stored tensors first would hold twice the weights at its peak)."""
    from tlie_amd import Engine
    raw = dict(CONFIGS["A"], hidden_size=512, intermediate_size=1024, num_hidden_layers=12, num_attention_heads=8,
               num_key_value_heads=2, head_dim=64, vocab_size=1000, tie_word_embeddings=True)
    folder = make_model(tmp_path / "model", raw, seed=4, dtype_name="bfloat16", std=0.02)
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_allocated()
    engine = Engine(folder, dtype="bfloat16", max_tokens=64, page_size=16, max_requests=2)
    peak = torch.cuda.max_memory_allocated() - before
    arena = engine.weight_arena
    model = engine.model
    kept = [model.embedding.table, model.final_norm.weight, model.head.linear.weight]
    for block in model.blocks:
        kept += [block.mixer.qkv.weight, block.mixer.o.weight, block.feed_forward.gate_up.weight, block.feed_forward.down.weight,
                 block.mixer_norm.weight, block.feed_forward_norm.weight]
    assert all(arena.holds(tensor) and tensor.data_ptr() % 256 == 0 for tensor in kept) and arena.outside == 0
    assert model.head.linear.weight.data_ptr() == model.embedding.table.data_ptr()
    stored = os.path.getsize(os.path.join(folder, "model.safetensors"))
    assert 0.98 * stored < arena.used <= arena.capacity < 1.02 * stored
    assert peak < 1.4 * arena.capacity, (peak, arena.capacity)
    tokens = random_tokens(3, 20, 1000)
    plain = plain_forward(*load_plain(folder), tokens)
    replay = Replayer(engine)
    replay.step([("r", tokens, list(range(20)))], end=["r"])
    assert_close(replay.logits_of("r", range(20)), plain, TOLERANCE["bfloat16"], "a model in the arena, whole")
