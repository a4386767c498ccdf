"""Measures decoding and prefill of the TinyLlama 1.1B shape with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 2048] [--dtype bfloat16]
                    [--shape tinyllama|llama2_7b|llama3_8b] [--layers N] [--no-points]
    python bench.py --workload serving|mixed [--shape ...] [--token-budget 2048]     (records of their own)
    python bench.py --prefill TOKENS                                                 (a prompt step alone)

A step is one decode step of the whole batch.  The batch's requests are first prefilled so that
after the warm-up and the K timed steps their length is `context`; then W untimed and exactly K
timed steps run, each through the engine's own step function and sampler (greedy), and one JSON
line is printed; that is done `--repeats` times and the median run counts.  `value` is decoded
tokens per second.  The same line carries the prefill of a 2,048-token prompt, the decode step's
share of the HBM roofline, and in `points` (every key a number): decoding at batch 1 and 64, the
workload of a 128-token prompt with 128 generated tokens, the same model in true 32-bit (decoding and
the prompt step), and decoding at the layer sizes of Llama-2-7B and Llama-3-8B with a quarter of
their layers (the counts are named); `*_frac` is the share of the published peak (HBM for decoding,
the matrix cores of the dtype for prompts).

Peaks are the MI355X's published ones: HBM 8 TB/s; dense MFMA 2.5 PFLOP/s for bfloat16, 157.3
TFLOP/s for float32.  `measured_peaks` holds what two microbenchmarks of the kernel library reach
on the machine at hand (a streaming read, chains of bfloat16 matrix instructions), and
`frac_of_measured` the same shares against those.
"""
import argparse
import json
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

HBM_PEAK = 8.0e12
MFMA_PEAK = {"bfloat16": 2.5e15, "float32": 157.3e12}

# the TinyLlama 1.1B configuration
TINYLLAMA = dict(model_type="llama", architectures=["LlamaForCausalLM"], hidden_size=2048, intermediate_size=5632,
                 num_hidden_layers=22, num_attention_heads=32, num_key_value_heads=4, max_position_embeddings=2048,
                 vocab_size=32000, rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=False, attention_bias=False,
                 hidden_act="silu", bos_token_id=1, eos_token_id=2, torch_dtype="bfloat16")


# the layer sizes of the Llama-2-7B and Llama-3-8B configurations, for `--shape`
OTHER_SHAPES = {
    "llama2_7b": ("Llama-2-7B shape", dict(hidden_size=4096, intermediate_size=11008, num_hidden_layers=32, num_attention_heads=32,
                                           num_key_value_heads=32, max_position_embeddings=4096, vocab_size=32000, rope_theta=10000.0)),
    "llama3_8b": ("Llama-3-8B shape", dict(hidden_size=4096, intermediate_size=14336, num_hidden_layers=32, num_attention_heads=32,
                                           num_key_value_heads=8, max_position_embeddings=8192, vocab_size=128256, rope_theta=500000.0)),
}


def weight_bytes_per_step(cfg, itemsize):
    """Bytes of weights a decode step reads: every matrix once, the norms, the head; of the
    embedding table only the batch's rows (not counted)."""
    h, i, d = cfg["hidden_size"], cfg["intermediate_size"], cfg["hidden_size"] // cfg["num_attention_heads"]
    qd, kvd = cfg["num_attention_heads"] * d, cfg["num_key_value_heads"] * d
    per_layer = (qd + 2 * kvd) * h + h * qd + 2 * i * h + h * i + 2 * h
    return (cfg["num_hidden_layers"] * per_layer + h + cfg["vocab_size"] * h) * itemsize


def kv_bytes_per_token(cfg, itemsize):
    d = cfg["hidden_size"] // cfg["num_attention_heads"]
    return 2 * cfg["num_key_value_heads"] * d * cfg["num_hidden_layers"] * itemsize


def prefill_flops(cfg, tokens):
    h, i, d = cfg["hidden_size"], cfg["intermediate_size"], cfg["hidden_size"] // cfg["num_attention_heads"]
    nq = cfg["num_attention_heads"]
    qd, kvd = nq * d, cfg["num_key_value_heads"] * d
    linear = 2 * tokens * cfg["num_hidden_layers"] * ((qd + 2 * kvd) * h + h * qd + 3 * i * h)
    attention = cfg["num_hidden_layers"] * 4 * nq * d * tokens * (tokens + 1) // 2
    head = 2 * cfg["vocab_size"] * h
    return linear + attention + head


def time_decode(engine, torch, batch, context, steps, warmup, vocab):
    """`batch` requests through the engine's own loop (scheduler, recorded decode steps, sampling
    on the device, tokens read a step behind): prompts first, then warmup + steps decode steps, the
    last token of each request being the `context`-th of its sequence; returns seconds for the
    timed steps."""
    from tlie_amd.engine import Request, SamplingParams, Scheduler
    prompt_len = context - steps - warmup - 1
    generator = torch.Generator().manual_seed(batch)
    # the token budget lets all prompts through in one step, so that every request decodes from the same step on
    scheduler = Scheduler(engine.cache, max_tokens_per_step=batch * prompt_len, max_seqs_per_step=batch,
                          max_positions=engine.spec.max_positions, eos_token_id=engine.spec.eos_token_id)
    requests = [Request(id=("bench", index), prompt=torch.randint(0, vocab, (prompt_len,), generator=generator).tolist(),
                        params=SamplingParams(max_tokens=steps + warmup + 1)) for index in range(batch)]
    for request in requests:
        scheduler.add(request)
    assert engine.run(scheduler, max_steps=1) == 1
    assert all(len(request.generated) == 1 for request in requests)
    assert engine.run(scheduler, max_steps=warmup) == warmup
    torch.cuda.synchronize()
    started = time.perf_counter()
    ran = engine.run(scheduler, max_steps=steps)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - started
    assert ran == steps and not scheduler.has_work() and all(len(request.generated) == steps + warmup + 1 for request in requests)
    return elapsed


def time_prefill(engine, torch, tokens, vocab, repeats=3):
    from tlie_amd import StepEntry
    generator = torch.Generator().manual_seed(tokens)
    prompt = torch.randint(0, vocab, (tokens,), generator=generator).tolist()
    best = None
    for _ in range(repeats + 1):
        engine.admit("prefill")
        torch.cuda.synchronize()
        started = time.perf_counter()
        logits = engine.step([StepEntry("prefill", prompt, [tokens - 1])])
        logits.argmax(-1).item()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - started
        engine.finish("prefill")
        best = elapsed if best is None else min(best, elapsed)       # the first run also warms up
    return best


def run_workload(engine, torch, workload, vocab, budget, chunk, slice_steps=8, prompt_cap=None):
    """A whole workload through the scheduler and the engine's loop, timed in slices of a few
    steps.  Returns the record's `value` parts and what the scheduler and the cache counted.
    serving: 64 requests at once, prompts of 128 to 2048 random tokens (or as many as leave the
    model's positions room for the output), 256 tokens decoded each, continuous batching.  mixed: 8 requests of 8192 positions (prompts of 8176 tokens, 16 decoded), cut into portions of `chunk`, beside 56
    streams with prompts of 32 to 128 tokens that decode 256 tokens each."""
    import random
    from tlie_amd.engine import Request, SamplingParams, Scheduler
    rng = random.Random(7)
    generator = torch.Generator().manual_seed(7)
    if workload == "serving":
        longest = min(2048, engine.spec.max_positions - 256)           # (a model of 2048 positions: prompts up to 1792)
        shapes = [(rng.randint(128, longest), 256) for _ in range(64)]
    else:
        shapes = [(rng.randint(32, 128), 256) for _ in range(56)] + [(8192 - 16, 16) for _ in range(8)]   # 8192 positions each
    scheduler = Scheduler(engine.cache, max_tokens_per_step=budget, max_seqs_per_step=len(shapes), chunk_size=chunk,
                          max_positions=engine.spec.max_positions, eos_token_id=engine.spec.eos_token_id,
                          prompt_tokens_beside_decodes=prompt_cap)
    requests = [Request(id=(workload, index), prompt=torch.randint(0, vocab, (length,), generator=generator).tolist(),
                        params=SamplingParams(max_tokens=new)) for index, (length, new) in enumerate(shapes)]
    for request in requests:
        scheduler.add(request)
    pages = engine.cache.num_pages
    slices, peak_pages = [], 0
    torch.cuda.synchronize()
    started = time.perf_counter()
    while scheduler.has_work():
        before = (time.perf_counter(), scheduler.stats["prefill_tokens"])
        ran = engine.run(scheduler, max_steps=slice_steps)
        torch.cuda.synchronize()
        slices.append(((time.perf_counter() - before[0]) / max(ran, 1), scheduler.stats["prefill_tokens"] > before[1]))
        peak_pages = max(peak_pages, pages - min(engine.cache.free_pages()))
    elapsed = time.perf_counter() - started
    assert all(len(request.generated) == new for request, (_, new) in zip(requests, shapes))
    with_prompts = sorted(seconds for seconds, prompts in slices if prompts)
    decode_only = sorted(seconds for seconds, prompts in slices if not prompts)
    middle = lambda values: values[len(values) // 2] * 1e3 if values else None
    prompt_tokens, new_tokens = sum(length for length, _ in shapes), sum(new for _, new in shapes)
    return {"seconds": elapsed, "tokens": prompt_tokens + new_tokens, "generated": new_tokens,
            "steps": scheduler.stats["steps"], "preemptions": scheduler.stats["preemptions"],
            "peak_pages_frac": peak_pages / pages, "ms_step_with_prompts": middle(with_prompts),
            "ms_step_decode_only": middle(decode_only)}


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=128)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--context", type=int, default=2048)
    parser.add_argument("--repeats", type=int, default=3,
                        help="the timed steps are run so many times, each after prompts and warm-up of its own; the median is reported")
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--layers", type=int, default=0, help="run fewer layers than the configuration has (named in the record)")
    parser.add_argument("--no-points", action="store_true", help="skip batch 1 and 64 and the prefill")
    parser.add_argument("--prefill", type=int, default=0, metavar="TOKENS",
                        help="only a prompt step of TOKENS tokens, ten times (for profiles): prints its record alone")
    parser.add_argument("--workload", default="decode", choices=["decode", "serving", "mixed"],
                        help="serving: 64 requests with prompts of 128 to 2048 tokens and 256 decoded tokens each, batched "
                             "continuously; mixed: 8 prompts of 8192 tokens in portions beside 56 short decode streams "
                             "(needs a shape with 8192 positions); each prints a record of its own")
    parser.add_argument("--token-budget", type=int, default=2048, help="tokens a step of a workload may hold")
    parser.add_argument("--prompt-cap", type=int, default=0,
                        help="workloads: the most prompt tokens in a step that also holds decoding requests (0: what the budget leaves)")
    parser.add_argument("--kernels", nargs="?", const="", default=None, metavar="NAME",
                        help="time the kernels of a decode step (--batch, --context) and of a prompt step one by one at the "
                             "shape's layer sizes, each inside a replayed recording that walks through copies of its weights; "
                             "NAME keeps the kernels whose name holds it; prints one JSON line per kernel")
    parser.add_argument("--shape", default="tinyllama", choices=["tinyllama", *OTHER_SHAPES],
                        help="layer sizes of another model of the same architecture (the default is the record's)")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this engine runs on a single MI355X)")
        return 2
    import torch
    from tlie_amd import Engine
    cfg, model_name = dict(TINYLLAMA), "TinyLlama 1.1B shape"
    if args.shape != "tinyllama":
        model_name = OTHER_SHAPES[args.shape][0]
        cfg.update(OTHER_SHAPES[args.shape][1])
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    if args.context > cfg["max_position_embeddings"] or args.steps + args.warmup >= args.context:
        print("context must fit the model's positions and exceed steps + warmup")
        return 2
    itemsize = 2 if args.dtype == "bfloat16" else 4
    vocab = cfg["vocab_size"]
    if args.kernels is not None:
        from tlie_amd.kernel_bench import bench_kernels
        for row in bench_kernels(cfg, batch=args.batch, context=args.context, prompt=args.prefill or 2048, only=args.kernels or None):
            print(json.dumps(row), flush=True)
        return 0
    if args.workload != "decode":
        if args.workload == "mixed" and cfg["max_position_embeddings"] < 8192:
            print("the mixed workload has prompts of 8192 tokens: take --shape llama3_8b")
            return 2
        live = 64 * (2048 + 256) if args.workload == "serving" else 8 * (8192 + 64) + 56 * (128 + 256 + 64)
        engine = Engine(None, dtype=args.dtype, config=cfg, random_seed=0, max_tokens=live, page_size=16, max_requests=65)
        chunk = None if args.workload == "serving" else 512
        cap = args.prompt_cap or None
        run_workload(engine, torch, args.workload, vocab, args.token_budget, chunk, prompt_cap=cap)   # warms up (recordings, plans)
        got = run_workload(engine, torch, args.workload, vocab, args.token_budget, chunk, prompt_cap=cap)
        print(json.dumps({"metric": f"total tok/s, {args.workload} workload ({model_name})", "value": got["tokens"] / got["seconds"],
                          "unit": "tokens/s", "generated_per_s": got["generated"] / got["seconds"], "seconds": got["seconds"],
                          "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "token_budget": args.token_budget,
                          "prompt_tokens_beside_decodes": args.prompt_cap or None,
                          "layers": cfg["num_hidden_layers"], "layers_of_model": full_layers,
                          **{key: got[key] for key in ("steps", "preemptions", "peak_pages_frac", "ms_step_with_prompts",
                                                       "ms_step_decode_only")}}))
        return 0
    if args.prefill:
        engine = Engine(None, dtype=args.dtype, config=cfg, random_seed=0, max_tokens=args.prefill + 2048, page_size=16, max_requests=2)
        seconds = time_prefill(engine, torch, args.prefill, vocab, repeats=10)
        print(json.dumps({"metric": f"prefill tok/s at {args.prefill} tokens ({model_name})", "value": args.prefill / seconds,
                          "unit": "tokens/s", "tokens": args.prefill, "ms": seconds * 1e3,
                          "frac": prefill_flops(cfg, args.prefill) / seconds / MFMA_PEAK[args.dtype]}))
        return 0
    most = max(args.batch, 1 if args.no_points else 64)
    started_all = time.perf_counter()
    engine = Engine(None, dtype=args.dtype, config=cfg, random_seed=0, max_tokens=most * args.context + 2048,
                    page_size=16, max_requests=most + 1)

    def median_decode(engine, batch, context, steps, warmup, vocab, repeats):
        """Seconds for `steps` timed decode steps: the median of `repeats` runs, each with its own
        prompts and `warmup` untimed steps before the timed ones."""
        runs = sorted(time_decode(engine, torch, batch, context, steps, warmup, vocab) for _ in range(repeats))
        return runs[len(runs) // 2]

    def step_bytes(cfg, itemsize, batch, context, steps):
        return weight_bytes_per_step(cfg, itemsize) + batch * (context - steps / 2) * kv_bytes_per_token(cfg, itemsize)

    elapsed = median_decode(engine, args.batch, args.context, args.steps, args.warmup, vocab, args.repeats)
    ms_per_step = elapsed / args.steps * 1e3
    value = args.batch * args.steps / elapsed
    achieved = step_bytes(cfg, itemsize, args.batch, args.context, args.steps) / (elapsed / args.steps)
    record = {
        "metric": f"decode tok/s at batch {args.batch}, context {args.context} ({model_name})", "value": value, "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: uniform random token ids, random weights N(0, 0.02)",
        "repeats": args.repeats,            # the timed steps were run so many times, each after its own warm-up; the median counts
        "config": {"model": model_name, "layers": cfg["num_hidden_layers"], "layers_of_model": full_layers,
                   "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"],
                   "head_dim": cfg["hidden_size"] // cfg["num_attention_heads"], "ffn": cfg["intermediate_size"],
                   "vocab": vocab, "global_batch": args.batch, "seq_len": args.context, "page_size": 16,
                   "parallelism": "single GPU"},
        "roofline": {"bound": "hbm", "achieved": achieved / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK},
    }
    if not args.no_points:
        from tlie_amd import ops
        peaks = ops.measured_peaks(engine.device)
        record["measured_peaks"] = {"stream_read_gbs": peaks["stream_read_gbs"], "mfma_bf16_tflops": peaks["mfma_bf16_tflops"]}
        record["roofline"]["frac_of_measured"] = achieved / (peaks["stream_read_gbs"] * 1e9)
        prefill_tokens = 2048
        seconds = time_prefill(engine, torch, prefill_tokens, vocab)
        flops = prefill_flops(cfg, prefill_tokens)
        record["prefill"] = {"value": prefill_tokens / seconds, "tokens": prefill_tokens, "ms": seconds * 1e3,
                             "frac": flops / seconds / MFMA_PEAK[args.dtype]}
        if args.dtype == "bfloat16":
            record["prefill"]["frac_of_measured"] = flops / seconds / (peaks["mfma_bf16_tflops"] * 1e12)
        points = {}
        for batch in (1, 64):
            steps = min(args.steps, 64)
            seconds = median_decode(engine, batch, args.context, steps, 4, vocab, args.repeats)
            points[f"decode_b{batch}"] = batch * steps / seconds
            points[f"decode_b{batch}_frac"] = step_bytes(cfg, itemsize, batch, args.context, steps) / (seconds / steps) / HBM_PEAK
        # a short prompt: its step is replayed from a recording (the long one's is launched kernel by kernel)
        points["prefill_256"] = 256 / time_prefill(engine, torch, 256, vocab)
        # the workload of a prompt of 128 tokens and 128 generated ones, at the record's batch and at 1 and 64
        warm = 8
        timed = 128 - warm - 1
        for batch in sorted({args.batch, 1, 64}):
            seconds = median_decode(engine, batch, 256, timed, warm, vocab, args.repeats)
            points[f"decode_b{batch}_prompt128"] = batch * timed / seconds
            points[f"decode_b{batch}_prompt128_frac"] = step_bytes(cfg, itemsize, batch, 256, timed) / (seconds / timed) / HBM_PEAK
        del engine
        torch.cuda.empty_cache()
        if args.dtype == "bfloat16" and args.shape == "tinyllama":
            # the same model in true 32-bit (the check path): decoding at the record's batch and the prompt step
            wide = Engine(None, dtype="float32", config=cfg, random_seed=0, max_tokens=args.batch * args.context + 4096,
                          page_size=16, max_requests=args.batch + 1)
            steps = 24
            seconds = median_decode(wide, args.batch, args.context, steps, 2, vocab, args.repeats)
            points[f"fp32_decode_b{args.batch}"] = args.batch * steps / seconds
            points[f"fp32_decode_b{args.batch}_frac"] = step_bytes(cfg, 4, args.batch, args.context, steps) / (seconds / steps) / HBM_PEAK
            seconds = time_prefill(wide, torch, prefill_tokens, vocab, repeats=2)
            points["fp32_prefill_2048"] = prefill_tokens / seconds
            points["fp32_prefill_2048_frac"] = flops / seconds / MFMA_PEAK["float32"]
            del wide
            torch.cuda.empty_cache()
            # the layer sizes of the two larger models of the same architecture, a quarter of their layers
            # (named beside the number), decoding at the record's batch at 2048 positions
            for shape, (name, sizes) in OTHER_SHAPES.items():
                larger = dict(TINYLLAMA)
                larger.update(sizes)
                layers_of_model = larger["num_hidden_layers"]
                larger["num_hidden_layers"] = layers_of_model // 4
                other = Engine(None, dtype="bfloat16", config=larger, random_seed=0, max_tokens=args.batch * 2048 + 2048,
                               page_size=16, max_requests=args.batch + 1)
                steps = 32
                seconds = median_decode(other, args.batch, 2048, steps, 4, larger["vocab_size"], args.repeats)
                key = f"{shape}_decode_b{args.batch}"
                points[key] = args.batch * steps / seconds
                points[key + "_ms"] = seconds / steps * 1e3
                points[key + "_frac"] = step_bytes(larger, 2, args.batch, 2048, steps) / (seconds / steps) / HBM_PEAK
                points[key + "_layers"] = larger["num_hidden_layers"]
                points[key + "_layers_of_model"] = layers_of_model
                del other
                torch.cuda.empty_cache()
                # and that model's whole workload through the scheduler (the same number of layers): 64
                # requests served at once, or 8 long prompts in portions beside 56 short decode streams;
                # the second run is timed, the first makes the recordings
                workload, chunk = ("serving", None) if larger["max_position_embeddings"] < 8192 else ("mixed", 512)
                live = 64 * (2048 + 256) if workload == "serving" else 8 * (8192 + 64) + 56 * (128 + 256 + 64)
                other = Engine(None, dtype="bfloat16", config=larger, random_seed=0, max_tokens=live, page_size=16, max_requests=65)
                run_workload(other, torch, workload, larger["vocab_size"], 2048, chunk)
                got = run_workload(other, torch, workload, larger["vocab_size"], 2048, chunk)
                key = f"{shape}_{workload}"
                points[key + "_tok_s"] = got["tokens"] / got["seconds"]
                points[key + "_generated_tok_s"] = got["generated"] / got["seconds"]
                points[key + "_ms_step_with_prompts"] = got["ms_step_with_prompts"]
                points[key + "_ms_step_decode_only"] = got["ms_step_decode_only"]
                points[key + "_preemptions"] = got["preemptions"]
                if workload == "mixed":
                    # the other end of the trade: prompts get at most 256 tokens in a step that also decodes, so
                    # the 56 decoding streams wait less for each of their tokens and the long prompts take longer
                    run_workload(other, torch, workload, larger["vocab_size"], 2048, chunk, prompt_cap=256)
                    got = run_workload(other, torch, workload, larger["vocab_size"], 2048, chunk, prompt_cap=256)
                    points[key + "_cap256_tok_s"] = got["tokens"] / got["seconds"]
                    points[key + "_cap256_generated_tok_s"] = got["generated"] / got["seconds"]
                    points[key + "_cap256_ms_step_with_prompts"] = got["ms_step_with_prompts"]
                    # and decoding at the model's longest context, 8192 positions, at the record's batch
                    steps = 24
                    seconds = median_decode(other, args.batch, 8192, steps, 4, larger["vocab_size"], args.repeats)
                    points[f"{shape}_decode_b{args.batch}_ctx8192"] = args.batch * steps / seconds
                    points[f"{shape}_decode_b{args.batch}_ctx8192_frac"] = step_bytes(larger, 2, args.batch, 8192, steps) / (seconds / steps) / HBM_PEAK
                del other
                torch.cuda.empty_cache()
        record["points"] = points
        record["bench_seconds"] = time.perf_counter() - started_all
    from tlie_amd import ops as kernel_faces
    # products of many rows that fell from the vendor's library to the plain 32-bit kernel (each many
    # times slower): a record measured with any would not be this engine's speed
    record["library_fallbacks"] = kernel_faces.library_fallbacks()
    assert record["library_fallbacks"] == 0, f"{record['library_fallbacks']} matrix products took the plain kernel instead of the library's"
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
