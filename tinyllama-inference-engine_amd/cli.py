"""The command line, in the manner of the reference's `tinyllama_cuda` (app/cuda_reference.cu:475-522)
and `tinyllama_reference` (app/reference_cli.cpp:40-125): positional arguments, JSON on standard
output, and errors as one JSON line `{"error": {"code", "message"}}` on standard error with a
non-zero exit status.

    tinyllama_amd generate  MODEL_DIR PROMPT MAX_TOKENS [GOLDEN_JSON]
    tinyllama_amd logits    MODEL_DIR PROMPT
    tinyllama_amd benchmark MODEL_DIR CONTEXT OUTPUT_TOKENS WARMUP SAMPLES
    tinyllama_amd batch     MODEL_DIR CONTEXT OUTPUT_TOKENS WARMUP SAMPLES   (batch 1 against batch N)
    tinyllama_amd random    MODEL_DIR CONFIG_JSON SEED          (writes a folder of random weights)

PROMPT is text when MODEL_DIR holds a tokenizer.model (the begin-of-sequence id is put in front,
as the reference does), or token ids written `ids:1,15043,3186`.  Several prompts run together
under the scheduler (continuous batching): `ids:1,2,3;ids:4,5` (token ids only), and/or
`--prompts-file FILE` with one prompt a line (PROMPT may then be `-`).  GOLDEN_JSON, when given,
holds `{"greedy_tokens": [...]}` and the (first prompt's) generated tokens must begin it
(app/cuda_reference.cu:198-211).
Options (after the positionals): --dtype bfloat16|float32, --temperature T, --top-p P, --seed S
(the reference's request options of the same names, app/server.cpp:601-613); the cache and the
scheduler: --max-cache-tokens N (positions the page pool holds), --page-size P, --max-requests R
(request slots), --max-tokens-per-step T (a step's token budget), --chunk-size C (the most tokens of
one prompt in a step), --prompt-tokens-beside-decodes N (the most prompt tokens in a step that also
decodes), --admit-partial (a waiting request is admitted as soon as a first portion of it fits the pool,
not only when all of it does); `batch`: --batch N (default 4), --min-ratio X (fail below this speed-up).
"""
from __future__ import annotations

import argparse
import json
import sys
import time

from .errors import EngineError, ErrorCode, invalid_argument

USAGE = ("usage: tinyllama_amd generate MODEL_DIR PROMPT MAX_TOKENS [GOLDEN_JSON]\n"
         "       tinyllama_amd logits MODEL_DIR PROMPT\n"
         "       tinyllama_amd benchmark MODEL_DIR CONTEXT OUTPUT_TOKENS WARMUP SAMPLES\n"
         "       tinyllama_amd batch MODEL_DIR CONTEXT OUTPUT_TOKENS WARMUP SAMPLES\n"
         "       tinyllama_amd random MODEL_DIR CONFIG_JSON SEED\n"
         "options: [--dtype bfloat16|float32] [--temperature T] [--top-p P] [--seed S] [--expect-sha256 HEX]\n"
         "         [--max-cache-tokens N] [--page-size P] [--max-requests R] [--max-tokens-per-step T] [--chunk-size C]\n"
         "         [--prompt-tokens-beside-decodes N] [--admit-partial] [--prompts-file FILE] [--batch N] [--min-ratio X]\n")


def parse_integer(text: str, name: str, minimum: int) -> int:
    """Whole-string integer >= minimum, else `invalid_argument` (app/reference_cli.cpp:27-36)."""
    try:
        if text.strip() != text or not text or text[0] == "+":
            raise ValueError
        value = int(text, 10)
    except ValueError:
        raise invalid_argument(f"{name} must be an integer >= {minimum}") from None
    if value < minimum:
        raise invalid_argument(f"{name} must be an integer >= {minimum}")
    return value


def prompt_ids(model_dir: str, prompt: str) -> tuple[list[int], object]:
    if prompt.startswith("ids:"):
        try:
            ids = [int(piece) for piece in prompt[4:].replace(",", " ").split()]
        except ValueError:
            raise invalid_argument("a prompt of token ids is written ids:1,2,3") from None
        if not ids:
            raise invalid_argument("the prompt holds no token")
        return ids, None
    from .tokenizer import Tokenizer
    tokenizer = Tokenizer(model_dir)
    return tokenizer.encode(prompt), tokenizer


def _engine(args, positions: int, requests: int = 1):
    """positions: what the live requests hold at most when the caller names no pool size (each
    request's share rounded up to whole pages)."""
    from .engine import Engine
    for name in ("page_size", "max_requests", "max_cache_tokens", "max_tokens_per_step", "chunk_size", "prompt_tokens_beside_decodes"):
        if getattr(args, name) < 0:
            raise invalid_argument(f"--{name.replace('_', '-')} must be positive")
    page_size = args.page_size or 16
    return Engine(args.model_dir, dtype=args.dtype,
                  max_tokens=args.max_cache_tokens or max(64, positions + requests * page_size), page_size=page_size,
                  max_requests=args.max_requests or max(4, requests), expect_sha256=args.expect_sha256)


def all_prompts(args) -> tuple[list[list[int]], object]:
    """The prompts of a `generate`: PROMPT (`ids:..;ids:..` holds several), then the lines of
    --prompts-file."""
    texts = []
    if args.prompt != "-" or not args.prompts_file:
        pieces = args.prompt.split(";") if args.prompt.startswith("ids:") else [args.prompt]
        if len(pieces) > 1 and not all(piece.strip().startswith("ids:") for piece in pieces):
            raise invalid_argument("several prompts in one argument are written ids:1,2;ids:3,4")
        texts += [piece.strip() for piece in pieces]
    if args.prompts_file:
        try:
            with open(args.prompts_file, "r", encoding="utf-8") as handle:
                texts += [line.rstrip("\n") for line in handle if line.strip()]
        except OSError as error:
            raise EngineError(ErrorCode.IO, f"unable to open the prompts file: {args.prompts_file} ({error.strerror})") from None
    if not texts:
        raise invalid_argument("no prompt is given")
    tokenizer, prompts = None, []
    for text in texts:
        ids, used = prompt_ids(args.model_dir, text)
        tokenizer = tokenizer or used
        prompts.append(ids)
    return prompts, tokenizer


def command_generate(args) -> int:
    max_tokens = parse_integer(args.rest[0], "MAX_TOKENS", 1)
    prompts, tokenizer = all_prompts(args)
    ids = prompts[0]
    engine = _engine(args, sum(len(prompt) + max_tokens for prompt in prompts), len(prompts))
    started = time.perf_counter()
    timings, stats = {}, {}
    outputs = engine.generate(prompts, max_tokens=max_tokens, temperature=args.temperature, top_p=args.top_p,
                              seed=args.seed, timings=timings, stats=stats,
                              max_tokens_per_step=args.max_tokens_per_step or 2048, chunk_size=args.chunk_size or None,
                              prompt_tokens_beside_decodes=args.prompt_tokens_beside_decodes or None,
                              admit_partial=args.admit_partial)
    generated = outputs[0]
    elapsed = (time.perf_counter() - started) * 1e3
    if len(args.rest) > 1:
        try:
            with open(args.rest[1], "r", encoding="utf-8") as handle:
                expected = json.load(handle)["greedy_tokens"]
        except (OSError, ValueError, KeyError):
            raise EngineError(ErrorCode.IO, "unable to open golden metadata") from None
        if len(generated) > len(expected) or list(expected[:len(generated)]) != generated:
            raise EngineError(ErrorCode.NUMERICAL, "greedy tokens do not match the golden tokens")
    result = {"prompt_tokens": len(ids), "generated_tokens": generated, "wall_ms": elapsed, **timings,
              "steps": stats.get("steps"), "preemptions": stats.get("preemptions")}
    if tokenizer is not None:
        result["text"] = tokenizer.decode(generated)
    if len(prompts) > 1:
        # one row per prompt, in the order given; the top-level keys stay the first prompt's
        result["requests"] = [{"prompt_tokens": len(prompt), "generated_tokens": output,
                               **({"text": tokenizer.decode(output)} if tokenizer is not None else {})}
                              for prompt, output in zip(prompts, outputs)]
    print(json.dumps(result))
    return 0


def command_logits(args) -> int:
    from .engine import StepEntry
    ids, _ = prompt_ids(args.model_dir, args.prompt)
    engine = _engine(args, len(ids))
    engine.admit("logits")
    logits = engine.step([StepEntry("logits", ids, [len(ids) - 1])], check_finite=True)     # src/cuda/model.cu:505-510
    print(json.dumps({"prompt_tokens": len(ids), "logits": logits[0].cpu().tolist()}))
    return 0


class _Range:
    """A named range for the profiler's timeline (roctx, through torch's marker calls), as the
    reference marks warmup / prefill / decode with NVTX ranges (app/cuda_reference.cu:31-37)."""

    def __init__(self, name: str):
        self.name = name

    def __enter__(self):
        import torch
        try:
            torch.cuda.nvtx.range_push(self.name)
            self.pushed = True
        except Exception:                      # (a build of torch without the marker library)
            self.pushed = False
        return self

    def __exit__(self, *unused):
        import torch
        if self.pushed:
            torch.cuda.nvtx.range_pop()
        return False


def command_benchmark(args) -> int:
    """One request: CONTEXT prompt tokens, OUTPUT_TOKENS greedy tokens; WARMUP runs, then SAMPLES
    timed ones; medians, the samples, and the device memory's accounting, as
    app/cuda_reference.cu:256-471 reports them (its keys where it has them)."""
    import statistics
    import torch
    from .engine import StepEntry
    context = parse_integer(args.rest[0], "CONTEXT", 1)
    output_tokens = parse_integer(args.rest[1], "OUTPUT_TOKENS", 1)
    warmup = parse_integer(args.rest[2], "WARMUP", 0)
    samples = parse_integer(args.rest[3], "SAMPLES", 1)
    if not torch.cuda.is_available():
        raise EngineError(ErrorCode.HIP, "no GPU is visible: the engine has no CPU path")
    before_model = torch.cuda.memory_allocated()
    engine = _engine(args, context + output_tokens)
    model_bytes = torch.cuda.memory_allocated() - before_model
    cache_bytes = sum(binding.cache.numel() * binding.cache.element_size()
                      for binding in {id(b.cache): b for b in engine.cache.bindings if b.cache is not None}.values())
    generator = torch.Generator().manual_seed(args.seed)
    prompt = torch.randint(0, engine.spec.vocab_size, (context,), generator=generator).tolist()
    ttft, tpot, tokens, sample_rows = [], [], None, []
    segments_before = None
    for run in range(warmup + samples):
        if run == warmup:
            segments_before = torch.cuda.memory_stats().get("segment.all.allocated", 0)
        with _Range("warmup" if run < warmup else "sample"):
            torch.cuda.synchronize()
            started = time.perf_counter()
            engine.admit("bench")
            with _Range("prefill"):
                logits = engine.step([StepEntry("bench", prompt, [context - 1])])
                token = int(logits.argmax(-1).item())
            first = time.perf_counter()
            generated = [token]
            with _Range("decode"):
                for _ in range(output_tokens - 1):
                    logits = engine.step([StepEntry("bench", [token], [0])])
                    token = int(logits.argmax(-1).item())
                    generated.append(token)
            finished = time.perf_counter()
            engine.finish("bench")
        if tokens is not None and generated != tokens:
            raise EngineError(ErrorCode.NUMERICAL, "benchmark samples did not produce identical tokens")
        tokens = generated
        if run >= warmup:
            ttft.append((first - started) * 1e3)
            row = {"ttft_ms": ttft[-1]}
            if output_tokens > 1:
                tpot.append((finished - first) * 1e3 / (output_tokens - 1))
                row["tpot_ms"] = tpot[-1]
            sample_rows.append(row)
    # (the reference fails its benchmark when the timed workload allocates device memory:
    # app/cuda_reference.cu:412-416; here the numbers of segments the allocator has taken from the
    # device before and after the samples are reported)
    segments_after = torch.cuda.memory_stats().get("segment.all.allocated", 0)
    properties = torch.cuda.get_device_properties(engine.device)
    result = {"schema_version": 1, "gpu": properties.name, "vram_bytes": properties.total_memory,
              "model_device_bytes": model_bytes, "engine_peak_device_bytes": torch.cuda.max_memory_allocated(),
              "device_segments_before_workload": segments_before, "device_segments_after_workload": segments_after,
              "kv_cache_bytes": cache_bytes, "dtype": args.dtype, "sampling": "greedy", "batch": 1,
              "context": context, "output_tokens": output_tokens, "warmup": warmup, "sample_count": samples,
              "samples": sample_rows, "generated_tokens": tokens,
              "ttft_ms_median": statistics.median(ttft),
              "prefill_tokens_per_second": context / (statistics.median(ttft) / 1e3)}
    if tpot:
        result["tpot_ms_median"] = statistics.median(tpot)
        result["decode_tokens_per_second"] = 1e3 / statistics.median(tpot)
    print(json.dumps(result))
    return 0


def command_batch(args) -> int:
    """The same prompt once, and N times at once, through the scheduler: every copy must generate
    the single run's tokens, and the record holds both rates and their ratio, as the reference's
    batch benchmark reports them for 1 against 4 (app/batch_benchmark.cu:124-203; its `--test` mode
    has no gate on the ratio, its `--benchmark` mode wants 1.5: here --min-ratio, default none)."""
    import statistics
    import torch
    context = parse_integer(args.rest[0], "CONTEXT", 1)
    output_tokens = parse_integer(args.rest[1], "OUTPUT_TOKENS", 1)
    warmup = parse_integer(args.rest[2], "WARMUP", 0)
    samples = parse_integer(args.rest[3], "SAMPLES", 1)
    batch = args.batch
    if batch < 2:
        raise invalid_argument("--batch must be at least 2")
    engine = _engine(args, batch * (context + output_tokens), batch)
    generator = torch.Generator().manual_seed(args.seed)
    prompt = torch.randint(0, engine.spec.vocab_size, (context,), generator=generator).tolist()

    def workload(copies):
        torch.cuda.synchronize()
        started = time.perf_counter()
        outputs = engine.generate([prompt] * copies, max_tokens=output_tokens, seed=args.seed,
                                  max_tokens_per_step=args.max_tokens_per_step or 2048, chunk_size=args.chunk_size or None)
        torch.cuda.synchronize()
        return outputs, time.perf_counter() - started
    for _ in range(warmup):
        workload(1)
        workload(batch)
    one_seconds, many_seconds, tokens_match, reference_tokens = [], [], True, None
    for _ in range(samples):
        one, seconds = workload(1)
        one_seconds.append(seconds)
        many, seconds = workload(batch)
        many_seconds.append(seconds)
        reference_tokens = one[0]
        tokens_match = tokens_match and all(output == reference_tokens for output in many)
    one_rate = output_tokens / statistics.median(one_seconds)
    many_rate = batch * output_tokens / statistics.median(many_seconds)
    ratio = many_rate / one_rate
    passed = tokens_match and ratio >= args.min_ratio
    print(json.dumps({"schema_version": 1, "dtype": args.dtype, "sampling": "greedy", "context": context,
                      "output_tokens": output_tokens, "warmup": warmup, "samples": samples, "batch": batch,
                      "batch_1_total_tokens_per_second": one_rate, f"batch_{batch}_total_tokens_per_second": many_rate,
                      f"batch_{batch}_over_batch_1": ratio, "tokens_match": tokens_match, "generated_tokens": reference_tokens,
                      "request_slots": engine.cache.max_requests, "passed": passed}))
    return 0 if passed else 1


def command_random(args) -> int:
    import torch
    from .config.llama import read_config_json
    from .registry import config_from_dict
    from . import models  # noqa: F401
    from .weights import write_random_model
    seed = parse_integer(args.rest[0], "SEED", 0)
    config = config_from_dict(read_config_json(args.prompt))
    dtype = torch.float32 if args.dtype == "float32" else torch.bfloat16
    write_random_model(args.model_dir, config, seed, dtype=dtype)
    print(json.dumps({"model_dir": args.model_dir, "seed": seed}))
    return 0


COMMANDS = {"generate": (command_generate, (1, 2)), "logits": (command_logits, (0, 0)),
            "benchmark": (command_benchmark, (4, 4)), "batch": (command_batch, (4, 4)), "random": (command_random, (1, 1))}


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    parser = argparse.ArgumentParser(add_help=False)
    parser.add_argument("--dtype", default="bfloat16")
    parser.add_argument("--temperature", type=float, default=0.0)
    parser.add_argument("--top-p", type=float, default=1.0)
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--max-cache-tokens", type=int, default=0)
    parser.add_argument("--page-size", type=int, default=0)
    parser.add_argument("--max-requests", type=int, default=0)
    parser.add_argument("--max-tokens-per-step", type=int, default=0)
    parser.add_argument("--chunk-size", type=int, default=0)
    parser.add_argument("--prompt-tokens-beside-decodes", type=int, default=0)
    parser.add_argument("--admit-partial", action="store_true")
    parser.add_argument("--prompts-file", default=None)
    parser.add_argument("--batch", type=int, default=4)
    parser.add_argument("--min-ratio", type=float, default=0.0)
    parser.add_argument("--expect-sha256", default=None)
    try:
        options, positional = parser.parse_known_args(argv)
    except SystemExit:
        sys.stderr.write(USAGE)
        return 1
    if not positional or positional[0] not in COMMANDS:
        sys.stderr.write(USAGE)
        return 1
    function, (least, most) = COMMANDS[positional[0]]
    if positional[0] in ("benchmark", "batch"):
        fixed, rest = positional[1:2], positional[2:]
        options.prompt = ""
    else:
        fixed, rest = positional[1:3], positional[3:]
        options.prompt = fixed[1] if len(fixed) > 1 else None
    if (positional[0] not in ("benchmark", "batch") and len(fixed) < 2) or not fixed or not least <= len(rest) <= most:
        sys.stderr.write("invalid tinyllama_amd command or arguments\n" + USAGE)
        return 1
    options.model_dir, options.rest = fixed[0], rest
    try:
        return function(options)
    except EngineError as error:
        print(error.to_json(), file=sys.stderr)
        return 1


if __name__ == "__main__":
    sys.exit(main())
