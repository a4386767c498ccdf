"""The command line, in the manner of the reference's `tinyllama_cuda` (app/cuda_reference.cu:475-522)
and `tinyllama_reference` (app/reference_cli.cpp:40-125): positional arguments, JSON on standard
output, and errors as one JSON line `{"error": {"code", "message"}}` on standard error with a
non-zero exit status.

    tinyllama_amd generate  MODEL_DIR PROMPT MAX_TOKENS [GOLDEN_JSON]
    tinyllama_amd logits    MODEL_DIR PROMPT
    tinyllama_amd benchmark MODEL_DIR CONTEXT OUTPUT_TOKENS WARMUP SAMPLES
    tinyllama_amd random    MODEL_DIR CONFIG_JSON SEED          (writes a folder of random weights)

PROMPT is text when MODEL_DIR holds a tokenizer.model (the begin-of-sequence id is put in front,
as the reference does), or token ids written `ids:1,15043,3186`.  GOLDEN_JSON, when given, holds
`{"greedy_tokens": [...]}` and the generated tokens must begin it (app/cuda_reference.cu:198-211).
Options (after the positionals): --dtype bfloat16|float32, --temperature T, --top-p P, --seed S
(the reference's request options of the same names, app/server.cpp:601-613), --max-cache-tokens N.
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
         "       tinyllama_amd random MODEL_DIR CONFIG_JSON SEED\n"
         "options: [--dtype bfloat16|float32] [--temperature T] [--top-p P] [--seed S] [--max-cache-tokens N]\n"
         "         [--expect-sha256 HEX]\n")


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


def _engine(args, positions: int):
    from .engine import Engine
    return Engine(args.model_dir, dtype=args.dtype, max_tokens=args.max_cache_tokens or max(64, positions),
                  max_requests=4, expect_sha256=args.expect_sha256)


def command_generate(args) -> int:
    max_tokens = parse_integer(args.rest[0], "MAX_TOKENS", 1)
    ids, tokenizer = prompt_ids(args.model_dir, args.prompt)
    engine = _engine(args, len(ids) + max_tokens)
    started = time.perf_counter()
    timings = {}
    generated = engine.generate([ids], max_tokens=max_tokens, temperature=args.temperature, top_p=args.top_p,
                                seed=args.seed, timings=timings)[0]
    elapsed = (time.perf_counter() - started) * 1e3
    if len(args.rest) > 1:
        try:
            with open(args.rest[1], "r", encoding="utf-8") as handle:
                expected = json.load(handle)["greedy_tokens"]
        except (OSError, ValueError, KeyError):
            raise EngineError(ErrorCode.IO, "unable to open golden metadata") from None
        if len(generated) > len(expected) or list(expected[:len(generated)]) != generated:
            raise EngineError(ErrorCode.NUMERICAL, "greedy tokens do not match the golden tokens")
    result = {"prompt_tokens": len(ids), "generated_tokens": generated, "wall_ms": elapsed, **timings}
    if tokenizer is not None:
        result["text"] = tokenizer.decode(generated)
    print(json.dumps(result))
    return 0


def command_logits(args) -> int:
    from .engine import StepEntry
    ids, _ = prompt_ids(args.model_dir, args.prompt)
    engine = _engine(args, len(ids))
    engine.admit("logits")
    logits = engine.step([StepEntry("logits", ids, [len(ids) - 1])])
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
            "benchmark": (command_benchmark, (4, 4)), "random": (command_random, (1, 1))}


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    parser = argparse.ArgumentParser(add_help=False)
    parser.add_argument("--dtype", default="bfloat16")
    parser.add_argument("--temperature", type=float, default=0.0)
    parser.add_argument("--top-p", type=float, default=1.0)
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--max-cache-tokens", type=int, default=0)
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
    if positional[0] == "benchmark":
        fixed, rest = positional[1:2], positional[2:]
        options.prompt = ""
    else:
        fixed, rest = positional[1:3], positional[3:]
        options.prompt = fixed[1] if len(fixed) > 1 else None
    if (positional[0] != "benchmark" and len(fixed) < 2) or not fixed or not least <= len(rest) <= most:
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
