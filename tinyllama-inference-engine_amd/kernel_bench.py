"""Times the engine's kernels one by one at a model's layer sizes: `python bench.py --kernels`.

reference: benchmarks/kernel_benchmarks.cu:127-163 times each of its kernels at TinyLlama's sizes
(warm-up, samples, median and p95).  Here every kernel of a decode step of `batch` requests at
`context` positions and of a prompt step of `prompt` tokens is launched through its face in
`ops`, as the parts launch it.  A kernel's launches are recorded into a HIP graph that walks
through copies of its weights (more than the chip's caches hold, so every launch reads its weights
from memory as it does inside a step), the graph is replayed `samples` times, and a launch's time is
a replay's time divided by its launches: what a kernel costs inside a replayed step, dependent
launch included.
"""
from __future__ import annotations

import math
import statistics
from types import SimpleNamespace

import numpy as np
import torch

from . import ops

COPIES_BYTES = 640 << 20          # a kernel's weights are cycled through copies of at least this many bytes together


def _timed(build, copies: int, samples: int, warmup: int = 3):
    """build(i) launches the kernel on copy i.  Returns per-launch microseconds, one per sample."""
    for index in range(copies):
        build(index)                                         # eager once: allocations and plans are made
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for index in range(copies):
            build(index)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    times = []
    for run in range(warmup + samples):
        start.record()
        graph.replay()
        stop.record()
        stop.synchronize()
        if run >= warmup:
            times.append(start.elapsed_time(stop) * 1e3 / copies)
    return times


def _row(name, times, read_bytes=0, flops=0):
    times = sorted(times)
    median = statistics.median(times)
    row = {"kernel": name, "median_us": round(median, 2), "p95_us": round(times[min(len(times) - 1, int(0.95 * len(times)))], 2)}
    if read_bytes:
        row["mb"] = round(read_bytes / 1e6, 2)
        row["gbs"] = round(read_bytes / median / 1e3, 0)
    if flops:
        row["tflops"] = round(flops / median / 1e6, 1)
    return row


def _copies(nbytes: int) -> int:
    return max(2, min(96, -(-COPIES_BYTES // max(nbytes, 1))))


def bench_kernels(cfg: dict, batch: int = 8, context: int = 2048, prompt: int = 2048, samples: int = 20, device="cuda:0",
                  only: str | None = None) -> list[dict]:
    """cfg: a config.json's keys (sizes of the layer and the vocabulary).  Returns one row per kernel."""
    device = torch.device(device)
    torch.cuda.set_device(device)
    hidden, inter, vocab = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nq, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    d = cfg.get("head_dim") or hidden // nq
    eps, theta = cfg["rms_norm_eps"], cfg.get("rope_theta", 10000.0)
    page_size = 16
    bf = torch.bfloat16
    rows = []

    def rand(*shape, scale=0.02, dtype=bf):
        return (torch.randn(shape, device=device, dtype=torch.float32) * scale).to(dtype)

    def want(name):
        return only is None or only in name
    inv_freq = torch.pow(torch.tensor(theta, dtype=torch.float32), -2.0 * torch.arange(d // 2, dtype=torch.float32) / d).to(device)
    norm_weight = rand(hidden, scale=1.0)
    blocks = (context + page_size - 1) // page_size
    pages = batch * blocks
    cache = rand(pages, 2, nkv, page_size * d, scale=0.5)
    table = torch.arange(pages, dtype=torch.int32, device=device).view(batch, blocks).contiguous()
    positions = torch.full((batch,), context - 1, dtype=torch.int32, device=device)
    slot_map = (table[:, -1] * page_size + (context - 1) % page_size).to(torch.int32).contiguous()
    few = ops.few_rows_route(batch, bf)

    # ---- a decode step's kernels --------------------------------------------------------------------
    def normed_rows(width):
        xg = rand(batch, width, scale=1.0)
        ssq = torch.rand(((width + 15) // 16, 16), device=device, dtype=torch.float32) * 16.0
        return ops.NormedRows(xg, ssq, eps)
    label = f"decode b{batch}"
    shapes = {"qkv": ((nq + 2 * nkv) * d, hidden), "o": (hidden, nq * d), "gate_up": (2 * inter, hidden), "down": (hidden, inter),
              "head": (vocab, hidden)}
    if few:
        for name, (n, k) in shapes.items():
            if not want(name):
                continue
            count = _copies(n * k * 2)
            weights = [rand(n, k) for _ in range(count)]
            x = normed_rows(k) if name in ("qkv", "gate_up", "head") else rand(batch, k, scale=1.0)
            residual = torch.zeros((batch, n), dtype=torch.float32, device=device)
            rope = ops.RopeTarget(positions, slot_map, inv_freq, d, cache, nq, nkv, d)
            if name == "qkv":
                launch = lambda i: ops.gemm_rows(x, weights[i], None, "rope", rope=rope)
            elif name == "gate_up":
                launch = lambda i: ops.gemm_rows(x, weights[i], None, "silu")
            elif name == "head":
                launch = lambda i: ops.gemm_rows(x, weights[i], None, "store")
            else:
                launch = lambda i: ops.gemm_rows(x, weights[i], None, "residual", residual=residual, next_norm=(norm_weight, eps))
            rows.append(_row(f"{label}: gemm_rows {name} [{n} x {k}]", _timed(launch, count, samples), read_bytes=n * k * 2))
            del weights
    else:
        for name, (n, k) in shapes.items():
            if not want(name):
                continue
            count = _copies(n * k * 2)
            weights = [rand(n, k) for _ in range(count)]
            x = rand(batch, k, scale=1.0)
            if batch <= ops.SKINNY_MAX_ROWS and name == "gate_up":
                launch, kind = (lambda i: ops.gemm_skinny(x, weights[i], None, gated=True)), "gemm_skinny (gated)"
            elif batch <= ops.SKINNY_MAX_ROWS:
                launch, kind = (lambda i: ops.gemm_skinny(x, weights[i], None)), "gemm_skinny"
            else:
                launch, kind = (lambda i: ops.library_mm(x, weights[i], torch.float32 if name == "head" else bf)), "library"
            rows.append(_row(f"{label}: {kind} {name} [{n} x {k}]", _timed(launch, count, samples), read_bytes=n * k * 2))
            del weights
    if want("attention"):
        ctx = SimpleNamespace(max_new=1, num_seqs=batch, num_tokens=batch, max_context=context, scratch={}, tile_owner=None,
                              compute_units=int(torch.cuda.get_device_properties(device).multi_processor_count), host={})
        tiles, col_tiles, nsplit, split_len, waves, shared = ops.attention_plan(ctx, nq // nkv, nkv, d)
        kv_bytes = batch * context * 2 * nkv * d * 2
        count = _copies(kv_bytes)
        caches = [rand(pages, 2, nkv, page_size * d, scale=0.5) for _ in range(count)]
        q = rand(batch, nq * d, scale=1.0)
        launch = lambda i: ops.attention_mfma(q, caches[i], table, tiles, positions, nq, nkv, d, None, d ** -0.5, nsplit, split_len,
                                              col_tiles, waves, shared)
        rows.append(_row(f"{label}: attention + merge, {context} positions ({nsplit} parts x {waves} waves)",
                         _timed(launch, count, samples), read_bytes=kv_bytes))
        del caches
    if want("embed") and few:
        table_rows = rand(vocab, hidden)
        tokens = torch.randint(0, vocab, (batch,), dtype=torch.int32, device=device)
        rows.append(_row(f"{label}: embed_rows", _timed(lambda i: ops.embed_rows(tokens, table_rows, (norm_weight, eps)), 8, samples)))
    if want("sample"):
        logits = rand(batch, vocab, scale=1.0, dtype=torch.float32)
        rows.append(_row(f"{label}: sample (greedy) [{batch} x {vocab}]", _timed(lambda i: ops.sample(logits), 8, samples),
                         read_bytes=batch * vocab * 4))

    # ---- a prompt step's kernels ----------------------------------------------------------------------
    if prompt > 0:
        label = f"prompt {prompt}"
        x_by_width = {}
        for name, (n, k) in shapes.items():
            if name == "head" or not want(name):
                continue
            count = _copies(n * k * 2)
            weights = [rand(n, k) for _ in range(count)]
            x = x_by_width.setdefault(k, rand(prompt, k, scale=1.0))
            rows.append(_row(f"{label}: library product {name} [{prompt} x {n} x {k}]",
                             _timed(lambda i: ops.library_mm(x, weights[i]), count, samples), flops=2.0 * prompt * n * k))
            del weights
        if want("attention"):
            blocks_p = (prompt + page_size - 1) // page_size
            cache_p = rand(blocks_p, 2, nkv, page_size * d, scale=0.5)
            table_p = torch.arange(blocks_p, dtype=torch.int32, device=device).view(1, blocks_p)
            positions_p = torch.arange(prompt, dtype=torch.int32, device=device)
            host = {"seq_start": np.asarray([0, prompt], dtype=np.int32), "seq_len": np.asarray([prompt], dtype=np.int32)}
            ctx = SimpleNamespace(max_new=prompt, num_seqs=1, num_tokens=prompt, max_context=prompt, scratch={}, tile_owner=None,
                                  compute_units=int(torch.cuda.get_device_properties(device).multi_processor_count), host=host,
                                  tokens=positions_p)
            tiles, col_tiles, nsplit, split_len, waves, shared = ops.attention_plan(ctx, nq // nkv, nkv, d)
            q = rand(prompt, nq * d, scale=1.0)
            launch = lambda i: ops.attention_mfma(q, cache_p, table_p, tiles, positions_p, nq, nkv, d, None, d ** -0.5, nsplit,
                                                  split_len, col_tiles, waves, shared)
            rows.append(_row(f"{label}: attention ({col_tiles} column groups, {waves} waves, shared {shared})",
                             _timed(launch, 4, samples), flops=4.0 * nq * d * prompt * (prompt + 1) / 2))
        if want("norm"):
            residual = rand(prompt, hidden, scale=1.0, dtype=torch.float32)
            delta = ops.Product(rand(prompt, hidden, scale=1.0), 1)
            rows.append(_row(f"{label}: add + rmsnorm [{prompt} x {hidden}]",
                             _timed(lambda i: ops.add_rmsnorm(residual, delta, norm_weight, eps, bf), 4, samples),
                             read_bytes=prompt * hidden * (4 + 2 + 4 + 2)))
        if want("silu"):
            gate_up = ops.Product(rand(prompt, 2 * inter, scale=1.0), 1)
            rows.append(_row(f"{label}: silu * up [{prompt} x {inter}]",
                             _timed(lambda i: ops.silu_mul(gate_up, bf, interleaved=True), 4, samples), read_bytes=prompt * inter * 6))
        if want("rope"):
            blocks_p = (prompt + page_size - 1) // page_size
            cache_p = rand(blocks_p, 2, nkv, page_size * d, scale=0.5)
            positions_p = torch.arange(prompt, dtype=torch.int32, device=device)
            qkv = ops.Product(rand(prompt, (nq + 2 * nkv) * d, scale=1.0), 1)
            rows.append(_row(f"{label}: rotation + cache write",
                             _timed(lambda i: ops.rope_cache(qkv, positions_p, positions_p, inv_freq, d, cache_p, nq, nkv, d, bf, paired=True),
                                    4, samples), read_bytes=prompt * (nq + 2 * nkv) * d * 4))
    return rows
