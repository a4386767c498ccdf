"""The engine: a model folder in, a step function and generation out.

`Engine(model_dir)` reads config.json, finds the architecture in the registry, checks and loads
the weights, builds the model from its parts, makes the cache pools, and offers
  step(entries)      the step function (see engine/step.py)
  admit / finish     a request's slot and pages
  generate(...)      prompts to tokens through the scheduler and the sampler
"""
from __future__ import annotations

from typing import Hashable, Sequence

import torch

from .. import models as _models  # noqa: F401  (registers architectures and parts)
from ..cache.manager import CacheManager
from ..config.llama import read_config_json
from ..errors import EngineError, ErrorCode, device_memory_errors, invalid_argument
from ..models.builder import build_model, expected_tensors
from ..registry import config_from_dict
from ..weights.store import WeightStore
from ..sampling.sampler import Sampler
from .scheduler import Request, SamplingParams, Scheduler
from .step import ModelRunner, StepEntry, StepTimings

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "f32": torch.float32,
           "fp32": torch.float32}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name in (torch.bfloat16, torch.float32):
            return name
    elif str(name).lower() in _DTYPES:
        return _DTYPES[str(name).lower()]
    raise EngineError(ErrorCode.INVALID_DTYPE, f"the engine runs in bfloat16 or float32, not {name}")


class Engine:
    def __init__(self, model_dir: str | None, dtype="bfloat16", max_tokens: int | None = 4096, page_size: int = 16,
                 max_requests: int = 64, device: str = "cuda:0", config: dict | None = None,
                 random_seed: int | None = None, use_graphs: bool = True, expect_sha256: str | None = None,
                 capture_graphs: bool = True, max_weight_file_bytes: int | None = None, max_cache_bytes: int | None = None,
                 cache_fraction: float | None = None):
        """max_tokens: how many positions the cache pools hold in all (rounded up to whole
        pages); max_requests: how many requests can be live at once.  Instead of max_tokens
        (None), cache_fraction sizes the pools as that share of the device memory that is free once
        the weights are loaded.  max_weight_file_bytes and max_cache_bytes are budgets: a folder or
        a pool beyond them is `out_of_memory` before anything is mapped or allocated.

        Without a folder, `config` (the contents of a config.json) and `random_seed` give a model
        of random weights drawn on the device, with no file in between (for measurements).
        expect_sha256: the digest the folder's weight file must have (`checksum_mismatch` otherwise).
        use_graphs=False: no step is recorded or padded to a recording's size.  capture_graphs=False:
        steps are padded and laid out as for a recording but launched kernel by kernel (for checks)."""
        if not torch.cuda.is_available():
            raise EngineError(ErrorCode.HIP, "no GPU is visible: the engine has no CPU path")
        self.dtype = parse_dtype(dtype)
        self.device = torch.device(device)
        torch.cuda.set_device(self.device)
        if model_dir is not None:
            self.config = config_from_dict(read_config_json(model_dir))
            self.spec = self.config.to_spec()
            store = WeightStore(model_dir, max_file_bytes=max_weight_file_bytes)
            if expect_sha256 is not None:
                store.expect_sha256(expect_sha256)
            with device_memory_errors("the weights"):
                weights = store.resident(expected_tensors(self.spec), self.dtype, self.device, self.spec.ignored_tensors)
        else:
            if config is None or random_seed is None:
                raise invalid_argument("without a model folder the engine needs a config and a random seed")
            from ..weights.random_init import resident_random_tensors
            self.config = config_from_dict(config)
            self.spec = self.config.to_spec()
            with device_memory_errors("the weights"):
                weights = resident_random_tensors(expected_tensors(self.spec), random_seed, dtype=self.dtype, device=self.device)
        with device_memory_errors("the weights"):
            self.model = build_model(self.spec, weights, self.dtype, self.device)
        self.weight_arena = weights.arena                  # the one allocation that holds what the parts kept
        needs = self.model.run_needs()
        if max_tokens is None:
            if cache_fraction is None or not 0.0 < cache_fraction <= 1.0:
                raise invalid_argument("without max_tokens the engine needs a cache_fraction in (0, 1]")
            free, _ = torch.cuda.mem_get_info(self.device)
            per_page = CacheManager.page_bytes(needs, page_size, self.dtype)
            num_pages = int(free * cache_fraction) // per_page if per_page else 1
            if num_pages <= 0:
                raise EngineError(ErrorCode.OUT_OF_MEMORY, f"{cache_fraction} of the {free} free bytes do not hold one page of {per_page}")
        else:
            if max_tokens <= 0:
                raise invalid_argument("max_tokens must be positive")
            num_pages = (max_tokens + page_size - 1) // page_size
        with device_memory_errors(f"cache pools of {num_pages} pages"):
            self.cache = CacheManager(needs, page_size, num_pages, max_requests, self.dtype, self.device,
                                      max_positions=self.spec.max_positions, max_bytes=max_cache_bytes)
        self.runner = ModelRunner(self.model, self.cache, use_graphs=use_graphs, capture=capture_graphs)
        self.sampler = Sampler(self.device, capacity=max(max_requests, 1))
        self.runner.device_tokens = self.sampler.device_tokens
        self.stats = {"steps": 0, "steps_ahead": 0}      # steps run by `run`; those whose tokens were read a step later

    # ---- the step function and what goes with it --------------------------------------------------
    def admit(self, request: Hashable) -> int:
        return self.cache.admit(request)

    def finish(self, request: Hashable) -> None:
        self.cache.release(request)

    def step(self, entries: Sequence[StepEntry], timings: StepTimings | None = None, trace: dict | None = None,
             check_finite: bool = False, trace_serving_route: bool = False) -> torch.Tensor:
        """One step of the model: see `ModelRunner.step`.  The logits are the caller's own (those
        of a step replayed from a recording are copied out of the recording's memory).  `trace`: a
        dict that receives the step's intermediate tensors by the names of the reference's ModelTrace,
        all of them; with trace_serving_route a bfloat16 step of at most 16 tokens takes the route it
        takes in serving (norms folded into the products) and leaves the names that exist there.
        check_finite: a NaN or an infinity among the logits is `numerical_error`, as the reference
        checks what it returns (src/cuda/model.cu:505-510); the step then waits for the device (the
        sampling kernel's test of a row runs over the logits and its marks are read)."""
        logits = self.runner.step(entries, timings, trace=trace, trace_serving_route=trace_serving_route)
        if check_finite and logits.shape[0] > 0:
            from ..ops import sample
            marks = sample(logits)
            if int(marks.min().item()) < 0:
                raise EngineError(ErrorCode.NUMERICAL, "the step's logits hold a NaN or an infinity")
        return logits

    # ---- generation -------------------------------------------------------------------------------
    def generate(self, prompts: Sequence[Sequence[int]], max_tokens: int = 16, temperature: float = 0.0,
                 top_p: float = 1.0, seed: int = 0, stop_on_eos: bool = False, max_tokens_per_step: int = 2048,
                 max_seqs_per_step: int | None = None, chunk_size: int | None = None,
                 timings: dict | None = None, stats: dict | None = None,
                 prompt_tokens_beside_decodes: int | None = None, admit_partial: bool = False) -> list[list[int]]:
        """Token ids in, generated token ids out, one list per prompt.  Request i samples with
        seed + i.  All prompts run together under the scheduler (continuous batching, prompts cut
        into portions under the token budget).  `timings`: a dict that receives the sums of the
        steps' compute and transfer times, apart for steps that bring prompt tokens and steps that
        only decode (the keys of the reference's `generate`, app/cuda_reference.cu:216-224).
        `stats`: a dict that receives what the scheduler counted (steps, prompt and decoded tokens,
        preemptions) and how many matrix products of this process fell from the vendor's library to the
        plain kernel (`library_fallbacks`).  prompt_tokens_beside_decodes, admit_partial: see `Scheduler`."""
        scheduler = Scheduler(self.cache, max_tokens_per_step=max_tokens_per_step,
                              max_seqs_per_step=max_seqs_per_step or self.cache.max_requests, chunk_size=chunk_size,
                              max_positions=self.spec.max_positions, eos_token_id=self.spec.eos_token_id,
                              prompt_tokens_beside_decodes=prompt_tokens_beside_decodes, admit_partial=admit_partial)
        requests = []
        for index, prompt in enumerate(prompts):
            params = SamplingParams(max_tokens=max_tokens, temperature=temperature, top_p=top_p, seed=seed + index,
                                    stop_on_eos=stop_on_eos)
            request = Request(id=("generate", index), prompt=[int(token) for token in prompt], params=params)
            scheduler.add(request)
            requests.append(request)
        try:
            self.run(scheduler, timings)
            if stats is not None:
                from ..ops import library_fallbacks
                stats.update(scheduler.stats)
                stats["library_fallbacks"] = library_fallbacks()    # products that fell to the plain kernel so far (slow: should be 0)
        except BaseException:
            # a step raised (no request can move, a NaN in the logits, a device error): what this
            # call's requests hold goes back, so that the engine can be used again
            for request in requests:
                if self.cache.is_live(request.id):
                    self.cache.release(request.id)
            raise
        return [request.generated for request in requests]

    def run(self, scheduler: Scheduler, timings: dict | None = None, max_steps: int | None = None) -> int:
        """The engine loop: plan a step, run it, sample, record; until nothing is left, or for
        `max_steps` steps.  Returns the number of steps run.

        The host stays one step behind the device where it can: a decode step's tokens are the
        last step's samples, which the recorded step takes from the sampler's device buffer, so
        the step is launched before those tokens have been read; they are read (and written into
        their requests) while it runs.  What the next plan depends on is known without them,
        unless a request stops at the end-of-sequence token or the plan has to recompute a
        preempted request: then the loop waits for the tokens first."""
        sampler = self.sampler
        if timings is not None:
            for key in ("prefill_compute_ms", "prefill_transfer_ms", "decode_compute_ms", "decode_transfer_ms"):
                timings.setdefault(key, 0.0)
        steps = 0
        behind = None            # (plan, PendingTokens, {request id: row}) of a step whose tokens the requests still lack

        def settle():
            nonlocal behind
            if behind is not None:
                scheduler.resolve(behind[0], behind[1].read())
                behind = None

        try:
            while scheduler.has_work() and (max_steps is None or steps < max_steps):
                plan = scheduler.schedule()
                if not plan:
                    raise EngineError(ErrorCode.OUT_OF_MEMORY, "no request can make progress with the pages that are free")
                sources = self._device_sources(plan, behind)
                if sources is None:
                    settle()
                    sources = [None] * len(plan)
                entries = [StepEntry(item.request.id,
                                     [0] if source is not None else item.request.token_slice(item.first, item.count),
                                     [item.count - 1] if item.samples else [], source)
                           for item, source in zip(plan, sources)]
                if timings is None:
                    logits = self.runner.step(entries, keep=False)
                else:
                    measured = StepTimings()
                    logits = self.runner.step(entries, measured, keep=False)
                    phase = "decode" if all(item.count == 1 and item.samples and item.request.generated for item in plan) else "prefill"
                    timings[phase + "_compute_ms"] += measured.compute_ms
                    timings[phase + "_transfer_ms"] += measured.transfer_ms
                sampling = [item for item in plan if item.samples]
                pending = sampler.sample_async(logits, [item.request.params for item in sampling],
                                               [len(item.request.generated) for item in sampling])
                settle()                                      # the step before this one, while this one runs
                steps += 1
                self.stats["steps"] += 1
                if scheduler.can_defer(plan) and sampling:
                    scheduler.update(plan, None)
                    behind = (plan, pending, {item.request.id: row for row, item in enumerate(sampling)})
                    self.stats["steps_ahead"] += 1
                else:
                    scheduler.update(plan, pending.read())
        except BaseException:
            if behind is not None:
                # the requests get the tokens that were sampled for them before the step that raised;
                # what reading them raises in turn (a NaN in that step's logits, say) must not
                # take the place of the error already on its way
                plan, pending, _ = behind
                behind = None
                try:
                    scheduler.resolve(plan, pending.read())
                except Exception:
                    pass
            raise
        if behind is not None:
            plan, pending, _ = behind
            behind = None
            scheduler.resolve(plan, pending.read())
        return steps

    def _device_sources(self, plan, behind):
        """For a plan whose step the recording replays: per item the row of the sampler's device
        tokens that is its token (None: the token is on the host).  None when some token that the
        plan needs is neither on the host nor a row of the last step's samples, or the step is
        not replayed."""
        if behind is None:
            return [None] * len(plan)
        rows = behind[2]
        sources = []
        for item in plan:
            request = item.request
            if not (request.pending and item.first + item.count == request.total):
                sources.append(None)                          # its tokens are all on the host
            elif item.count == 1 and request.id in rows:
                sources.append(rows[request.id])
            else:
                return None
        if any(source is not None for source in sources):
            if not (all(item.count == 1 and item.samples for item in plan) and self.runner.replays_single_tokens(len(plan))):
                return None
        return sources
