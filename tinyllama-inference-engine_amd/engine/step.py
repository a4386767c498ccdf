"""The step function: one batch of (request, its next tokens) through the model, from the cache.

reference: `ForwardBatch(tokens, positions, kv_slots)` (src/cuda/model.cu:531-725) takes one
token per sequence, checks batch size, token range, slot range, that positions continue where the
slot stopped, and that no slot comes twice (:539-561), runs the rows as one batch, returns the
logits of every row, and moves `next_positions` only after success (:721-723).  Here an entry
brings any number of next tokens (a portion of a prompt, or one decoded token), the positions are
the cache manager's, logits come back only for the wanted places, and the request's length moves
after the step is enqueued.
"""
from __future__ import annotations

import gc
import weakref
from dataclasses import dataclass, field
from typing import Hashable, Sequence

import numpy as np
import torch

from ..cache.manager import ABSENT, CacheManager
from ..ops import feed_tokens as ops_feed_tokens
from ..errors import invalid_argument, out_of_bounds, out_of_memory


@dataclass
class StepEntry:
    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=list)    # places among `tokens` whose logits are asked for
    # The entry's one token is not on the host yet: it is row `source` of the device tokens that
    # the last step's sampling left (`ModelRunner.device_tokens`); `tokens` then holds a stand-in.
    # Only a step of single tokens that is replayed from a recording takes such entries.
    source: int | None = None


@dataclass
class StepTimings:
    """Where a step's time went, in milliseconds, when asked for (the step then waits for the
    device before it returns).  reference: CudaStepTimings, compute / transfer / wall
    (include/tlie/cuda/model.hpp:14-18), filled by ForwardBatch (src/cuda/model.cu:512-526).
    transfer: the step's arrays to the device (logits stay on the device here); compute: the
    model's kernels; wall: the whole call on the host, with validation and page reservation."""
    compute_ms: float = 0.0
    transfer_ms: float = 0.0
    wall_ms: float = 0.0


@dataclass
class GroupView:
    """One page group as the kernels see it in this step."""
    block_table: torch.Tensor      # int32 [sequences, max_blocks]; absent entries hold page 0 and are never read
    slot_map: torch.Tensor         # int32 [tokens]: cache row of each token
    max_blocks: int


@dataclass
class StepContext:
    """Everything a part may need to know about the step, on the device (and on the host).

    A step that is replayed from a recording is padded to the recording's size.  Padding tokens
    (those from index seq_start[num_seqs] on) are token 0 at position 0, belong to no request
    (`token_slot` -1), are written nowhere (slot maps -1) and their results are dropped; padding
    sequences have `seq_slot` -1 and, in a step of portions, no tokens.  A part that keeps state
    per request must change it only for tokens and sequences whose slot is not negative, and must
    not let a padding token's activations reach a live token's: they may hold anything (a kernel
    may leave the rows of tokens that belong to no sequence unwritten), also values that are not
    finite, so they are selected away, not multiplied by zero."""
    num_tokens: int
    num_seqs: int
    num_wanted: int
    max_new: int                   # most tokens any sequence brings
    max_context: int               # longest sequence after this step
    tokens: torch.Tensor           # int32 [T]
    positions: torch.Tensor        # int32 [T] absolute position of each token in its sequence
    token_seq: torch.Tensor        # int32 [T] index of the token's sequence in this step
    no_slots: torch.Tensor         # int32 [T] of -1: a slot map that writes nothing
    seq_start: torch.Tensor        # int32 [S + 1] first token of each sequence among the T
    seq_first_pos: torch.Tensor    # int32 [S] position of its first token
    seq_len: torch.Tensor          # int32 [S] length after this step
    seq_slot: torch.Tensor         # int32 [S] request slot (row of the state areas); -1: a padding sequence
    token_slot: torch.Tensor       # int32 [T] request slot of the token's sequence; -1: a padding token
    want_rows: torch.Tensor        # int32 [num_wanted] token indices
    groups: list[GroupView]
    host: dict                     # the same arrays as numpy, by name
    wants_all_rows: bool = False   # the wanted rows are all the step's tokens, in order
    compute_units: int = 256       # of the device: how many workgroups start at once
    # a recorded step of prompt portions: work lists that parts make on the host live at fixed
    # addresses, at a fixed size (the recording's owner keeps them: `tiles_for(key, list) -> tensor`,
    # and makes them again for every replay); None: a list per step
    tile_owner: object = None
    # a dict that receives named copies of the step's intermediate tensors (such a step is never
    # replayed from a recording and takes no fused route), and the name's prefix for the layer that runs
    trace: dict | None = None
    trace_prefix: str = ""
    # with a trace: False, every name of the trace is left (no norm is folded into a product); True, the step
    # takes the route it would take without a trace and leaves the names that exist as tensors there
    trace_serving_route: bool = False
    # what parts keep for the length of this step, under keys of their own (work lists that several
    # layers share, say); the step function never looks inside
    scratch: dict = field(default_factory=dict)


class ModelRunner:
    def __init__(self, model, cache: CacheManager, use_graphs: bool = True, capture: bool = True):
        self.model = model
        self.cache = cache
        self.device = model.device
        self.vocab_size = model.spec.vocab_size
        # Steps of up to some hundred tokens are bound by launches, not by the kernels (the host
        # needs some 15 us a launch, the library's products 20): a step of single tokens is captured
        # once per batch-size bucket and range of sequence lengths as a HIP graph and replayed, and
        # so is a step of prompt portions per (tokens, sequences, range of lengths) padded up.
        # Parts say whether they may be captured (`graph_safe`).
        self.use_graphs = use_graphs and getattr(model, "graph_safe", False) and torch.device(self.device).type == "cuda"
        # capture=False: the steps a recording would serve are still padded to its sizes and run on
        # its fixed arrays, but launched kernel by kernel every time (what a replay must equal bit for bit)
        self.capture = capture
        self.device_tokens: torch.Tensor | None = None     # int32, where sampling leaves a step's tokens (set by the engine)
        self._graphs: dict[tuple[int, int], "DecodeGraph"] = {}      # by (most sequences, longest sequence)
        self._portion_graphs: dict[tuple[int, int, int], "PortionGraph"] = {}   # by (most tokens, most sequences, longest sequence)

    # ---- checks and context ------------------------------------------------------------------
    def _validate(self, entries: Sequence[StepEntry]) -> None:
        if not entries:
            raise invalid_argument("a step needs at least one entry")
        seen = set()
        for entry in entries:
            if entry.request in seen:
                raise invalid_argument(f"request {entry.request!r} comes twice in one step")
            seen.add(entry.request)
            if len(entry.tokens) == 0:
                raise invalid_argument(f"request {entry.request!r} brings no tokens")
            if entry.source is not None and (self.device_tokens is None or len(entry.tokens) != 1
                                             or not 0 <= entry.source < self.device_tokens.shape[0]):
                raise invalid_argument(f"request {entry.request!r} names a device token that is not there")
            for token in entry.tokens:
                if not 0 <= int(token) < self.vocab_size:
                    raise out_of_bounds(f"token {token} of request {entry.request!r} is outside the vocabulary of {self.vocab_size}")
            for place in entry.want:
                if not 0 <= int(place) < len(entry.tokens):
                    raise out_of_bounds(f"wanted place {place} of request {entry.request!r} is not among its {len(entry.tokens)} tokens")
            if not self.cache.is_live(entry.request):
                raise invalid_argument(f"request {entry.request!r} is not live (admit it first)")
            limit = self.cache.max_positions
            if limit is not None and self.cache.length(entry.request) + len(entry.tokens) > limit:
                raise out_of_bounds(f"request {entry.request!r} would pass the model's {limit} positions")

    def build_context(self, entries: Sequence[StepEntry]) -> StepContext:
        return build_context(self.cache, entries, self.device)

    def _length_bucket(self, longest: int) -> int:
        """The sequence length a recording is made for: the next power of two from 256 on, up to
        what the cache can hold.  How attention cuts the keys is fixed in a recording, for its
        longest sequence: one recording for the model's whole range would serve short sequences
        of a long-range model with a handful of workgroups."""
        limit = self.cache.max_positions or self.cache.num_pages * self.cache.page_size
        bucket = 256
        while bucket < longest:
            bucket *= 2
        return min(bucket, max(limit, longest))

    def replays_single_tokens(self, count: int) -> bool:
        """Whether a recording serves a step of `count` entries of one token each, every logit wanted."""
        return self.use_graphs and count <= DecodeGraph.MAX_BATCH

    def replays(self, entries: Sequence[StepEntry]) -> bool:
        """Whether the step is one of single tokens, every logit wanted, that a recording serves."""
        return (self.replays_single_tokens(len(entries))
                and all(len(entry.tokens) == 1 and list(entry.want) == [0] for entry in entries))

    def records(self, entries: Sequence[StepEntry]) -> tuple[int, int] | None:
        """For a step of prompt portions (beside single tokens, if any) that a recording serves:
        the recording's (tokens, sequences); else None.  Such steps are bound by the host, which
        needs some 15 us a launch, up to several hundred tokens; a recording pads the step to its
        own size, so there are recordings in steps of 64 tokens, up to `PortionGraph.MAX_TOKENS`,
        for up to 8 or up to 64 sequences, with as many wanted rows as sequences at most."""
        if not self.use_graphs or any(entry.source is not None for entry in entries):
            return None
        total, wanted = sum(len(entry.tokens) for entry in entries), sum(len(entry.want) for entry in entries)
        if total > PortionGraph.MAX_TOKENS or len(entries) > PortionGraph.MAX_SEQS:
            return None
        tokens = 16 if total <= 16 else (32 if total <= 32 else (total + 63) // 64 * 64)
        seqs = min(tokens, 8 if len(entries) <= 8 else PortionGraph.MAX_SEQS)
        return (tokens, seqs) if wanted <= seqs else None

    # ---- the step ----------------------------------------------------------------------------
    def step(self, entries: Sequence[StepEntry], timings: StepTimings | None = None, keep: bool = True,
             trace: dict | None = None, trace_serving_route: bool = False) -> torch.Tensor:
        """Runs exactly the tokens the entries bring, as one batch, from the cache that earlier
        steps left.  Returns float32 logits [wanted places, vocab] on the device, in the order of
        the entries and of each entry's `want`.  With `timings` the step is timed with events
        on its stream and waits for them before it returns.  keep=False: the logits may lie in
        a recording's memory, which the recording's next replay writes again (for a caller that
        has used them up by then); otherwise they are the caller's own.  trace: a dict that
        receives the step's intermediate tensors by name (see `DecoderModel.forward`); the step
        is then launched kernel by kernel, and, unless trace_serving_route is set, on the route
        that leaves every name (a bfloat16 step of few tokens would otherwise fold its norms into
        its products)."""
        marks = None
        if timings is not None:
            import time
            started = time.perf_counter()
            marks = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
        self._validate(entries)
        wanted = [(entry.request, len(entry.tokens)) for entry in entries]
        if not self.cache.reserve_all(wanted):
            raise out_of_memory(f"the step needs more pages than are free ({self.cache.free_pages()} free)")
        try:
            if marks:
                marks[0].record()
            if trace is None and self.replays(entries):
                longest = max(self.cache.length(request) + count for request, count in wanted)
                key = (DecodeGraph.bucket_of(len(entries)), self._length_bucket(longest))
                if key not in self._graphs:
                    self._graphs[key] = DecodeGraph(self, *key)
                logits = self._graphs[key].run(entries, marks[1] if marks else None)
                if keep:
                    logits = logits.clone()
            elif trace is None and (sizes := self.records(entries)) is not None:
                longest = max(self.cache.length(request) + count for request, count in wanted)
                key = (*sizes, self._length_bucket(longest))
                if key not in self._portion_graphs:
                    self._portion_graphs[key] = PortionGraph(self, *key)
                logits = self._portion_graphs[key].run(entries, marks[1] if marks else None)
                if keep:
                    logits = logits.clone()
            else:
                if any(entry.source is not None for entry in entries):
                    raise invalid_argument("a token that is still on the device can only feed a replayed decode step")
                ctx = self.build_context(entries)
                ctx.trace = trace
                ctx.trace_serving_route = trace_serving_route
                if marks:
                    marks[1].record()
                logits = self.model.forward(ctx, self.cache.bindings)
            if marks:
                marks[2].record()
                marks[2].synchronize()
                timings.transfer_ms = marks[0].elapsed_time(marks[1])
                timings.compute_ms = marks[1].elapsed_time(marks[2])
                timings.wall_ms = (time.perf_counter() - started) * 1e3
        except BaseException:
            # nothing of the step counts: the pages it reserved go back (the requests keep what
            # their committed positions lie on), so that a later step finds the lists it expects
            for request, _ in wanted:
                self.cache.unreserve(request)
            for recording in (*self._graphs.values(), *self._portion_graphs.values()):
                recording.forget()                      # (a page list that shrank and grew again is not the list a row remembers)
            raise
        for request, count in wanted:
            self.cache.commit(request, count)
        return logits


class DecodeGraph:
    """A decode step for up to `bucket` sequences, one token each, every token's logits wanted:
    the step's arrays live at fixed addresses, the model's kernels are recorded once into a HIP
    graph and replayed with new contents.  Rows beyond the step's sequences are padding: token 0
    at position 0 of a sequence with no page written (slot -1), whose results are dropped.
    How the attention kernel cuts the key range is fixed at capture, for sequences up to
    `longest` positions (the runner keeps a recording per power of two); each part computes its own
    bounds from the positions on the device."""
    MAX_BATCH = 256         # beyond, a step's kernels take longer than the host needs to launch them

    @staticmethod
    def bucket_of(count: int) -> int:
        bucket = 1
        while bucket < count:
            bucket *= 2
        return bucket

    def __init__(self, runner: "ModelRunner", bucket: int, longest: int, seqs: int | None = None):
        # bucket: the recording's tokens; seqs: its sequences (None: as many, one token each).
        # The runner owns its recordings; a recording that owned its runner in turn would make the
        # pair garbage that only the cycle collector frees, at a moment of its choosing: if that
        # moment falls inside another recording's capture, the graph's destructor (which waits for
        # the device) is an operation the capture forbids, and the process ends.
        self._runner = weakref.ref(runner)
        self.bucket = bucket
        single = seqs is None
        seqs = bucket if single else seqs
        self.seqs = seqs
        cache = runner.cache
        self.longest = longest
        self.widths = [max(1, (longest + cache.page_size - 1) // cache.page_size) for _ in cache.groups]
        layout = [("tokens", (bucket,)), ("positions", (bucket,)), ("token_seq", (bucket,)), ("no_slots", (bucket,)),
                  ("seq_start", (seqs + 1,)), ("seq_first_pos", (seqs,)), ("seq_len", (seqs,)), ("seq_slot", (seqs,)),
                  ("token_slot", (bucket,)), ("want_rows", (seqs,)), ("token_source", (bucket,))]
        for group, width in enumerate(self.widths):
            layout += [(f"block_table{group}", (seqs, width)), (f"slot_map{group}", (bucket,))]
        total = sum(int(np.prod(shape)) for _, shape in layout)
        self.pinned = torch.zeros(total, dtype=torch.int32, pin_memory=True)
        self.device_flat = torch.zeros(total, dtype=torch.int32, device=runner.device)
        flat = self.pinned.numpy()
        self.host, views, cursor = {}, {}, 0
        for name, shape in layout:
            size = int(np.prod(shape))
            self.host[name] = flat[cursor:cursor + size].reshape(shape)
            views[name] = self.device_flat[cursor:cursor + size].view(shape)
            cursor += size
        if single:
            self.host["token_seq"][:] = np.arange(bucket)
            self.host["seq_start"][:] = np.arange(bucket + 1)
            self.host["want_rows"][:] = np.arange(bucket)
        self.host["no_slots"][:] = -1
        self.host["token_source"][:] = -1
        self.host["seq_slot"][:] = -1
        self.host["token_slot"][:] = -1
        self.token_source = views["token_source"]
        self.copied = torch.cuda.Event()                    # the last transfer of the pinned buffer has been made
        self.copy_pending = False
        groups = [GroupView(views[f"block_table{group}"], views[f"slot_map{group}"], width)
                  for group, width in enumerate(self.widths)]
        self.ctx = StepContext(
            num_tokens=bucket, num_seqs=seqs, num_wanted=seqs, max_new=1 if single else bucket, max_context=longest,
            tokens=views["tokens"], positions=views["positions"], token_seq=views["token_seq"], no_slots=views["no_slots"],
            seq_start=views["seq_start"], seq_first_pos=views["seq_first_pos"], seq_len=views["seq_len"],
            seq_slot=views["seq_slot"], token_slot=views["token_slot"], want_rows=views["want_rows"], groups=groups,
            host=self.host, wants_all_rows=single,
            compute_units=_compute_units(runner.device), tile_owner=None if single else self)
        self.graph = None
        self.logits = None
        self._rows_filled = bucket                           # rows that may hold a step's values
        self._known = [[(0, 0)] * bucket for _ in cache.groups]   # per group and row: (admission, blocks written)

    def forget(self) -> None:
        """What the rows of the block tables are known to hold is no longer trusted: the next step
        writes them whole."""
        self._known = [[(0, 0)] * self.bucket for _ in self._known]

    @property
    def runner(self) -> "ModelRunner":
        runner = self._runner()
        if runner is None:
            raise invalid_argument("the recording has outlived its runner")
        return runner

    def _fill(self, entries: Sequence[StepEntry]) -> int:
        """The step's arrays in the pinned buffer; returns the number of logits rows the step
        asks for.  A row's part of a block table is kept from
        step to step while the same admission of a request stays in the row: its page list only
        grows, so only the new entries are written.  (Entries of pages that a window has given
        back since keep the old page number: any page number is good there, the kernels mask
        those positions.)"""
        cache, host, count = self.runner.cache, self.host, len(entries)
        page_size, shift = cache.page_size, cache.page_size.bit_length() - 1
        held = [cache.held(entry.request) for entry in entries]
        positions = [info.length for info in held]
        stale = max(self._rows_filled, count)
        for name in ("tokens", "positions", "seq_first_pos"):
            host[name][count:stale] = 0
        host["seq_len"][count:stale] = 1
        host["seq_slot"][count:stale] = -1                   # padding rows belong to no request: no state row is theirs
        host["token_slot"][count:stale] = -1
        host["tokens"][:count] = [int(entry.tokens[0]) for entry in entries]
        host["token_source"][:count] = [-1 if entry.source is None else int(entry.source) for entry in entries]
        host["token_source"][count:stale] = -1
        host["positions"][:count] = positions
        host["seq_first_pos"][:count] = positions
        host["seq_len"][:count] = [position + 1 for position in positions]
        host["seq_slot"][:count] = [info.slot for info in held]
        host["token_slot"][:count] = host["seq_slot"][:count]
        for group in range(len(cache.groups)):
            table, slots, known = host[f"block_table{group}"], host[f"slot_map{group}"], self._known[group]
            table[count:stale] = 0
            slots[count:stale] = -1
            for row in range(count, stale):
                known[row] = (0, 0)
            rows = []
            for row, info in enumerate(held):
                pages = info.pages[group]
                serial, copied = known[row]
                if serial != info.serial or copied > len(pages):
                    table[row] = 0
                    copied = 0
                if copied < len(pages):
                    fresh = pages[copied:]
                    table[row, copied:len(pages)] = [page if page != ABSENT else 0 for page in fresh] if ABSENT in fresh else fresh
                    known[row] = (info.serial, len(pages))
                page = pages[positions[row] >> shift]
                if page == ABSENT:
                    raise out_of_bounds(f"position {positions[row]} of request {entries[row].request!r} has no page")
                rows.append(page * page_size + (positions[row] & (page_size - 1)))
            slots[:count] = rows
        self._rows_filled = count
        return count

    def run(self, entries: Sequence[StepEntry], transferred=None) -> torch.Tensor:
        """`transferred`: an event to record once the step's arrays are on their way."""
        runner = self.runner
        if self.copy_pending:
            # the pinned buffer is written again only after its last transfer has read it (a caller
            # may run steps without ever waiting for one)
            self.copied.synchronize()
        wanted = self._fill(entries)
        self.device_flat.copy_(self.pinned, non_blocking=True)
        self._send_lists()
        self.copied.record()
        self.copy_pending = True
        if any(entry.source is not None for entry in entries):
            ops_feed_tokens(self.ctx.tokens, self.token_source, runner.device_tokens, runner.vocab_size)
        if transferred is not None:
            transferred.record()
        if self.graph is None:
            # the first step of this size runs eagerly (its result is used, and it leaves the
            # context's work lists made); the same launches are then recorded for the steps to come
            logits = runner.model.forward(self.ctx, runner.cache.bindings)
            if not runner.capture:
                return logits[:wanted]
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            # no garbage collection while the capture is open: collecting some dead object that
            # holds device resources (another engine's recording, say) would call into the device
            # in ways a capture forbids.  (Switched off, not run beforehand: a collection takes
            # 20 ms of the 27 that making a recording took with it.)
            collecting = gc.isenabled()
            gc.disable()
            try:
                with torch.cuda.graph(graph):
                    self.logits = runner.model.forward(self.ctx, runner.cache.bindings)
            finally:
                if collecting:
                    gc.enable()
            self.graph = graph
            return logits[:wanted]
        self.graph.replay()
        return self.logits[:wanted]

    def _send_lists(self) -> None:
        """Work lists that depend on how the step is cut (a decode step has none)."""


class PortionGraph(DecodeGraph):
    """A recorded step of up to `tokens` tokens in up to `seqs` sequences, cut anywhere: portions
    of prompts beside single tokens, with at most `seqs` wanted rows.  Tokens beyond the step's
    are padding (token 0 at position 0 of the step's first sequence, written nowhere: slot -1, in
    no attention tile), sequences beyond the step's have no tokens, wanted rows beyond the step's
    name row 0; their results are dropped.  The attention kernel's work list has a fixed size
    too: the tiles of the step, then empty ones."""
    MAX_TOKENS = 512        # beyond, a step's kernels take longer than the host needs to launch them
    MAX_SEQS = 64

    def __init__(self, runner: "ModelRunner", tokens: int, seqs: int, longest: int):
        super().__init__(runner, tokens, longest, seqs=seqs)
        self._lists: dict = {}            # a part's key -> (pinned list, the list on the device, the function that makes it)

    def tiles_for(self, key, make, capacity: int) -> torch.Tensor:
        """A part's work list `key` of this recording, at its fixed place.  `make(host)` builds it
        from the step's host arrays as int32 [n, 4] (it is called now, and again before every
        replay); `capacity`: the most rows it can have in a step of this recording's size.  Rows
        beyond the step's are zero."""
        if key not in self._lists:
            if torch.cuda.is_current_stream_capturing():
                raise invalid_argument("a work list first asked for inside a recording")
            self._lists[key] = (torch.zeros((capacity, 4), dtype=torch.int32, pin_memory=True),
                                torch.zeros((capacity, 4), dtype=torch.int32, device=self.device_flat.device), make)
        pinned, device, make = self._lists[key]
        made = make(self.host)
        if made.shape[0] > pinned.shape[0]:
            raise invalid_argument(f"{made.shape[0]} rows of a work list do not fit the recording's {pinned.shape[0]}")
        host = pinned.numpy()
        host[:made.shape[0]] = made
        host[made.shape[0]:] = 0                                  # (an attention tile without tokens: the kernel leaves at once)
        device.copy_(pinned, non_blocking=True)
        return device

    def _send_lists(self) -> None:
        for key, (_, _, make) in self._lists.items():
            self.tiles_for(key, make, 0)

    def _fill(self, entries: Sequence[StepEntry]) -> int:
        cache, host = self.runner.cache, self.host
        counts = [len(entry.tokens) for entry in entries]
        total, seqs = sum(counts), len(entries)
        first = [cache.length(entry.request) for entry in entries]
        host["tokens"][:total] = np.concatenate([np.asarray(entry.tokens, dtype=np.int32) for entry in entries])
        host["tokens"][total:] = 0
        host["positions"][:total] = np.concatenate([np.arange(start, start + n, dtype=np.int32) for start, n in zip(first, counts)])
        host["positions"][total:] = 0
        host["token_seq"][:total] = np.repeat(np.arange(seqs, dtype=np.int32), counts)
        host["token_seq"][total:] = 0
        host["seq_start"][0] = 0
        host["seq_start"][1:seqs + 1] = np.cumsum(counts)
        host["seq_start"][seqs + 1:] = total
        host["seq_first_pos"][:seqs] = first
        host["seq_first_pos"][seqs:] = 0
        host["seq_len"][:seqs] = [start + n for start, n in zip(first, counts)]
        host["seq_len"][seqs:] = 1
        host["seq_slot"][:seqs] = [cache.slot(entry.request) for entry in entries]
        host["seq_slot"][seqs:] = -1                           # padding sequences belong to no request
        host["token_slot"][:total] = np.repeat(host["seq_slot"][:seqs], counts)
        host["token_slot"][total:] = -1
        want = [int(host["seq_start"][index]) + int(place) for index, entry in enumerate(entries) for place in entry.want]
        host["want_rows"][:len(want)] = want
        host["want_rows"][len(want):] = 0
        for group in range(len(cache.groups)):
            table, slots = host[f"block_table{group}"], host[f"slot_map{group}"]
            table[:] = 0
            for row, entry in enumerate(entries):
                pages = cache.page_list(entry.request, group)
                table[row, :len(pages)] = [page if page != ABSENT else 0 for page in pages]
            slots[:total] = np.concatenate([np.asarray(cache.rows(entry.request, group, start, n), dtype=np.int32)
                                            for entry, start, n in zip(entries, first, counts)])
            slots[total:] = -1
        return len(want)


def _compute_units(device) -> int:
    device = torch.device(device)
    if device.type != "cuda":
        return 256
    return int(torch.cuda.get_device_properties(device).multi_processor_count)


def build_context(cache: CacheManager, entries: Sequence[StepEntry], device) -> StepContext:
    """The step's arrays for entries whose pages are reserved: built on the host, sent in one
    transfer."""
    counts = [len(entry.tokens) for entry in entries]
    total, seqs = sum(counts), len(entries)
    first = [cache.length(entry.request) for entry in entries]
    tokens = np.concatenate([np.asarray(entry.tokens, dtype=np.int32) for entry in entries])
    positions = np.concatenate([np.arange(start, start + n, dtype=np.int32) for start, n in zip(first, counts)])
    token_seq = np.repeat(np.arange(seqs, dtype=np.int32), counts)
    seq_start = np.zeros(seqs + 1, dtype=np.int32)
    seq_start[1:] = np.cumsum(counts)
    want_rows = np.asarray([seq_start[index] + int(place) for index, entry in enumerate(entries) for place in entry.want],
                           dtype=np.int32)
    host = {
        "tokens": tokens, "positions": positions, "token_seq": token_seq,
        "no_slots": np.full(total, -1, dtype=np.int32), "seq_start": seq_start,
        "seq_first_pos": np.asarray(first, dtype=np.int32),
        "seq_len": np.asarray([start + n for start, n in zip(first, counts)], dtype=np.int32),
        "seq_slot": np.asarray([cache.slot(entry.request) for entry in entries], dtype=np.int32),
        "want_rows": want_rows,
    }
    host["token_slot"] = np.repeat(host["seq_slot"], counts)
    group_shapes = []
    for group in range(len(cache.groups)):
        lists = [cache.page_list(entry.request, group) for entry in entries]
        width = max(1, max(len(pages) for pages in lists))
        table = np.zeros((seqs, width), dtype=np.int32)
        for row, pages in enumerate(lists):
            table[row, :len(pages)] = [page if page != ABSENT else 0 for page in pages]
        slot_map = np.concatenate([np.asarray(cache.rows(entry.request, group, start, n), dtype=np.int32)
                                   for entry, start, n in zip(entries, first, counts)])
        host[f"block_table{group}"] = table
        host[f"slot_map{group}"] = slot_map
        group_shapes.append(width)
    # one transfer for all of it
    names = list(host)
    flat = np.concatenate([host[name].ravel() for name in names])
    device_flat = torch.from_numpy(flat).to(device, non_blocking=False)
    views, cursor = {}, 0
    for name in names:
        size = host[name].size
        views[name] = device_flat[cursor:cursor + size].view(host[name].shape)
        cursor += size
    groups = [GroupView(views[f"block_table{group}"], views[f"slot_map{group}"], width)
              for group, width in enumerate(group_shapes)]
    return StepContext(
        num_tokens=total, num_seqs=seqs, num_wanted=int(want_rows.size), max_new=max(counts),
        max_context=int(host["seq_len"].max()), tokens=views["tokens"], positions=views["positions"],
        token_seq=views["token_seq"], no_slots=views["no_slots"], seq_start=views["seq_start"],
        seq_first_pos=views["seq_first_pos"], seq_len=views["seq_len"], seq_slot=views["seq_slot"],
        token_slot=views["token_slot"], want_rows=views["want_rows"], groups=groups, host=host,
        wants_all_rows=bool(want_rows.size == total and np.array_equal(want_rows, np.arange(total))),
        compute_units=_compute_units(device))

