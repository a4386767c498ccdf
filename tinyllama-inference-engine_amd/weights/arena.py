"""Where a model's weights live on the device: one allocation, cut into places of 256-byte alignment,
filled while the model's parts load, one part after the other.

The reference allocates and copies tensor by tensor (src/cuda/weight_store.cpp:270-283) and keeps
every tensor as it is stored.  Here the parts fuse at load time (q, k and v into one matrix, gate and up
interleaved), so what is kept is not what is stored; two things follow.  The stored tensors go to the
device only when a part asks for them, and are let go of when that part has loaded: never are all stored
tensors and all kept ones on the device together, and a model of 200 GB loads into 288.  And what a part
keeps for good it hands to `keep`, which copies it to its place in the one allocation and gives back the
view; the temporary that the part had made is then free again.

`ResidentWeights` is what a part's `load(weights, ...)` receives in the engine: a mapping from tensor
name to tensor, as a dict is (`weights[name]`, `weights.get(name)`, `name in weights`), with `keep` and
`release` beside.  A part that does not call `keep` works as well; its tensors then lie where torch put
them.  A plain dict of device tensors is still accepted everywhere a `ResidentWeights` is: `keep_in`
calls `keep` where there is one.
"""
from __future__ import annotations

from typing import Callable, Iterator, Mapping

import torch

from ..errors import EngineError, ErrorCode

ALIGNMENT = 256


def _aligned(nbytes: int) -> int:
    return (nbytes + ALIGNMENT - 1) // ALIGNMENT * ALIGNMENT


class WeightArena:
    """One allocation of `capacity` bytes on `device`; `place` hands out its parts front to back."""

    def __init__(self, capacity: int, device):
        self.capacity = _aligned(max(int(capacity), 0))
        self.buffer = torch.empty((self.capacity + ALIGNMENT,), dtype=torch.uint8, device=device)
        # torch's allocations are aligned to more than this already; the arena does not rely on it
        self._start = (-self.buffer.data_ptr()) % ALIGNMENT
        self.used = 0                     # bytes handed out, padding included
        self.outside = 0                  # bytes of tensors that did not fit and stayed where they were

    def holds(self, tensor: torch.Tensor) -> bool:
        """Whether `tensor`'s memory is this arena's."""
        return tensor.untyped_storage().data_ptr() == self.buffer.untyped_storage().data_ptr()

    def place(self, tensor: torch.Tensor) -> torch.Tensor:
        """A copy of `tensor` (contiguous, of its shape and type) at the next free place, 256 bytes
        aligned; `tensor` itself if it lies in the arena already, or if the arena is full (sized for
        what is stored, it can be, when a part keeps more than it read)."""
        if self.holds(tensor):
            return tensor
        nbytes = tensor.numel() * tensor.element_size()
        if self.used + _aligned(nbytes) > self.capacity:
            self.outside += nbytes
            return tensor
        offset = self._start + self.used
        view = self.buffer[offset:offset + nbytes].view(tensor.dtype).view(tensor.shape)
        view.copy_(tensor)
        self.used += _aligned(nbytes)
        return view


class ResidentWeights(Mapping):
    """Tensors by name, brought to the device when asked for; and the arena for what is kept.

    fetch[name]() makes the tensor (an upload, a random draw); sizes[name] is its size in bytes, known
    beforehand: the arena is made for their sum.  A name asked for twice before `release` gives the
    same tensor.  A tensor that was handed to `keep` as it came (not fused with others) is remembered by
    its name: who asks for that name later gets the kept one (a head tied to the embedding's table)."""

    def __init__(self, fetch: dict[str, Callable[[], torch.Tensor]], sizes: dict[str, int], device):
        self._fetch = dict(fetch)
        self._fresh: dict[str, torch.Tensor] = {}
        self._kept: dict[str, torch.Tensor] = {}
        self.arena = WeightArena(sum(_aligned(sizes[name]) for name in self._fetch), device)

    def __getitem__(self, name: str) -> torch.Tensor:
        if name in self._kept:
            return self._kept[name]
        if name not in self._fresh:
            if name not in self._fetch:
                raise EngineError(ErrorCode.INVALID_SHAPE, f"required tensor is missing: {name}")
            self._fresh[name] = self._fetch[name]()
        return self._fresh[name]

    def get(self, name: str, default=None):
        return self[name] if name in self._fetch else default

    def __iter__(self) -> Iterator[str]:
        return iter(self._fetch)

    def __len__(self) -> int:
        return len(self._fetch)

    def __contains__(self, name) -> bool:
        return name in self._fetch

    def keep(self, tensor: torch.Tensor) -> torch.Tensor:
        """The tensor at its place for good: a part calls this with every tensor it will read in
        steps, and uses what comes back."""
        source = tensor
        view = self.arena.place(tensor.contiguous())
        for name, fresh in self._fresh.items():
            if fresh is source:
                self._kept[name] = view
        return view

    def release(self) -> None:
        """Lets go of what was brought since the last call (the model calls this when a part has loaded)."""
        self._fresh.clear()


def keep_in(weights, tensor: torch.Tensor) -> torch.Tensor:
    """`weights.keep(tensor)` where the mapping has a place for kept tensors, `tensor` itself otherwise."""
    keep = getattr(weights, "keep", None)
    return keep(tensor) if keep is not None else tensor
