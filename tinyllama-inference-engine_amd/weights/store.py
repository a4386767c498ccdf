"""Weights by tensor name, checked against what the model's parts expect.

The reference's store answers `Get(name)` and `Validate(specs)`: every expected name present,
with the expected shape, and no tensor beyond the expected ones (src/weight_store.cpp:264-295).
It reports the first fault; here one error lists all of them: missing tensors, unexpected ones
and wrong shapes.  Its code is `invalid_shape`, as the reference's is for each of the three.

Kept precision: a tensor stored in 16-bit floating point is kept in bfloat16, a tensor stored in
32-bit stays in 32-bit, integer tables become int32.  In the 32-bit mode every floating tensor is
widened to float32.
"""
from __future__ import annotations

import json
import os
import re
from typing import Iterable

import torch

from ..config.spec import TensorSpec
from ..errors import EngineError, ErrorCode
from .safetensors_io import SafetensorsFile


class WeightStore:
    """All safetensors files of a model folder behind one `get(name)`."""

    def __init__(self, model_dir: str, max_file_bytes: int | None = None):
        """max_file_bytes: a budget for the weight files together; a folder beyond it is refused
        with `out_of_memory` before any file is mapped (src/weight_store.cpp:134-138)."""
        self.model_dir = model_dir
        self._files: list[SafetensorsFile] = []
        self._where: dict[str, SafetensorsFile] = {}
        index_path = os.path.join(model_dir, "model.safetensors.index.json")
        single = os.path.join(model_dir, "model.safetensors")
        if os.path.isfile(index_path):
            try:
                with open(index_path, "r", encoding="utf-8") as handle:
                    weight_map = json.load(handle)["weight_map"]
                names = sorted(set(weight_map.values()))
            except (OSError, ValueError, KeyError, AttributeError) as error:
                raise EngineError(ErrorCode.INVALID_FORMAT, f"{index_path}: not a shard index ({error})") from None
        elif os.path.isfile(single):
            names = ["model.safetensors"]
        else:
            raise EngineError(ErrorCode.IO, f"unable to open weights: {single} does not exist")
        if max_file_bytes is not None:
            try:
                total = sum(os.path.getsize(os.path.join(model_dir, name)) for name in names)
            except OSError as error:
                raise EngineError(ErrorCode.IO, f"unable to stat the weight files of {model_dir} ({error.strerror})") from None
            if total > max_file_bytes:
                raise EngineError(ErrorCode.OUT_OF_MEMORY, f"the weight files hold {total} bytes, which exceeds the configured "
                                                           f"budget of {max_file_bytes} before mapping")
        for name in names:
            file = SafetensorsFile(os.path.join(model_dir, name))
            self._files.append(file)
            for tensor_name in file.tensors:
                if tensor_name in self._where:
                    raise EngineError(ErrorCode.INVALID_FORMAT, f"tensor '{tensor_name}' is stored in two files")
                self._where[tensor_name] = file

    def sha256(self) -> str:
        """The SHA-256 of the weight files' bytes, in the order of their names (one file: that
        file's digest, as `sha256sum model.safetensors` prints it)."""
        import hashlib
        digest = hashlib.sha256()
        for file in self._files:
            with open(file.path, "rb") as handle:
                for block in iter(lambda: handle.read(1 << 24), b""):
                    digest.update(block)
        return digest.hexdigest()

    def expect_sha256(self, expected: str) -> None:
        """reference: the weights' digest is a pinned trust root there, checked at load
        (include/tlie/pinned_model.hpp:7-14, src/weight_store.cpp:162-165: `checksum_mismatch`);
        here the caller may name one."""
        found = self.sha256()
        if found != expected.strip().lower():
            raise EngineError(ErrorCode.CHECKSUM_MISMATCH, f"the weights' SHA-256 is {found}, expected {expected.strip().lower()}")

    def names(self) -> list[str]:
        return sorted(self._where)

    def __contains__(self, name: str) -> bool:
        return name in self._where

    def shape(self, name: str) -> tuple[int, ...]:
        return self._where[name].tensors[name].shape

    def get(self, name: str) -> torch.Tensor:
        if name not in self._where:
            raise EngineError(ErrorCode.INVALID_SHAPE, f"required tensor is missing: {name}")
        return self._where[name].tensor(name)

    def validate(self, specs: Iterable[TensorSpec], ignored: Iterable[str] = ()) -> None:
        """ignored: patterns (regular expressions, matched against the whole name) of tensors
        that the architecture's files may carry although no part reads them (the model's
        specification names them: `ModelSpec.ignored_tensors`)."""
        specs = list(specs)
        patterns = [re.compile(pattern) for pattern in ignored]
        expected = {spec.name: spec for spec in specs}
        missing = [spec.name for spec in specs if not spec.optional and spec.name not in self._where]
        unexpected = [name for name in self.names()
                      if name not in expected and not any(pattern.fullmatch(name) for pattern in patterns)]
        wrong = []
        for spec in specs:
            if spec.name in self._where and tuple(self.shape(spec.name)) != tuple(spec.shape):
                wrong.append(f"{spec.name}: stored {list(self.shape(spec.name))}, expected {list(spec.shape)}")
        if missing or unexpected or wrong:
            parts = []
            if missing:
                parts.append(f"{len(missing)} missing: " + ", ".join(missing))
            if unexpected:
                parts.append(f"{len(unexpected)} unexpected: " + ", ".join(unexpected))
            if wrong:
                parts.append(f"{len(wrong)} with a wrong shape: " + "; ".join(wrong))
            raise EngineError(ErrorCode.INVALID_SHAPE,
                              f"weights in {self.model_dir} do not fit the model — " + " | ".join(parts))

    def load(self, specs: Iterable[TensorSpec], dtype: torch.dtype, device,
             ignored: Iterable[str] = ()) -> dict[str, torch.Tensor]:
        """Validates, then uploads every required tensor, in its kept precision, each an allocation
        of its own (see `resident` for what the engine uses).  A tensor the
        model marks optional (a tied head's matrix that some files still carry) is checked when
        present and not uploaded: no part reads it.  A matrix stored in 32-bit stays 32-bit also in
        a bfloat16 run (its products then go to the true 32-bit kernel, at a fraction of the
        speed): that is said once, as a warning, because nothing else shows it."""
        names = self._checked(specs, dtype, ignored)
        return {name: to_kept_precision(self.get(name), dtype).to(device) for name in names}

    def resident(self, specs: Iterable[TensorSpec], dtype: torch.dtype, device, ignored: Iterable[str] = ()):
        """Validates like `load`, uploads nothing yet: a `ResidentWeights` that uploads a tensor when a
        part asks for it, with one device allocation for everything that the parts keep."""
        from .arena import ResidentWeights
        names = self._checked(specs, dtype, ignored)

        def upload(name):
            return lambda: to_kept_precision(self.get(name), dtype).to(device)
        sizes = {}
        for name in names:
            entry = self._where[name].tensors[name]
            count = 1
            for extent in entry.shape:
                count *= int(extent)
            sizes[name] = count * kept_dtype(entry.dtype, dtype).itemsize
        return ResidentWeights({name: upload(name) for name in names}, sizes, device)

    def _checked(self, specs: Iterable[TensorSpec], dtype: torch.dtype, ignored: Iterable[str]) -> list[str]:
        """The names to upload, after validation and the warning about matrices stored in 32-bit."""
        specs = list(specs)
        self.validate(specs, ignored)
        names = [spec.name for spec in specs if spec.name in self._where and not spec.optional]
        wide = [name for name in names if dtype == torch.bfloat16 and len(self.shape(name)) >= 2
                and kept_dtype(self._where[name].tensors[name].dtype, dtype) == torch.float32]
        if wide:
            import warnings
            warnings.warn(f"{len(wide)} matrices of {self.model_dir} are stored in 32-bit and are kept so in this bfloat16 run "
                          f"(first: {wide[0]}); their products take the 32-bit kernel, which is many times slower",
                          stacklevel=3)
        return names


def kept_dtype(stored: torch.dtype, dtype: torch.dtype) -> torch.dtype:
    """The type a tensor stored as `stored` is kept in when the model runs in `dtype`."""
    if stored in (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8, torch.bool):
        return torch.int32
    if dtype == torch.float32:
        return torch.float32
    if dtype == torch.bfloat16:
        return torch.float32 if stored in (torch.float32, torch.float64) else torch.bfloat16
    raise EngineError(ErrorCode.INVALID_DTYPE, f"the engine runs in bfloat16 or float32, not {dtype}")


def to_kept_precision(tensor: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """The stored tensor in the precision it is kept in when the model runs in `dtype`."""
    return tensor.to(kept_dtype(tensor.dtype, dtype))
