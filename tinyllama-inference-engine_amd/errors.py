"""Structured errors: one code and one message, as the reference reports them.

The twelve codes and their snake_case names follow include/tlie/error.hpp:7-20 and
src/error.cpp:5-33 of the reference; its `cuda_error` is `hip_error` here.  The command line
prints an error as one JSON line, `{"error": {"code": ..., "message": ...}}`
(app/reference_cli.cpp:20-25).
"""
from __future__ import annotations

import enum
import json


class ErrorCode(enum.Enum):
    IO = "io_error"
    INVALID_FORMAT = "invalid_format"
    CHECKSUM_MISMATCH = "checksum_mismatch"
    INVALID_CONFIG = "invalid_config"
    INVALID_SHAPE = "invalid_shape"
    INVALID_DTYPE = "invalid_dtype"
    OUT_OF_MEMORY = "out_of_memory"
    OUT_OF_BOUNDS = "out_of_bounds"
    TOKENIZER = "tokenizer_error"
    NUMERICAL = "numerical_error"
    INVALID_ARGUMENT = "invalid_argument"
    HIP = "hip_error"


class EngineError(Exception):
    """An error with a code from `ErrorCode`; everything the engine raises on purpose is one."""

    def __init__(self, code: ErrorCode, message: str):
        super().__init__(f"{code.value}: {message}")
        self.code = code
        self.message = message

    def to_json(self) -> str:
        return json.dumps({"error": {"code": self.code.value, "message": self.message}})


def invalid_config(message: str) -> EngineError:
    return EngineError(ErrorCode.INVALID_CONFIG, message)


def invalid_argument(message: str) -> EngineError:
    return EngineError(ErrorCode.INVALID_ARGUMENT, message)


def invalid_shape(message: str) -> EngineError:
    return EngineError(ErrorCode.INVALID_SHAPE, message)


def out_of_bounds(message: str) -> EngineError:
    return EngineError(ErrorCode.OUT_OF_BOUNDS, message)


def out_of_memory(message: str) -> EngineError:
    return EngineError(ErrorCode.OUT_OF_MEMORY, message)


class device_memory_errors:
    """`with device_memory_errors("the cache pools"):` turns the device allocator's refusal into
    `out_of_memory`, as the reference maps a failed device allocation of its weights and of its
    cache (src/cuda/weight_store.cpp:273-274, src/cuda/model.cu:262-270)."""

    def __init__(self, what: str):
        self.what = what

    def __enter__(self):
        return self

    def __exit__(self, kind, error, traceback):
        import torch
        if kind is not None and issubclass(kind, torch.cuda.OutOfMemoryError):
            raise EngineError(ErrorCode.OUT_OF_MEMORY, f"the device has no memory for {self.what}: {error}") from None
        return False
