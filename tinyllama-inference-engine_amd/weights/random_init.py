"""Random weights: writes a model folder (config.json, model.safetensors) from a configuration
and a seed.  The reference has no such mode (every model-level test of it needs the real
checkpoint); the list of tensors comes from the parts the model is built of, so a model with
other parts gets other tensors without a change here.

Each tensor is drawn from a generator seeded by (seed, tensor name): its values do not depend on
which other tensors exist or in which order they are drawn.
"""
from __future__ import annotations

import hashlib
import json
import os

import torch

from ..config.spec import TensorSpec
from .safetensors_io import write_safetensors


def _generator(seed: int, name: str, device="cpu") -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode("utf-8")).digest()
    generator = torch.Generator(device=device)
    generator.manual_seed(int.from_bytes(digest[:8], "little") & 0x7FFF_FFFF_FFFF_FFFF)
    return generator


def random_tensors(specs: list[TensorSpec], seed: int, std: float = 0.02, norm_std: float = 0.01,
                   dtype: torch.dtype = torch.bfloat16, device="cpu") -> dict[str, torch.Tensor]:
    """Drawn on `device`; the values of a (seed, name) are the same on every run on one kind of
    device, but differ between the CPU's and the GPU's generators."""
    return {spec.name: _draw(spec, seed, std, norm_std, dtype, device) for spec in specs if not spec.optional}


def _draw(spec: TensorSpec, seed: int, std: float, norm_std: float, dtype: torch.dtype, device) -> torch.Tensor:
    generator = _generator(seed, spec.name, device)
    values = torch.randn(spec.shape, generator=generator, dtype=torch.float32, device=device)
    if spec.init == "normal":
        values = values * std
    elif spec.init == "norm":
        values = 1.0 + values * norm_std
    elif spec.init == "zeros":
        values = torch.zeros(spec.shape, device=device)
    else:
        raise ValueError(f"unknown init '{spec.init}' for {spec.name}")
    return values.to(dtype)


def resident_random_tensors(specs: list[TensorSpec], seed: int, std: float = 0.02, norm_std: float = 0.01,
                            dtype: torch.dtype = torch.bfloat16, device="cpu"):
    """The tensors of `random_tensors`, each drawn when a part asks for it, as a `ResidentWeights`
    (one device allocation for what the parts keep)."""
    from .arena import ResidentWeights
    wanted = [spec for spec in specs if not spec.optional]

    def draw(spec):
        return lambda: _draw(spec, seed, std, norm_std, dtype, device)
    sizes = {}
    for spec in wanted:
        count = 1
        for extent in spec.shape:
            count *= int(extent)
        sizes[spec.name] = count * dtype.itemsize
    return ResidentWeights({spec.name: draw(spec) for spec in wanted}, sizes, device)


def write_random_model(model_dir: str, config, seed: int, std: float = 0.02, norm_std: float = 0.01,
                       dtype: torch.dtype = torch.bfloat16) -> None:
    """`config` is a configuration object of a registered architecture (it has `to_dict` and
    `to_spec`).  The folder is created if needed."""
    from ..models.builder import expected_tensors
    os.makedirs(model_dir, exist_ok=True)
    specs = expected_tensors(config.to_spec())
    raw = config.to_dict()
    raw["torch_dtype"] = {torch.bfloat16: "bfloat16", torch.float32: "float32", torch.float16: "float16"}[dtype]
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as handle:
        json.dump(raw, handle, indent=2, sort_keys=True)
    write_safetensors(os.path.join(model_dir, "model.safetensors"),
                      random_tensors(specs, seed, std, norm_std, dtype),
                      metadata={"format": "pt", "seed": str(seed)})
