"""The random-weights mode: fill the tensors a model asks for from a seed, in memory
or as a model folder (config.json + model.safetensors) that the loader reads back.

Matrices are N(0, 0.02) as the reference initialises them
(yalis/external/model.py:113-120); norm weights are 1 + N(0, 0.1) rather than the
reference's ones (:974) so that the norm's multiply shows in tests.  Each tensor has
a generator of its own, seeded from (seed, tensor name), so that values do not depend
on the order in which tensors are made.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Iterator, Tuple

import torch

from .loader import TensorSpec
from .safetensors_io import write_file


def _tensor_seed(seed: int, name: str) -> int:
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & 0x7FFFFFFFFFFFFFFF


def random_tensor(name: str, spec: TensorSpec, seed: int, dtype: torch.dtype, device: str = "cpu") -> torch.Tensor:
    """One tensor of the random model.  On the CPU the values are the documented ones;
    on a GPU the same distribution from the device's generator."""
    g = torch.Generator(device=device).manual_seed(_tensor_seed(seed, name))
    kind = spec.init[0]
    if spec.kind == "int":
        high = spec.init[1] if kind == "randint" else 2
        return torch.randint(0, high, spec.shape, generator=g, device=device, dtype=torch.int32)
    if kind == "normal":
        t = torch.randn(spec.shape, generator=g, device=device, dtype=torch.float32) * spec.init[1]
    elif kind == "one_plus_normal":
        t = 1.0 + torch.randn(spec.shape, generator=g, device=device, dtype=torch.float32) * spec.init[1]
    elif kind == "zeros":
        t = torch.zeros(spec.shape, device=device, dtype=torch.float32)
    else:
        raise ValueError(f"tensor {name!r}: unknown init {spec.init!r}")
    return t.to(dtype)


def random_tensors(specs: Dict[str, TensorSpec], seed: int, dtype: torch.dtype, device: str = "cpu") -> Iterator[Tuple[str, torch.Tensor]]:
    for name, spec in specs.items():
        yield name, random_tensor(name, spec, seed, dtype, device)


def write_random_model(folder: str, config_dict: dict, seed: int, dtype: str = "bfloat16") -> str:
    """Write ``folder/config.json`` and ``folder/model.safetensors`` for the
    architecture that ``config_dict`` names; returns the folder."""
    from ..engine.factory import tensor_specs_for  # late: the factory imports the parts

    tdtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
    specs = tensor_specs_for(config_dict)
    os.makedirs(folder, exist_ok=True)
    cfg = dict(config_dict)
    cfg["torch_dtype"] = dtype
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f, indent=1)
    shapes = {
        name: (torch.int32 if s.kind == "int" else tdtype, tuple(s.shape)) for name, s in specs.items()
    }
    write_file(os.path.join(folder, "model.safetensors"), random_tensors(specs, seed, tdtype), shapes)
    return folder
