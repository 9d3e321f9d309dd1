"""From a model folder (or a configuration and a seed) to a model ready to step.

The order is the reference's (yalis/model.py:11-59: configuration, construction
without initialisation, weights, eval): read config.json, pick the architecture from
the registry, describe it as parts, build the parts, load their tensors by name.
"""
from __future__ import annotations

from typing import Dict

import torch

from ..config.reader import read_config_json
from ..config.registry import architecture_of
from ..config.runtime import EngineConfig
from ..models.decoder import DecoderModel
from ..parts.base import Runtime
from ..weights.loader import TensorSource, TensorSpec, open_tensors
from ..weights.random_init import random_tensor
from .step import ModelRunner


class _ShapeOnlyOps:
    """Stands in for the kernel library where parts are built only to ask them which
    tensors they need: no kernel is ever called, and whatever a part's constructor asks the
    library (a tile size, whether a fused path exists, a packed layout's group) is answered
    with 1, a value that is a valid size and a true flag.  A new part needs no entry here."""

    def __getattr__(self, name):
        if name.startswith("__"):
            raise AttributeError(name)
        return lambda *a, **k: 1


def spec_from_config(config_dict: dict):
    arch = architecture_of(config_dict)
    cfg = arch.config_class.from_dict(config_dict)
    return arch, cfg, arch.build_spec(cfg)


def tensor_specs_for(config_dict: dict) -> Dict[str, TensorSpec]:
    """Name -> shape of every tensor the architecture's checkpoint holds."""
    _, _, spec = spec_from_config(config_dict)
    rt = Runtime(device="cpu", engine_dtype="float32", ops=_ShapeOnlyOps(), max_positions=1)
    return DecoderModel(spec, rt).tensor_specs()


def default_ops(device: str):
    from ..ops.hip import HipOps

    return HipOps(device)


def build_model(
    config_dict: dict,
    engine: EngineConfig,
    ops=None,
) -> DecoderModel:
    arch, cfg, spec = spec_from_config(config_dict)
    if engine.max_model_len > spec.max_positions:
        raise ValueError(
            f"max_model_len={engine.max_model_len} exceeds the model's max_position_embeddings={spec.max_positions}"
        )
    if ops is None:
        ops = default_ops(engine.device)
        ops.tune_library_products(engine.tune_library_products)
    rt = Runtime(
        device=engine.device,
        engine_dtype=engine.dtype,
        ops=ops,
        max_positions=engine.max_model_len,
        page_size=engine.page_size,
    )
    return DecoderModel(spec, rt)


def load_runner(model_dir: str, engine: EngineConfig, ops=None, progress=None) -> ModelRunner:
    """A runner over the checkpoint in ``model_dir``."""
    model = build_model(read_config_json(model_dir), engine, ops)
    model.load(open_tensors(model_dir, model.tensor_specs(), model.tensor_uses(), engine.dtype, engine.device, progress,
                            wide_tensors=engine.wide_tensors))
    return ModelRunner(model, engine)


def random_runner(config_dict: dict, engine: EngineConfig, seed: int, ops=None, on_device: bool = True) -> ModelRunner:
    """A runner over random weights made in memory (no folder): on the device itself
    when ``on_device`` (large models), else on the CPU with the documented values."""
    model = build_model(config_dict, engine, ops)
    wdtype = torch.float32 if engine.dtype == "float32" else torch.bfloat16
    gen_device = engine.device if on_device else "cpu"
    specs = model.tensor_specs()
    model.load(TensorSource(
        model.tensor_uses(),
        lambda name: random_tensor(name, specs[name], seed, wdtype, gen_device).to(engine.device),
    ))
    return ModelRunner(model, engine)
