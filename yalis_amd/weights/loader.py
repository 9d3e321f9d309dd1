"""Loading a model's tensors by name.

The parts of a model declare what they need (``TensorSpec`` by checkpoint name);
``open_tensors`` reads exactly those from the folder and fails with ONE error that
lists every missing tensor, every unexpected tensor and every wrong shape (the
reference gets the same from ``load_state_dict(strict=True)``,
yalis/model_loading.py:201-249).

Precision rule: a floating tensor stored in 16 bits is kept in bfloat16, integer tables
become int32, and in the 32-bit mode of the engine every floating tensor is widened to float32
(exact).  A tensor stored in 32 bits inside a 16-bit checkpoint stays in 32 bits in the bfloat16
engine (such tensors are stored wide because they need it).  A checkpoint stored WHOLLY in 32
bits is a 32-bit copy of the model, not a statement about single tensors: the bfloat16 engine
narrows it to bfloat16, as the reference casts every tensor to its parameter's dtype
(yalis/model_loading.py:172-173).  ``wide_tensors`` overrides the rule: "keep" leaves every
32-bit tensor wide (a float32 matrix in the bfloat16 engine then runs on the float32 kernels,
which is said once, loudly), "cast" narrows all of them.  Tensors stored in float16 are rounded
to bfloat16 by the bfloat16 engine (to nearest even; every float16 value lies within bfloat16's
range), again as the reference casts to the parameter's dtype, and a warning says that three
bits of each such weight's fraction are dropped; the float32 engine widens them exactly.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, Mapping, Optional, Tuple

import torch

from ..utils.logger import get_logger
from .safetensors_io import TensorEntry, index_folder, read_tensor

logger = get_logger("weights")


@dataclass(frozen=True)
class TensorSpec:
    """What a part needs under one checkpoint name.

    kind: "float" or "int".
    init: how the random-weights mode fills it: ("normal", std) or
        ("one_plus_normal", std) or ("zeros",) or ("randint", high).
    """

    shape: Tuple[int, ...]
    kind: str = "float"
    init: Tuple = ("normal", 0.02)


class WeightsError(RuntimeError):
    """The checkpoint does not hold what the model needs."""

    def __init__(self, where: str, missing, unexpected, wrong_shape, wrong_kind=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_kind = list(wrong_kind)
        lines = [f"checkpoint in {where!r} does not match the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, got, want in self.wrong_shape:
            lines.append(f"  wrong shape: {name} has {tuple(got)}, the model needs {tuple(want)}")
        for name, got, want in self.wrong_kind:
            lines.append(f"  wrong type: {name} is stored as {got}, the model needs {want}")
        super().__init__("\n".join(lines))


_FLOAT_TAGS = {"F64", "F32", "F16", "BF16"}
_INT_TAGS = {"I64", "I32", "I16", "I8", "U8"}

# Names a checkpoint may hold that no part asks for and that carry no weights
# (the reference's converter drops them too, yalis/external/convert_hf_checkpoint.py:705-736).
IGNORED_SUFFIXES = ("rotary_emb.inv_freq",)


def target_dtype(storage_tag: str, kind: str, engine_dtype: str, keep_wide: bool = True) -> torch.dtype:
    """``keep_wide``: whether a tensor stored in 32 bits stays so in the bfloat16 engine."""
    if kind == "int":
        return torch.int32
    if engine_dtype == "float32":
        return torch.float32
    if storage_tag in ("F32", "F64") and keep_wide:
        return torch.float32
    return torch.bfloat16


def keeps_wide(entries: Dict[str, TensorEntry], wanted: Dict[str, "TensorSpec"], wide_tensors: str) -> bool:
    """The precision rule's decision for a checkpoint: True when tensors stored in 32 bits
    stay in 32 bits in the bfloat16 engine."""
    if wide_tensors not in ("auto", "keep", "cast"):
        raise ValueError(f"wide_tensors must be 'auto', 'keep' or 'cast', got {wide_tensors!r}")
    if wide_tensors != "auto":
        return wide_tensors == "keep"
    tags = {entries[n].dtype for n, sp in wanted.items() if sp.kind == "float" and n in entries}
    return not tags <= {"F32", "F64"}  # a checkpoint wholly in 32 bits is narrowed


def check_against(entries: Dict[str, TensorEntry], wanted: Dict[str, TensorSpec], where: str, engine_dtype: Optional[str] = None) -> None:
    missing = [n for n in wanted if n not in entries]
    unexpected = [
        n for n in entries if n not in wanted and not n.endswith(IGNORED_SUFFIXES)
    ]
    wrong_shape = [
        (n, entries[n].shape, s.shape)
        for n, s in wanted.items()
        if n in entries and tuple(entries[n].shape) != tuple(s.shape)
    ]
    wrong_kind = []
    for n, s in wanted.items():
        if n in entries:
            tag = entries[n].dtype
            ok = tag in (_FLOAT_TAGS if s.kind == "float" else _INT_TAGS)
            if not ok:
                wrong_kind.append((n, tag, s.kind))
    if missing or unexpected or wrong_shape or wrong_kind:
        raise WeightsError(where, sorted(missing), sorted(unexpected), wrong_shape, wrong_kind)


class TensorSource(Mapping):
    """Tensors made when a part asks for them, so that a large model never holds both the
    checkpoint's tensors and what the parts fuse from them.  ``uses`` says how many parts
    ask for each name: a tensor that several parts take (a tied table) is made once and
    kept until the last of them has had it."""

    def __init__(self, uses: Dict[str, int], make: Callable[[str], torch.Tensor]):
        self._left = dict(uses)
        self._make = make
        self._kept: Dict[str, torch.Tensor] = {}

    def __getitem__(self, name: str) -> torch.Tensor:
        if name not in self._left:
            raise KeyError(name)
        t = self._kept.pop(name, None)
        if t is None:
            t = self._make(name)
        self._left[name] -= 1
        if self._left[name] > 0:
            self._kept[name] = t
        return t

    def __iter__(self):
        return iter(self._left)

    def __len__(self) -> int:
        return len(self._left)


def open_tensors(
    model_dir: str,
    wanted: Dict[str, TensorSpec],
    uses: Dict[str, int],
    engine_dtype: str,
    device: str,
    progress: Optional[Callable[[str], None]] = None,
    wide_tensors: str = "auto",
) -> TensorSource:
    """Check the folder against ``wanted`` (the one error lists everything that is wrong)
    and return a source that reads each tensor onto ``device`` when it is asked for."""
    entries = index_folder(model_dir)
    check_against(entries, wanted, model_dir, engine_dtype)
    keep_wide = keeps_wide(entries, wanted, wide_tensors)
    if engine_dtype == "bfloat16":
        halves = [n for n, sp in wanted.items() if sp.kind == "float" and entries[n].dtype == "F16"]
        if halves:
            logger.warning("%d tensors of %s are stored in float16: the bfloat16 engine rounds them to bfloat16 (three bits of "
                           "each weight's fraction are dropped; precision fp32 keeps them exactly); first: %s",
                           len(halves), model_dir, halves[0])
        wide = [n for n, sp in wanted.items() if sp.kind == "float" and entries[n].dtype in ("F32", "F64")]
        matrices = [n for n in wide if len(wanted[n].shape) >= 2]
        if wide and not keep_wide:
            logger.info("%s: %d tensors stored in 32 bits are narrowed to bfloat16 for the bfloat16 engine "
                        "(wide_tensors='keep' leaves them wide)", model_dir, len(wide))
        elif matrices:
            logger.warning(
                "%d matrices of %s are stored in 32 bits and stay so: the bfloat16 engine runs their products on its "
                "float32 kernels (twice the memory, far slower than the matrix cores); first: %s", len(matrices), model_dir, matrices[0])
    done = [0]

    def make(name: str) -> torch.Tensor:
        e = entries[name]
        dt = target_dtype(e.dtype, wanted[name].kind, engine_dtype, keep_wide)
        t = read_tensor(e).to(device=device, dtype=dt).contiguous()
        done[0] += 1
        if progress is not None and done[0] % 32 == 1:
            progress(f"loaded {done[0]}/{len(wanted)} tensors")
        return t

    return TensorSource(uses, make)
