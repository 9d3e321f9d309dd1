"""Run-time configuration: which model, and how the engine is sized.

``ModelConfig`` and ``InferenceConfig`` keep the names and meanings of the
reference's classes (yalis/config.py:8-85 and :88-228).  Options of the reference
that select things this engine does not have (tensor-parallel dims, attention
backends, symmetric all-reduce) are accepted where that is harmless and refused
where honouring them is impossible.  ``EngineConfig`` holds what the paged engine
adds: page size, page count, the per-step token budget.
"""
from __future__ import annotations

import os
from dataclasses import dataclass, field
from typing import Optional, Tuple

_PRECISIONS = {
    "fp32": "float32",
    "float32": "float32",
    "bf16": "bfloat16",
    "bfloat16": "bfloat16",
}


def canonical_dtype(name: str) -> str:
    if name not in _PRECISIONS:
        raise ValueError(
            f"Invalid precision: {name}. Supported values are 'fp32' and 'bf16' "
            "(also spelled 'float32', 'bfloat16'); 'fp16' of the reference is not offered."
        )
    return _PRECISIONS[name]


class ModelConfig:
    """Which model and at which precision (yalis/config.py:13-37).

    ``model_path`` defaults to ``$YALIS_CACHE/checkpoints/<model_name>``
    (yalis/config.py:39-64) and must exist.  The folder holds config.json and
    model.safetensors (or shards with their index).
    """

    def __init__(
        self,
        model_name: Optional[str] = None,
        model_path: Optional[str] = None,
        precision: str = "bf16",
        disable_tp: bool = False,
    ):
        if model_name is None and model_path is None:
            raise ValueError("Either 'model_name' or 'model_path' must be provided.")
        self.model_name = model_name
        self.precision = precision
        self.dtype = canonical_dtype(precision)
        self.disable_tp = disable_tp
        if model_path is None:
            cache_dir = os.getenv("YALIS_CACHE", "~/.cache/yalis/")
            model_path = os.path.join(os.path.expanduser(cache_dir), "checkpoints", model_name)
        if not os.path.exists(model_path):
            raise ValueError(f"Model path does not exist: {model_path}")
        self.model_path = model_path

    def __repr__(self) -> str:
        return (
            f"ModelConfig(model_name={self.model_name}, model_path={self.model_path}, "
            f"precision={self.precision})"
        )


class InferenceConfig:
    """Sampling and batch limits (yalis/config.py:93-161, validation :163-211)."""

    def __init__(
        self,
        max_batch_size: int = 1,
        max_length_of_generated_sequences: int = 1024,
        top_k: Optional[int] = None,
        top_p: Optional[float] = 1.0,
        temperature: Optional[float] = 1.0,
        metrics: bool = False,
        tp_dims: Optional[Tuple[int, int, int]] = None,
        attention_backend: str = "hip",
        use_paged_kv_caching: bool = True,
        seed: int = 1234,
    ):
        self.max_batch_size = max_batch_size
        self.max_length = max_length_of_generated_sequences
        self.temperature = 1.0 if temperature is None else temperature
        self.top_k = top_k
        self.top_p = 1.0 if top_p is None else top_p
        self.metrics = metrics
        self.tp_dims = tp_dims
        self.attention_backend = attention_backend
        self.use_paged_kv_caching = use_paged_kv_caching
        self.seed = seed  # the reference seeds everything with 1234 (yalis/initialize.py:27)
        self._validate()

    def _validate(self) -> None:
        if self.max_batch_size <= 0:
            raise ValueError("max_batch_size must be a positive integer.")
        if self.max_length <= 0:
            raise ValueError("max_length must be a positive integer.")
        if self.temperature < 0.0:
            raise ValueError("temperature must be >=0.0.")
        if self.top_k is not None and self.top_k <= 0:
            raise ValueError("top_k must be a positive integer.")
        if self.top_p < 0.0 or self.top_p > 1.0:
            raise ValueError("top_p must be in the range [0.0, 1.0].")
        if self.tp_dims is not None and tuple(self.tp_dims) != (1, 1, 1):
            raise ValueError("tp_dims: this engine runs on one GPU; leave tp_dims unset.")
        if self.attention_backend != "hip":
            raise ValueError(
                f"Invalid attention backend: {self.attention_backend}. This engine has one: 'hip'."
            )
        if not self.use_paged_kv_caching:
            raise ValueError("use_paged_kv_caching=False: this engine's cache is always paged.")

    def __repr__(self) -> str:
        return (
            f"InferenceConfig(max_batch_size={self.max_batch_size}, "
            f"max_length_of_generated_sequences={self.max_length}, top_k={self.top_k}, "
            f"top_p={self.top_p}, temperature={self.temperature})"
        )


@dataclass
class EngineConfig:
    """Sizes of the paged engine.

    page_size: tokens per cache page (a multiple of 16).
    num_pages: pages in each cache group's pool; None sizes the pool for
        ``max_num_seqs`` requests of ``max_model_len`` tokens.
    max_num_seqs: requests that may be live at once (also the number of state slots).
    max_model_len: longest sequence (prompt plus generated) a request may reach.
    max_num_batched_tokens: token budget of one step (decode tokens plus prompt portions).
    dtype: "bfloat16" or "float32" (the latter is the true 32-bit path).
    decode_graphs: replay steps that hold single tokens only from captured HIP graphs
        (the reference's YALIS_DISABLE_DECODE_CUDAGRAPHS switches the same off,
        yalis/engine.py:44-48).
    graph_memory_bytes, wide_tensors, tune_library_products: see the fields.
    """

    page_size: int = 64
    num_pages: Optional[int] = None
    max_num_seqs: int = 8
    max_model_len: int = 2048
    max_num_batched_tokens: int = 2048
    dtype: str = "bfloat16"
    device: str = "cuda:0"
    # capture steps of single tokens as HIP graphs; YALIS_DISABLE_DECODE_CUDAGRAPHS=1 turns the
    # default off, as it does in the reference
    decode_graphs: bool = field(default_factory=lambda: os.environ.get("YALIS_DISABLE_DECODE_CUDAGRAPHS", "0") != "1")
    # device memory that captured graphs may hold together (their logits, integer buffers and
    # private pools); the least recently replayed ones are dropped beyond it
    graph_memory_bytes: int = 1 << 30
    # "auto": a checkpoint stored wholly in 32 bits is narrowed to bfloat16 by the bfloat16
    # engine, as the reference casts every tensor to its parameter's dtype
    # (yalis/model_loading.py:172-173), while single tensors stored in 32 bits inside a 16-bit
    # checkpoint stay 32-bit; "keep": every tensor stored in 32 bits stays so; "cast": none does
    wide_tensors: str = "auto"
    # time the vendor library's candidates for new product shapes of up to 256 rows and keep the
    # fastest (the choice then depends on the run); off: its first candidate, the same everywhere
    tune_library_products: bool = False

    def __post_init__(self) -> None:
        self.dtype = canonical_dtype(self.dtype)
        if self.page_size <= 0 or self.page_size % 16 != 0:
            raise ValueError(f"page_size must be a positive multiple of 16, got {self.page_size}")
        if self.max_num_seqs <= 0:
            raise ValueError("max_num_seqs must be positive")
        if self.max_model_len <= 0:
            raise ValueError("max_model_len must be positive")
        if self.max_num_batched_tokens <= 0:
            raise ValueError("max_num_batched_tokens must be positive")
        if self.num_pages is not None and self.num_pages <= 0:
            raise ValueError("num_pages must be positive")
        if self.wide_tensors not in ("auto", "keep", "cast"):
            raise ValueError(f"wide_tensors must be 'auto', 'keep' or 'cast', got {self.wide_tensors!r}")
        if self.graph_memory_bytes < 0:
            raise ValueError("graph_memory_bytes must not be negative")

    def pages_per_request(self) -> int:
        return -(-self.max_model_len // self.page_size)

    def resolved_num_pages(self) -> int:
        if self.num_pages is not None:
            return self.num_pages
        return self.pages_per_request() * self.max_num_seqs
