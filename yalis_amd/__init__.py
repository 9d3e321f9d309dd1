"""yalis_amd: a small, whole inference engine for one MI355X.

The public names follow the reference (yalis/__init__.py:2-13).
"""
from .config.runtime import EngineConfig, InferenceConfig, ModelConfig  # noqa: F401
from .engine.llm_engine import LLMEngine, print_rank0  # noqa: F401
from .sampling.sampler import SamplingParams  # noqa: F401
