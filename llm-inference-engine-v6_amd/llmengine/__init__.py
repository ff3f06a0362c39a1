"""llmengine: a small, whole LLM inference engine for one AMD Instinct MI355X.

Public names follow the reference's Python package (python/llmengine/__init__.py:6-26):
`Engine`, `BlockManager`, `ContinuousBatchScheduler`, `SequenceResult`.
"""
from . import config, parts, models, cache, weights, sampling          # noqa: F401  (models registers Llama)
from .config import ConfigError, LlamaConfig, load_config, register_architecture
from .engine import (BlockManager, CapacityError, ContinuousBatchScheduler, Engine, SequenceResult,
                     StepCommittedError, StepEntry)
from .weights import WeightError, write_random_model

__version__ = "0.1.0"

__all__ = ["Engine", "BlockManager", "ContinuousBatchScheduler", "SequenceResult", "StepEntry",
           "CapacityError", "StepCommittedError", "ConfigError", "WeightError", "LlamaConfig", "load_config",
           "register_architecture", "write_random_model"]
