from .step import (CacheContext, CapacityError, ModelRunner, StepCommittedError, StepContext, StepEntry,
                   Workspace)
from .scheduler import ContinuousBatchScheduler, SequenceResult
from .engine import BlockManager, Engine, parse_dtype

__all__ = ["CacheContext", "CapacityError", "ModelRunner", "StepCommittedError", "StepContext", "StepEntry", "Workspace",
           "ContinuousBatchScheduler", "SequenceResult", "BlockManager", "Engine", "parse_dtype"]
