from .batch import Arena, BatchBuilder, PagedMeta, StepContext, StepEntry
from .model import Model, expected_tensors
from .engine import Engine
from .sizing import MemoryPlan, plan_memory

__all__ = ["Arena", "BatchBuilder", "PagedMeta", "StepContext", "StepEntry", "Model", "expected_tensors", "Engine", "MemoryPlan",
           "plan_memory"]
