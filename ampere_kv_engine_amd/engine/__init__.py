from .batch import LAST_TOKEN, Arena, BatchBuilder, PagedMeta, StepContext, StepEntry
from .model import Model, expected_tensors
from .engine import Engine
from .sizing import MemoryPlan, plan_memory

__all__ = ["LAST_TOKEN", "Arena", "BatchBuilder", "PagedMeta", "StepContext", "StepEntry", "Model", "expected_tensors", "Engine", "MemoryPlan",
           "plan_memory"]
