from .engine import CacheFull, Engine, Generated, Request, RunMetrics
from .generate import generate, plan_batch

__all__ = ["CacheFull", "Engine", "Generated", "Request", "RunMetrics", "generate", "plan_batch"]
