from .engine import Engine, EngineOptions, StepEntry, StepError
from .graph import SampledTokens, TokenRef
from .model import CachePlan, Model, collect_weight_specs
from .scheduler import Request, Scheduler, SchedulerError, StepPlan

__all__ = ["Engine", "EngineOptions", "StepEntry", "StepError", "CachePlan", "Model",
           "collect_weight_specs", "SampledTokens", "TokenRef", "Request", "Scheduler", "SchedulerError", "StepPlan"]
