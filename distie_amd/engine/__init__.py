from .batch import StepEntry
from .llm import LLM, RequestOutput, Trace
from .model import Model
from .runner import ModelRunner
from .scheduler import BlockPoolExhausted, Emission, Scheduler, Phase, Portion, Request, StepPlan

__all__ = ["StepEntry", "LLM", "RequestOutput", "Trace", "Model", "ModelRunner", "BlockPoolExhausted",
           "Emission", "Scheduler", "Phase", "Portion", "Request", "StepPlan"]
