"""MI355X-native inference engine for the Qwen2 dense decoder."""

from .config import EngineConfig
from .engine import LLM, RequestOutput, StepEntry, Trace
from .sampling import SamplingParams

__all__ = ["EngineConfig", "LLM", "RequestOutput", "SamplingParams", "StepEntry", "Trace"]
