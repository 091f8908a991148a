from .batch import StepBatch, StepEntry
from .runner import ModelRunner, StepError
from .llm_engine import EngineOptions, GenerationResult, LLMEngine
from .scheduler import Request, RequestRefused, Scheduler, SchedulerOptions
