from .batch import BatchBuilder, StepEntry
from .engine import Engine, GenerationResult, generate
from .llm import LLM, Output
from .metrics import percentile, summarize
from .request import Request, Scheduled, StepRecord
from .runner import ModelRunner, load_runner
from .scheduler import Scheduler

__all__ = ["BatchBuilder", "StepEntry", "Engine", "GenerationResult", "generate", "LLM", "Output", "Request",
           "Scheduled", "StepRecord", "ModelRunner", "load_runner", "Scheduler", "percentile", "summarize"]
