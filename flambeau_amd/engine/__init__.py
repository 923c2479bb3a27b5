from .llm import EngineOptions, LLMEngine, generate
from .loading import load_model, parse_dtype, random_model
from .runtime import Runtime
from .scheduler import AdmissionError, Request, Scheduled, Scheduler
from .step import ModelRunner, StepEntry, StepError
