from .loading import load_model, parse_dtype, random_model
from .runtime import Runtime
from .step import ModelRunner, StepEntry, StepError
