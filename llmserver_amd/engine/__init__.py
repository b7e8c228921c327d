from .batch import Staging, StepContext, StepEntry
from .loading import load_model, parse_dtype
from .step import ModelRunner

__all__ = ["Staging", "StepContext", "StepEntry", "load_model", "parse_dtype", "ModelRunner"]
