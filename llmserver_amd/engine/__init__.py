from .batch import Staging, StepContext, StepEntry
from .engine import CompletedHistory, Engine, EngineConfig
from .loading import load_model, parse_dtype
from .request import (CompletedRequest, Request, RequestFinishReason, RequestStateError, RequestStatus, SamplingParams)
from .scheduler import PageBudget, Scheduler, StepPlan
from .step import ModelRunner
from .stream import STREAM_END, ByteLevelText, ByteLevelVocabulary, TokenStream

__all__ = ["Staging", "StepContext", "StepEntry", "CompletedHistory", "Engine", "EngineConfig", "load_model", "parse_dtype",
           "STREAM_END", "CompletedRequest", "Request", "RequestFinishReason", "RequestStateError", "RequestStatus",
           "SamplingParams", "TokenStream", "ByteLevelText", "ByteLevelVocabulary", "PageBudget", "Scheduler", "StepPlan",
           "ModelRunner"]
