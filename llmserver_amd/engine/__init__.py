from .batch import Staging, StepContext, StepEntry
from .engine import Engine
from .loading import load_model, parse_dtype
from .request import (STREAM_END, CompletedRequest, Request, RequestFinishReason, RequestStateError, RequestStatus,
                      SamplingParams, TokenStream)
from .scheduler import Scheduler, SchedulerOutput
from .step import ModelRunner

__all__ = ["Staging", "StepContext", "StepEntry", "Engine", "load_model", "parse_dtype", "STREAM_END", "CompletedRequest",
           "Request", "RequestFinishReason", "RequestStateError", "RequestStatus", "SamplingParams", "TokenStream",
           "Scheduler", "SchedulerOutput", "ModelRunner"]
