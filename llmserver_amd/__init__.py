"""llmserver_amd: a small single-GPU inference engine for the Qwen3 dense decoder on MI355X."""
from . import models  # noqa: F401  (registers the architectures)
from .config import load_config, register_architecture
from .engine import Engine, ModelRunner, StepEntry, load_model
from .entrypoints import generate, model_loader

__version__ = "0.1.0"
__all__ = ["load_config", "register_architecture", "Engine", "ModelRunner", "StepEntry", "load_model", "generate",
           "model_loader"]
