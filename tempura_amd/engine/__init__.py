from .model import CausalLM, expected_weights
from .runner import ModelRunner, StepEntry, StepContext
from .scheduler import Scheduler, SchedulerConfig, Request, RequestState
from .loading import load_model, random_model
from .engine import Engine

__all__ = ["CausalLM", "expected_weights", "ModelRunner", "StepEntry", "StepContext", "Scheduler",
           "SchedulerConfig", "Request", "RequestState", "load_model", "random_model", "Engine"]
