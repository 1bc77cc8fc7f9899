from .step import ModelRunner, OutOfPages, StepContext, StepEntry
from .loading import build_model, load_model, make_runner, parse_dtype, random_model

__all__ = ["ModelRunner", "OutOfPages", "StepContext", "StepEntry", "build_model",
           "load_model", "make_runner", "parse_dtype", "random_model"]
from .scheduler import ReqResult, Request, Scheduled, Scheduler, SchedulerConfig  # noqa: E402
from .engine import Engine  # noqa: E402

__all__ += ["ReqResult", "Request", "Scheduled", "Scheduler", "SchedulerConfig", "Engine"]
