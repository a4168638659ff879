"""The step function, the scheduler above it, the engine loop and trace replay."""
from .request import GenerateRequestOutput, InferenceOutput, Request, RequestMetrics, Status
from .scheduler import ScheduledEntry, ScheduleOutput, Scheduler
from .step import ModelRunner, RunnerCache, StepContext, StepEntry, StepError

__all__ = ["GenerateRequestOutput", "InferenceOutput", "Request", "RequestMetrics", "Status", "ScheduledEntry",
           "ScheduleOutput", "Scheduler", "ModelRunner", "RunnerCache", "StepContext", "StepEntry", "StepError"]
