from .step import StepEntry, StepContext, ModelRunner, StepError
from .scheduler import Scheduler, Request, StepPlan, Scheduled
from .engine import Engine
