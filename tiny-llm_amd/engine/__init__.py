from .step import StepEntry, SampleSpec, StepContext, ModelRunner, StepError, StepGraph, Layout, fill_metadata
from .scheduler import Scheduler, Request, StepPlan, Scheduled
from .engine import Engine
