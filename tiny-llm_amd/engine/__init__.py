from .step import StepEntry, StepContext, ModelRunner, StepError
