from .engine import Engine, OutOfPages, StepEntry, StepError
