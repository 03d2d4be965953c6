from .engine import Engine, OutOfPages, StepEntry, StepError
from .scheduler import (BatchConfig, DecodeTask, FinishReason, GenerationEvent, PrefillTask, Scheduler,
                        SchedulerOutput, SequencePhase, SequenceState)
from .runtime import GenerationError, Runtime, load_tokenizer
