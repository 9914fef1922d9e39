"""The step function, its batch, and the scheduler above it."""
from .batch import Entry, StepBatch
from .engine import DEFAULT_PAGE_SIZE, Engine, OutOfPages, StepError
from .generate import Generation, GenerationStats, Generator, generate
from .scheduler import (MAX_PREFILL_CHUNK, ContinuousBatchScheduler, FinishReason, Sequence, SequenceState,
                        StepOutput)
