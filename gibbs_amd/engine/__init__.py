"""The step function, its batch, and the scheduler above it."""
from .batch import Entry, StepBatch
from .engine import Engine, OutOfPages, StepError
