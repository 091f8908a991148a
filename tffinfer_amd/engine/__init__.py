from .batch import StepBatch, StepEntry
from .runner import ModelRunner, StepError
