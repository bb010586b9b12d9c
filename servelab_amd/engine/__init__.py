from .batch import StepBatch, StepEntry, pack_batch
from .runner import ModelRunner, OutOfPages
