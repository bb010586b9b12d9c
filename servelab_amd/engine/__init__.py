from .batch import StepBatch, StepEntry, pack_batch
from .runner import ModelRunner, OutOfPages
from .sampling_params import SamplingParams
from .sequence import Sequence, SequenceStatus, RequestMetrics
from .output import CompletionOutput, RequestOutput
from .scheduler import Scheduler, SchedulerOutput, PrefillSched
from .llm_engine import LLMEngine
