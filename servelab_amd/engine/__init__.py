from .batch import StepBatch, StepEntry, pack_batch
from .runner import ModelRunner, OutOfPages
from .sampling_params import SamplingParams
from .request import Request, Timeline
from .output import CompletionOutput, RequestOutput, result_of
from .scheduler import Plan, Planned, Scheduler
from .llm_engine import LLMEngine
