from .batch import StepBatch, StepEntry
from .runner import ModelRunner, load_model, resolve_dtype
from .scheduler import Scheduled, Scheduler
from .sequence import Sequence, SequenceStatus
