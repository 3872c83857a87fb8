from .batch import GroupStep, StepContext
from .model import DecoderModel, parse_dtype
from .engine import Engine, Entry, StepError
from .replay import TraceError, run_trace
