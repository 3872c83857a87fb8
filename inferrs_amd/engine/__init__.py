from .batch import GroupStep, StepBuilder, StepContext
from .model import DecoderModel, parse_dtype
from .engine import Engine, Entry, StepError
from .replay import TraceError, run_trace
from .trace import Trace, make_trace
from .scheduler import Plan, PlannedEntry, Request, Scheduler
from .generate import Generation, GenerationLoop, generate
