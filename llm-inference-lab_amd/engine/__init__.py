from .model import CausalLM, EntryView
from .step import StepEntry, StepContext, StepFunction, GroupView
from .engine import Engine, parse_dtype, settle_collector, write_random_model
