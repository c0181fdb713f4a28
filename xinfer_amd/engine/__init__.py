from .loading import build_model, load_model, parse_dtype
from .model import CausalLM
from .runner import ModelRunner, StepEntry, StepError
from .scheduler import PlannedEntry, RequestTooLarge, Scheduler, SchedulerError
from .llm_engine import LLMEngine
