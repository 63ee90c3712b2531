from .llm_engine import LLMEngine, StepOutput
from .runner import ModelRunner, StepContext, StepEntry
from .scheduler import Request, ScheduledEntry, ScheduledStep, Scheduler
