from .llm_engine import LLMEngine, RequestOutput, StepOutput
from .runner import ModelRunner, StepContext, StepEntry
from .scheduler import Request, ScheduledEntry, ScheduledStep, Scheduler
