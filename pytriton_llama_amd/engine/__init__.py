from .batch import StepContext, StepEntry, build_context
from .request import Request, SamplingParams, StepOutput
from .scheduler import Scheduler, StepPlan
from .runner import ModelRunner
from .llm import Engine
