from .batch import SeqInfo, StepEntry, StepLayout, StepState, build_step, layout_step
from .llm_engine import LLMEngine
from .request import Request, RequestStatus
from .runner import ModelRunner
from .scheduler import Portion, Scheduler

__all__ = ["LLMEngine", "ModelRunner", "Portion", "Request", "RequestStatus", "Scheduler", "SeqInfo", "StepEntry",
           "StepState", "build_step"]
