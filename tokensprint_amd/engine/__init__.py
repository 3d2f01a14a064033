from tokensprint_amd.engine.batch import BatchBuilder, StepBatch, StepEntry
from tokensprint_amd.engine.runner import ModelRunner

__all__ = ["BatchBuilder", "StepBatch", "StepEntry", "ModelRunner", "LLMEngine", "Scheduler",
           "Request", "RequestStatus"]


def __getattr__(name):
    if name == "LLMEngine":
        from tokensprint_amd.engine.llm_engine import LLMEngine
        return LLMEngine
    if name == "Scheduler":
        from tokensprint_amd.engine.scheduler import Scheduler
        return Scheduler
    if name in ("Request", "RequestStatus"):
        from tokensprint_amd.engine import request
        return getattr(request, name)
    raise AttributeError(name)
