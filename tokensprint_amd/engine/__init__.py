from tokensprint_amd.engine.batch import BatchBuilder, StepBatch, StepEntry
from tokensprint_amd.engine.runner import ModelRunner

__all__ = ["BatchBuilder", "StepBatch", "StepEntry", "ModelRunner"]
