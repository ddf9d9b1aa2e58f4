from .batch import StepBatch, StepEntry, build_batch
from .step import commit_step, run_step

__all__ = ["StepBatch", "StepEntry", "build_batch", "commit_step", "run_step"]
