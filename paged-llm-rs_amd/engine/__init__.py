from .batch import StepBatch, StepEntry, build_batch
from .engine import Completion, Engine, generate
from .replay import Replayer
from .scheduler import Outcome, Plan, Scheduler
from .step import StepOutput, StepRunner, commit_step, run_step

__all__ = ["StepBatch", "StepEntry", "build_batch", "Completion", "Engine", "generate", "Replayer", "Outcome",
           "Plan", "Scheduler", "StepOutput", "StepRunner", "commit_step", "run_step"]
