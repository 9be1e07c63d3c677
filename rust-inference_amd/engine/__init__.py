from .generate import GenerationResult, GenerationStats, generate, plan_batches, run_batch
from .step import Engine, StepEntry, plan_step, wanted_indices

__all__ = ["GenerationResult", "GenerationStats", "generate", "plan_batches", "run_batch", "Engine", "StepEntry",
           "plan_step", "wanted_indices"]
