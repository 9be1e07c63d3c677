from .generate import GenerationResult, GenerationStats, generate, plan_batches, run_batch
from .step import Engine, StepEntry, wanted_indices

__all__ = ["GenerationResult", "GenerationStats", "generate", "plan_batches", "run_batch", "Engine", "StepEntry",
           "wanted_indices"]
