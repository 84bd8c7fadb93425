from .batched_seam import BatchedDecodePlan, BatchedStepPlanner

__all__ = ["BatchedDecodePlan", "BatchedStepPlanner"]
