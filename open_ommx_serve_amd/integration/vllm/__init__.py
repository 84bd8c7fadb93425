"""vLLM-facing seam: serving config, per-step managers, attention-backend classes."""
from .config import OMMXServingConfig, resolve_serving_config
from .metadata import (STEP_ROUTE_UNCLASSIFIED, OMMXBatchedStepManager, OMMXSlotAllocationError,
                       OMMXStepManager, assign_slots, detect_full_prefill, detect_step_route)

__all__ = ["OMMXServingConfig", "resolve_serving_config", "OMMXStepManager",
           "OMMXBatchedStepManager", "OMMXSlotAllocationError", "assign_slots",
           "detect_step_route", "detect_full_prefill", "STEP_ROUTE_UNCLASSIFIED"]
