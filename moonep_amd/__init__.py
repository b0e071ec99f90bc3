"""moonep_amd: MoonEP's per-rank hot path (planner, dispatch, combine,
prefetch_weight, reduce_grad) as hand-written HIP kernels for MI355X, behind
the ``moonep.Buffer`` API.  ``import moonep_amd as moonep`` is the drop-in."""

from .api import Buffer, EmulatedWorld
from .planning import MoonEPCommPlan

__all__ = ["Buffer", "MoonEPCommPlan", "EmulatedWorld"]
