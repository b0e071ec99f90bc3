"""The reference's import name for the MI355X build: ``from moonep import Buffer,
MoonEPCommPlan`` (reference moonep/__init__.py:1-9) and ``moonep.api``, ``moonep.planning``,
``moonep.dispatch`` ... resolve to the modules of ``moonep_amd``.  Nothing lives here."""

import importlib
import sys

from moonep_amd import Buffer, MoonEPCommPlan

__all__ = ["Buffer", "MoonEPCommPlan"]

_SAME_NAME = ("api", "planning", "dispatch", "combine", "prefetch", "grad_reduce", "constants")
# the reference keeps the two destination-side launchers in files of their own
_ELSEWHERE = {"dispatch_epilogue": "dispatch", "combine_prologue": "combine"}

for _name, _target in [(n, n) for n in _SAME_NAME] + list(_ELSEWHERE.items()):
    _module = importlib.import_module(f"moonep_amd.{_target}")
    sys.modules[f"{__name__}.{_name}"] = _module
    setattr(sys.modules[__name__], _name, _module)
