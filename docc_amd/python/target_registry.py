"""Registry of target hooks, with the reference's names and signatures
(python/docc/python/target_registry.py:4-42):

    schedule_fn(sdfg, category: str, options: dict) -> None
    compile_fn(sdfg, output_folder: str, instrumentation_mode: str, capture_args: bool, options: dict) -> str

The `rocm` target registers itself through this same door (see docc_amd/python/__init__.py).
"""
from __future__ import annotations

from typing import Any, Callable, Dict, Optional

from docc_amd.sdfg import StructuredSDFG

TargetScheduleFn = Callable[[StructuredSDFG, str, Dict[str, Any]], None]
LegacyTargetScheduleFn = Callable[[StructuredSDFG, str], None]
TargetCompileFn = Callable[[StructuredSDFG, str, str, bool, Dict[str, Any]], str]

_target_schedule_registry: Dict[str, TargetScheduleFn] = {}
_target_compile_registry: Dict[str, TargetCompileFn] = {}


def register_target(name: str, schedule_fn: Optional[LegacyTargetScheduleFn]) -> None:
    """Two-argument (legacy) schedule hook."""
    if schedule_fn is None:
        return

    def wrapper(sdfg: StructuredSDFG, category: str, options: Optional[Dict[str, Any]] = None) -> None:
        schedule_fn(sdfg, category)

    register_target_overrides(name, schedule_fn=wrapper, compile_fn=None)


def register_target_overrides(name: str, schedule_fn: Optional[TargetScheduleFn],
                              compile_fn: Optional[TargetCompileFn] = None) -> None:
    if schedule_fn is not None:
        _target_schedule_registry[name] = schedule_fn
    if compile_fn is not None:
        _target_compile_registry[name] = compile_fn


def unregister_target(name: str) -> None:
    _target_schedule_registry.pop(name, None)
    _target_compile_registry.pop(name, None)


def get_target_schedule_fn(name: str) -> Optional[TargetScheduleFn]:
    return _target_schedule_registry.get(name)


def get_target_compile_fn(name: str) -> Optional[TargetCompileFn]:
    return _target_compile_registry.get(name)
