"""Base class of the JIT front ends; same constructor and abstract surface as the
reference's DoccProgram (python/docc/compiler/docc_program.py:8-49)."""
from __future__ import annotations

from abc import ABC, abstractmethod
from typing import Any, Optional

from docc_amd.compiler.compiled_sdfg import CompiledSDFG
from docc_amd.sdfg import StructuredSDFG


class DoccProgram(ABC):
    def __init__(self, name: str, target: str = "none", category: str = "server",
                 instrumentation_mode: Optional[str] = None, capture_args: Optional[bool] = None,
                 remote_tuning: bool = False):
        self.name = name
        self.target = target
        self.category = category
        self.instrumentation_mode = instrumentation_mode
        self.capture_args = capture_args
        self.remote_tuning = remote_tuning
        self.last_sdfg: Optional[StructuredSDFG] = None
        self.cache: dict = {}

    @abstractmethod
    def __call__(self, *args: Any) -> Any: ...

    @abstractmethod
    def compile(self, *args: Any, output_folder: Optional[str] = None) -> CompiledSDFG: ...

    @abstractmethod
    def to_sdfg(self, *args: Any) -> StructuredSDFG: ...

    @abstractmethod
    def _convert_inputs(self, args: tuple) -> tuple: ...

    @abstractmethod
    def _convert_outputs(self, result: Any, original_args: tuple) -> Any: ...

    def _get_cache_key(self, *args: Any) -> str:
        return ""
