from docc_amd.compiler.compiled_sdfg import CompiledSDFG
from docc_amd.compiler.docc_program import DoccProgram

__all__ = ["CompiledSDFG", "DoccProgram"]
