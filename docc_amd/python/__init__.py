"""`docc_amd.python`: the `@native` front end and the target registry, with the names the
reference exports from `docc.python` (python/docc/python/__init__.py:1-13).

Importing this package registers the `rocm` target through the same hook a third-party
target would use (`register_target_overrides`)."""
from docc_amd.python.functions import conv2d, erf, relu, sigmoid, softmax
from docc_amd.python.python_program import PythonProgram, _map_python_type, bfloat16, native
from docc_amd.python.target_registry import (get_target_compile_fn, get_target_schedule_fn, register_target,
                                             register_target_overrides, unregister_target)


def _rocm_schedule(sdfg, category, options):
    """schedule_fn of the rocm target: node mapping, offloading, transfer minimisation."""
    sdfg.schedule("rocm", category, False, options)


def _rocm_compile(sdfg, output_folder, instrumentation_mode, capture_args, options):
    """compile_fn of the rocm target: host C++ against the thin HIP runtime -> lib<name>.so."""
    return sdfg._compile(output_folder, "rocm", instrumentation_mode, capture_args)


register_target_overrides("rocm", _rocm_schedule, _rocm_compile)

__all__ = ["PythonProgram", "native", "bfloat16", "register_target", "register_target_overrides", "unregister_target",
           "get_target_schedule_fn", "get_target_compile_fn", "softmax", "conv2d", "relu", "sigmoid", "erf", "_map_python_type"]
