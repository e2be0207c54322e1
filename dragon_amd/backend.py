"""Loads the compiled module of the host layer, ``lib/libdragon_hip_python*.so``
(pybind11 over the C++ Workspace / Tensor / HIPContext classes), the way the
reference's ``backend.py`` imports its ``libdragon_python``
(dragon/python/core/framework/backend.py:27-37). Attribute access on this
module forwards to it: ``backend.Workspace``, ``backend.hipGetDeviceCount()`` ...
"""

import glob
import importlib.util
import os

from . import _lib

_HERE = os.path.dirname(os.path.abspath(__file__))
_module = None


def load():
    """The compiled module; raises if it is not built (there is no Python fallback)."""
    global _module
    if _module is None:
        paths = sorted(glob.glob(os.path.join(_HERE, "lib", "libdragon_hip_python*.so")))
        if not paths:
            raise RuntimeError("dragon_amd/lib/libdragon_hip_python*.so is missing: build it with "
                               "`python -c 'import __graft_entry__ as g; g.build()'`")
        _lib.lib()  # binds the kernel library (and the HIP runtime torch ships) first
        spec = importlib.util.spec_from_file_location("libdragon_hip_python", paths[0])
        module = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(module)
        _module = module
    return _module


def __getattr__(name):
    return getattr(load(), name)
