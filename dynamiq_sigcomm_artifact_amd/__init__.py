"""MI355X-native implementation of the gradient-compression path behind
DynamiQ's ``eden_utils`` extension.

``eden_utils``   the drop-in Python module (same functions as the reference's)
``capi``         ctypes access to the C ABI of ``libdynamiq_eden.so``

Both need the in-tree native build (``python -m dynamiq_sigcomm_artifact_amd.build``)
and raise if it is missing; there is no CPU fallback.
"""
import importlib
import os
import sys

__all__ = ["capi", "load_eden_utils"]

from . import capi  # noqa: E402


def load_eden_utils():
    """Import the pybind11 module that sits next to this file."""
    name = __name__ + ".eden_utils"
    if name in sys.modules:
        return sys.modules[name]
    try:
        return importlib.import_module(name)
    except ImportError as exc:
        raise RuntimeError(
            "the eden_utils extension is not built (%s): run `python -m dynamiq_sigcomm_artifact_amd.build`"
            % exc) from exc


def __getattr__(attr):
    if attr == "eden_utils":
        return load_eden_utils()
    raise AttributeError(attr)
