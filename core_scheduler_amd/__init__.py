"""MI355X-native GPT-2 training kernels behind the CoreScheduler op API.

Layers, bottom up:
  csrc/kernels/*.hip   hand-written gfx950 kernels + the C ABI (include/cs_hip_kernels.h)
  _capi.py             ctypes binding of that C ABI
  ops.py               the ops on torch tensors (device memory and streams only)
  csrc/host/           C++ mirror of the reference's cs::compute / cs::optimizer API
"""
from . import _capi  # noqa: F401

__all__ = ["_capi", "ops"]


def __getattr__(name):
    if name == "ops":
        import importlib

        return importlib.import_module(".ops", __name__)
    raise AttributeError(name)
