"""MI355X-native backend behind cltorch's ``torch.ClTensor`` operator API.

``libthcl_hip.so`` (built by ``python -m cltorch_amd.build``) is the product: a
C-ABI library exporting the reference's ``THClTensor_*`` entry points for the
pointwise / copy / reduce / addmm path.  ``ClTensor`` mirrors the Lua methods
on top of it.  Importing this package does not touch a GPU; the first tensor
does, and raises if no device or no built library is present.
"""
from .tensor import (pinned_array, about, dumpTimings, getDevice, getDeviceProperties, manualSeed, setDetailedTimings, setDevice, setEnableTiming, setTiming, setTrace,  # noqa: F401
                     ClError, ClKernel, ClStorage, ClTensor, dumpProfiling, emptyCache, memoryStats, setProfiling, finish, ger, getDeviceCount, mm, mv, setAddFinish, state,  # noqa: F401
                     synchronize)
from .serialize import load, save  # noqa: F401
from .printing import storage_tostring, tensor_tostring  # noqa: F401
from . import _lib  # noqa: F401

__all__ = ["pinned_array", "about", "dumpTimings", "getDevice", "getDeviceProperties", "manualSeed", "setDetailedTimings", "setDevice", "setEnableTiming", "setTiming", "setTrace", "ClTensor", "ClStorage", "ClError", "ClKernel", "mm", "mv", "ger", "synchronize", "finish", "setProfiling", "dumpProfiling", "memoryStats", "emptyCache", "getDeviceCount", "setAddFinish", "state", "save", "load", "tensor_tostring", "storage_tostring"]
