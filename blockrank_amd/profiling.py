"""Raw HIP events for timing one kernel inside a longer sequence of work.

torch.cuda.Event can only be recorded from Python between launches; the library's
br_prefill_fwd_events records a pair of events around its main kernel itself, and needs plain
hipEvent_t handles for that.  These come from the same HIP runtime PyTorch has already loaded.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_void_p

_hip = None


def _rt():
    global _hip
    if _hip is None:
        _hip = ctypes.CDLL("libamdhip64.so")
        _hip.hipEventCreate.argtypes = [ctypes.POINTER(c_void_p)]
        _hip.hipEventDestroy.argtypes = [c_void_p]
        _hip.hipEventSynchronize.argtypes = [c_void_p]
        _hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(c_float), c_void_p, c_void_p]
    return _hip


class EventPair:
    """Two hipEvent_t; pass ``pair.handles`` as ``kernel_events`` and read ``elapsed_ms()`` after a
    synchronisation point."""

    def __init__(self):
        rt = _rt()
        self.start, self.stop = c_void_p(), c_void_p()
        for e in (self.start, self.stop):
            rc = rt.hipEventCreate(ctypes.byref(e))
            if rc != 0:
                raise RuntimeError(f"hipEventCreate failed with {rc}")

    @property
    def handles(self):
        return (self.start, self.stop)

    def elapsed_ms(self) -> float:
        rt = _rt()
        rt.hipEventSynchronize(self.stop)
        ms = c_float()
        rc = rt.hipEventElapsedTime(ctypes.byref(ms), self.start, self.stop)
        if rc != 0:
            raise RuntimeError(f"hipEventElapsedTime failed with {rc}")
        return ms.value

    def __del__(self):
        try:
            rt = _rt()
            rt.hipEventDestroy(self.start)
            rt.hipEventDestroy(self.stop)
        except Exception:
            pass
