"""HIP events through ctypes, for timing work on the very stream the library launches on.

The handles are plain ``hipEvent_t`` values, which is what ``odsd_moe_forward_events`` takes;
``torch.cuda.Event`` creates its handle lazily and records on torch's current stream only.
"""
from __future__ import annotations

import ctypes as C
from typing import List, Optional

_rt: Optional[C.CDLL] = None


def runtime() -> C.CDLL:
    """The HIP runtime already loaded into this process (by torch and by libodsd_moe.so)."""
    global _rt
    if _rt is None:
        rt = _open_runtime()
        rt.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        rt.hipEventDestroy.argtypes = [C.c_void_p]
        rt.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        rt.hipEventSynchronize.argtypes = [C.c_void_p]
        rt.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        _rt = rt
    return _rt


def _open_runtime() -> C.CDLL:
    """The copy of libamdhip64 that is mapped into this process, whatever its version suffix or
    directory (a torch wheel may bring its own); failing that, the usual names in turn."""
    try:
        with open("/proc/self/maps") as f:
            for line in f:
                path = line.rsplit(None, 1)[-1]
                if "libamdhip64.so" in path and path.startswith("/"):
                    return C.CDLL(path)
    except OSError:
        pass
    last = None
    for name in ("libamdhip64.so", "libamdhip64.so.7", "libamdhip64.so.6", "libamdhip64.so.5"):
        try:
            return C.CDLL(name)
        except OSError as e:
            last = e
    raise OSError(f"the HIP runtime (libamdhip64) is neither mapped into this process nor loadable: {last}")


def _check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what} failed with HIP error {rc}")


class EventList:
    """n timing events; ``array`` is the ``void *[n]`` a C call expects."""

    def __init__(self, n: int):
        rt = runtime()
        self.n = n
        self.array = (C.c_void_p * n)()
        for i in range(n):
            ev = C.c_void_p()
            _check(rt.hipEventCreate(C.byref(ev)), "hipEventCreate")
            self.array[i] = ev

    def record(self, i: int, stream: int) -> None:
        _check(runtime().hipEventRecord(self.array[i], C.c_void_p(stream)), "hipEventRecord")

    def elapsed_ms(self, i: int, j: int) -> float:
        out = C.c_float()
        _check(runtime().hipEventElapsedTime(C.byref(out), self.array[i], self.array[j]), "hipEventElapsedTime")
        return out.value

    def kernel_ms(self, mask: int) -> List[float]:
        """Events (2k, 2k+1) are the start / stop events of kernel slot k: the duration of every
        slot whose bit is set in ``mask``, 0.0 for the others."""
        return [self.elapsed_ms(2 * k, 2 * k + 1) if (mask >> k) & 1 else 0.0 for k in range(self.n // 2)]

    def kernel_ms_at(self, base: int, mask: int, n_slots: int) -> List[float]:
        """The same for a list that holds the events of several calls one after the other: the
        ``n_slots`` kernel slots whose events start at index ``base``."""
        return [self.elapsed_ms(base + 2 * k, base + 2 * k + 1) if (mask >> k) & 1 else 0.0 for k in range(n_slots)]

    def __del__(self):
        try:
            rt = runtime()
            for i in range(self.n):
                rt.hipEventDestroy(self.array[i])
        except Exception:
            pass
