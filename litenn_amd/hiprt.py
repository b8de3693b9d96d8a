"""Minimal ctypes view of the HIP runtime for harness code: streams, events and graph capture.

The benchmark and tests use it to time kernels with events recorded on the stream the kernels are
launched on, and to replay a captured sequence of launches without host overhead.  Nothing here
computes anything.
"""
from __future__ import annotations

import ctypes as C
import ctypes.util


class HipError(RuntimeError):
    pass


_rt = None


def rt() -> C.CDLL:
    global _rt
    if _rt is None:
        for name in ("libamdhip64.so", "libamdhip64.so.7", "/opt/rocm/lib/libamdhip64.so"):
            try:
                _rt = C.CDLL(name)
                break
            except OSError:
                continue
        else:
            raise HipError("libamdhip64.so not found")
        _rt.hipGetErrorString.restype = C.c_char_p
    return _rt


def _check(err: int) -> None:
    if err != 0:
        raise HipError(rt().hipGetErrorString(err).decode())


class Stream:
    def __init__(self):
        self.handle = C.c_void_p()
        _check(rt().hipStreamCreate(C.byref(self.handle)))

    def synchronize(self) -> None:
        _check(rt().hipStreamSynchronize(self.handle))

    def begin_capture(self) -> None:
        _check(rt().hipStreamBeginCapture(self.handle, 2))  # hipStreamCaptureModeRelaxed

    def end_capture(self) -> "Graph":
        g = C.c_void_p()
        _check(rt().hipStreamEndCapture(self.handle, C.byref(g)))
        return Graph(g)

    def destroy(self) -> None:
        if self.handle:
            rt().hipStreamDestroy(self.handle)
            self.handle = C.c_void_p()


class Graph:
    def __init__(self, graph):
        self.graph = graph
        self.exec = C.c_void_p()
        _check(rt().hipGraphInstantiate(C.byref(self.exec), graph, None, None, C.c_size_t(0)))

    def launch(self, stream: Stream) -> None:
        _check(rt().hipGraphLaunch(self.exec, stream.handle))

    def destroy(self) -> None:
        if self.exec:
            rt().hipGraphExecDestroy(self.exec)
            rt().hipGraphDestroy(self.graph)
            self.exec = C.c_void_p()


class Event:
    def __init__(self):
        self.handle = C.c_void_p()
        _check(rt().hipEventCreate(C.byref(self.handle)))

    def record(self, stream: Stream) -> None:
        _check(rt().hipEventRecord(self.handle, stream.handle))

    def synchronize(self) -> None:
        _check(rt().hipEventSynchronize(self.handle))

    def elapsed_ms(self, later: "Event") -> float:
        ms = C.c_float()
        _check(rt().hipEventElapsedTime(C.byref(ms), self.handle, later.handle))
        return float(ms.value)


def device_synchronize() -> None:
    _check(rt().hipDeviceSynchronize())
