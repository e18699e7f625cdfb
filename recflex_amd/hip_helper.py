"""Device queries and profiler range control through ``libamdhip64.so`` (ctypes).

Stands where the reference has ``RecFlex/cuda_helper.py:21-85`` (``CudaInfoQuerier`` on libcuda:
SM count, max threads per SM, compute capability; ``CudaProfiler`` on libcudart).  The GPU pool
is ``HIP_VISIBLE_DEVICES`` (or ``CUDA_VISIBLE_DEVICES``, which the HIP runtime honours too); if
neither is set, every device the runtime reports is used -- the reference requires the
variable to be set (``cuda_helper.py:25``).
"""

import ctypes
import os
from typing import List, Tuple

HIP_SUCCESS = 0
# values of hipDeviceAttribute_t in hip/hip_runtime_api.h (ROCm 7)
HIP_DEVICE_ATTRIBUTE_CLOCK_RATE = 5
HIP_DEVICE_ATTRIBUTE_L2_CACHE_SIZE = 19
HIP_DEVICE_ATTRIBUTE_COMPUTE_CAPABILITY_MAJOR = 23
HIP_DEVICE_ATTRIBUTE_MAX_THREADS_PER_MULTIPROCESSOR = 57
HIP_DEVICE_ATTRIBUTE_COMPUTE_CAPABILITY_MINOR = 61
HIP_DEVICE_ATTRIBUTE_MULTIPROCESSOR_COUNT = 63
HIP_DEVICE_ATTRIBUTE_WARP_SIZE = 87
HIP_DEVICE_ATTRIBUTE_MAX_SHARED_MEMORY_PER_MULTIPROCESSOR = 10002
HIP_DEVICE_ATTRIBUTE_WALL_CLOCK_RATE = 10017


def _load_hip() -> ctypes.CDLL:
    for name in ("libamdhip64.so", "/opt/rocm/lib/libamdhip64.so"):
        try:
            return ctypes.CDLL(name)
        except OSError:
            continue
    raise OSError("libamdhip64.so not found")


class HipInfoQuerier:
    def __init__(self):
        self.hip = _load_hip()
        self.hip.hipGetErrorString.restype = ctypes.c_char_p
        visible = os.environ.get("HIP_VISIBLE_DEVICES") or os.environ.get("CUDA_VISIBLE_DEVICES")
        if visible:
            self.gpu_ids: List[int] = [int(v) for v in visible.split(',') if v.strip() != ""]
        else:
            self.gpu_ids = list(range(self.get_device_count()))

    def hip_check(self, result: int) -> None:
        if result != HIP_SUCCESS:
            msg = self.hip.hipGetErrorString(result)
            raise Exception(f"HIP function call failed with error code {result}: "
                            f"{msg.decode() if msg else '?'}")

    def get_device_count(self) -> int:
        n = ctypes.c_int(0)
        self.hip_check(self.hip.hipGetDeviceCount(ctypes.byref(n)))
        return n.value

    def get_attribute(self, attr: int, dev_ordinal: int = 0) -> int:
        v = ctypes.c_int(0)
        self.hip_check(self.hip.hipDeviceGetAttribute(ctypes.byref(v), attr, dev_ordinal))
        return v.value

    def get_compute_capability(self, dev_ordinal: int = 0) -> Tuple[int, int]:
        return (self.get_attribute(HIP_DEVICE_ATTRIBUTE_COMPUTE_CAPABILITY_MAJOR, dev_ordinal),
                self.get_attribute(HIP_DEVICE_ATTRIBUTE_COMPUTE_CAPABILITY_MINOR, dev_ordinal))

    def get_sm_thread_count(self, dev_ordinal: int = 0) -> Tuple[int, int]:
        """(compute units, max resident threads per compute unit)."""
        return (self.get_attribute(HIP_DEVICE_ATTRIBUTE_MULTIPROCESSOR_COUNT, dev_ordinal),
                self.get_attribute(HIP_DEVICE_ATTRIBUTE_MAX_THREADS_PER_MULTIPROCESSOR, dev_ordinal))

    def get_lds_per_cu(self, dev_ordinal: int = 0) -> int:
        return self.get_attribute(HIP_DEVICE_ATTRIBUTE_MAX_SHARED_MEMORY_PER_MULTIPROCESSOR, dev_ordinal)

    def get_clock_rates_khz(self, dev_ordinal: int = 0) -> Tuple[int, int]:
        """(shader clock, constant wall clock) in kHz."""
        return (self.get_attribute(HIP_DEVICE_ATTRIBUTE_CLOCK_RATE, dev_ordinal),
                self.get_attribute(HIP_DEVICE_ATTRIBUTE_WALL_CLOCK_RATE, dev_ordinal))


HIP_ERROR_NOT_SUPPORTED = 801


class HipProfiler:
    """Range gate for an external profiler (hipProfilerStart/Stop).  rocprofv3 traces the whole
    process and the tuner picks the kernel by name, so a runtime that does not implement these
    calls (ROCm 7 answers hipErrorNotSupported) changes nothing: that answer is accepted, any
    other error is raised as in the reference (RecFlex/cuda_helper.py CudaProfiler)."""

    def __init__(self):
        self._hip = _load_hip()
        self.supported = True

    def _call(self, name: str) -> None:
        ret = getattr(self._hip, name)()
        if ret == HIP_ERROR_NOT_SUPPORTED:
            self.supported = False
            self._hip.hipGetLastError()     # do not leave the refusal for the next caller to find
        elif ret != 0:
            raise Exception(f"{name}() returned {ret}")

    def start(self):
        self._call("hipProfilerStart")

    def stop(self):
        self._call("hipProfilerStop")


class HipEvent:
    """A ``hipEvent_t`` with timing enabled, for the ``start_event`` / ``stop_event`` of
    ``recom_process``: the library hands the pair to ``hipExtLaunchKernel``, which stamps them
    with the begin and end of the fused kernel's own dispatch.  ``handle`` is the raw event."""

    _hip = None

    def __init__(self):
        if HipEvent._hip is None:
            hip = _load_hip()
            hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
            hip.hipEventDestroy.argtypes = [ctypes.c_void_p]
            hip.hipEventSynchronize.argtypes = [ctypes.c_void_p]
            hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p,
                                                ctypes.c_void_p]
            hip.hipGetErrorString.restype = ctypes.c_char_p
            HipEvent._hip = hip
        ev = ctypes.c_void_p()
        self._check(self._hip.hipEventCreate(ctypes.byref(ev)), "hipEventCreate")
        self.handle = ev.value

    @classmethod
    def _check(cls, ret: int, what: str) -> None:
        if ret != HIP_SUCCESS:
            msg = cls._hip.hipGetErrorString(ret)
            raise RuntimeError(f"{what}: hipError_t {ret} ({msg.decode() if msg else '?'})")

    def synchronize(self) -> None:
        self._check(self._hip.hipEventSynchronize(self.handle), "hipEventSynchronize")

    def elapsed_us(self, later: "HipEvent") -> float:
        """Microseconds from this event to ``later`` (both must have completed)."""
        ms = ctypes.c_float()
        self._check(self._hip.hipEventElapsedTime(ctypes.byref(ms), self.handle, later.handle),
                    "hipEventElapsedTime")
        return ms.value * 1e3

    def __del__(self):
        if getattr(self, "handle", None) and self._hip is not None:
            self._hip.hipEventDestroy(self.handle)
            self.handle = None


# names of the reference module, for scripts written against it
CudaInfoQuerier = HipInfoQuerier
CudaProfiler = HipProfiler


if __name__ == "__main__":
    querier = HipInfoQuerier()
    print(querier.gpu_ids)
    print(querier.get_compute_capability())
    print(querier.get_sm_thread_count())
    print(querier.get_lds_per_cu(), querier.get_clock_rates_khz())
