"""Gather probe: time the bare fetch of the rows a batch looks up (``csrc/gather_probe.hip``).

Measurement aid for ``bench.py``: the same tables and index streams as the fused kernel, 16-byte
loads, no sums and no output, swept over the loads in flight per lane, the resident workgroups
per CU, the bytes per chunk and the XCD-segmented walk; the fastest setting is reported.  Its
time is an empirical reference -- another kernel that fetches the same rows and does nothing
else -- not a bound: the fused kernel has been faster than it on some batches.
"""

import ctypes
import os
import subprocess
from typing import List, Sequence

import numpy as np

from recflex_amd.code_emitter.build_basic import BasicBuilder

CHUNK_LOOKUPS = 1024
SWEEP_IN_FLIGHT = (4, 8)
SWEEP_WORKGROUPS_PER_CU = (4, 8)
SWEEP_SEGMENTS = (0, 16, 32)
SWEEP_CHUNK_BYTES = (16384, 65536)


AID_DIR = os.path.dirname(os.path.abspath(__file__))


def lib_path() -> str:
    return os.path.join(AID_DIR, "build", "libgather_probe.so")


def build(force: bool = False) -> str:
    basic = BasicBuilder()
    lib = lib_path()
    if force or not os.path.exists(lib):
        os.makedirs(os.path.dirname(lib), exist_ok=True)
        src = os.path.join(AID_DIR, "csrc", "gather_probe.hip")
        tmp = lib + f".tmp{os.getpid()}"
        subprocess.run([basic.hipcc, *basic.hip_flags, "-O3", src, "-o", tmp], check=True)
        os.replace(tmp, lib)
    return lib


def make_chunks(num_lookups: Sequence[int], row_vectors: Sequence[int],
                chunk_lookups: int = CHUNK_LOOKUPS, chunk_bytes: int = 0) -> np.ndarray:
    """int32 [n, 4] records (feat, begin, count, log2 of the lanes per row), ordered by feature
    like the fused kernel's tile space.  ``chunk_bytes`` > 0 sizes the chunks of every feature to
    about that many row bytes (32..4096 lookups) instead of ``chunk_lookups`` lookups."""
    out: List[tuple] = []
    for f, (n, v) in enumerate(zip(num_lookups, row_vectors)):
        log2x = min(6, max(0, int(np.ceil(np.log2(max(1, v))))))
        per = max(32, min(4096, chunk_bytes // (16 * max(1, v)))) if chunk_bytes > 0 else chunk_lookups
        out.extend((f, b, min(per, n - b), log2x) for b in range(0, n, per))
    return np.asarray(out, dtype=np.int32).reshape(-1, 4)


CALIBRATION_KERNEL = "CalibrationCopyKnl"


def calibration_copy(nbytes: int, device="cuda:0") -> None:
    """One launch of ``CalibrationCopyKnl`` copying ``nbytes`` (rounded down to 16) between two
    fresh device buffers: the dispatch of known traffic that a memory-counter run is scaled by."""
    import torch
    path = lib_path()
    if not os.path.exists(path):
        raise FileNotFoundError(f"{path} is missing: build it with benchaid.gather_probe.build()")
    lib = ctypes.CDLL(path)
    lib.calibration_copy_launch.restype = ctypes.c_int
    lib.calibration_copy_launch.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64,
                                            ctypes.c_int, ctypes.c_void_p]
    n = nbytes // 16 * 4
    src = torch.ones(n, dtype=torch.float32, device=device)
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    blocks = torch.cuda.get_device_properties(device).multi_processor_count * 8
    rc = lib.calibration_copy_launch(src.data_ptr(), dst.data_ptr(), n * 4, blocks,
                                     torch.cuda.current_stream(device).cuda_stream)
    if rc:
        raise RuntimeError(f"calibration_copy_launch: hipError_t {rc}")
    torch.cuda.synchronize()
    if not bool((dst[:: max(1, n // 1024)] == 1).all()):
        raise RuntimeError("calibration copy: destination differs from source")
    del src, dst
    torch.cuda.empty_cache()


class GatherProbe:
    def __init__(self, device, tables, d_indices, row_strides: Sequence[int]):
        import torch
        path = lib_path()
        if not os.path.exists(path):
            raise FileNotFoundError(f"{path} is missing: build it with benchaid.gather_probe.build()")
        self.lib = ctypes.CDLL(path)
        self.lib.gather_probe_launch.restype = ctypes.c_int
        self.lib.gather_probe_launch.argtypes = [ctypes.c_void_p, ctypes.c_int] + [ctypes.c_void_p] * 5 + \
                                                [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                                 ctypes.c_void_p, ctypes.c_int64]
        self.device = device
        self.tables, self.d_indices = tables, d_indices          # kept alive
        self.num_lookups = [int(i.numel()) for i in d_indices]
        # whole 16-byte vectors only: a row tail shorter than that is not read (reading it as a
        # vector would run past the end of the table's last row), a row shorter than 16 bytes
        # not at all
        self.row_vectors = [s // 16 for s in row_strides]
        self.num_lookups = [n if v else 0 for n, v in zip(self.num_lookups, self.row_vectors)]
        self.d_tables = torch.tensor([t.data_ptr() for t in tables], dtype=torch.int64, device=device)
        self.d_index_ptrs = torch.tensor([i.data_ptr() for i in d_indices], dtype=torch.int64, device=device)
        self.d_strides = torch.tensor(list(row_strides), dtype=torch.int32, device=device)
        self.d_vectors = torch.tensor(self.row_vectors, dtype=torch.int32, device=device)
        self.d_sink = torch.zeros(256, dtype=torch.float32, device=device)
        self.cus = torch.cuda.get_device_properties(device).multi_processor_count
        self.set_chunks(CHUNK_LOOKUPS)

    def set_chunks(self, chunk_lookups: int = CHUNK_LOOKUPS, chunk_bytes: int = 0) -> None:
        import torch
        chunks = make_chunks(self.num_lookups, self.row_vectors, chunk_lookups, chunk_bytes)
        self.n_chunks = len(chunks)
        self.d_chunks = torch.from_numpy(chunks).to(self.device) if len(chunks) else \
            torch.zeros((1, 4), dtype=torch.int32, device=self.device)

    def launch(self, in_flight: int = 4, workgroups_per_cu: int = 8, segments: int = 0,
               out=None) -> None:
        """``out``: a device tensor the probe also fills once (whole cache lines, spread over the
        run): the gather plus the writing of an output of that size."""
        import torch
        rc = self.lib.gather_probe_launch(self.d_chunks.data_ptr(), self.n_chunks, self.d_tables.data_ptr(),
                                          self.d_index_ptrs.data_ptr(), self.d_strides.data_ptr(),
                                          self.d_vectors.data_ptr(), self.d_sink.data_ptr(),
                                          self.cus * workgroups_per_cu, in_flight, segments,
                                          torch.cuda.current_stream(self.device).cuda_stream,
                                          out.data_ptr() if out is not None else None,
                                          out.numel() * out.element_size() if out is not None else 0)
        if rc:
            raise RuntimeError(f"gather_probe_launch: hipError_t {rc}")

    def time_us(self, steps: int = 10, warmup: int = 3, **launch_kwargs) -> float:
        """Median duration of one launch with the given setting."""
        import torch
        for _ in range(warmup):
            self.launch(**launch_kwargs)
        torch.cuda.synchronize()
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                 for _ in range(steps)]
        for s, e in pairs:
            s.record()
            self.launch(**launch_kwargs)
            e.record()
        torch.cuda.synchronize()
        d = sorted(s.elapsed_time(e) * 1e3 for s, e in pairs)
        return d[len(d) // 2]

    def best_time_us(self, steps: int = 10) -> dict:
        """Sweeps the settings; returns the fastest as {"us", "in_flight", "workgroups_per_cu",
        "segments", "chunk_bytes"}."""
        best = None
        for chunk in SWEEP_CHUNK_BYTES:
            self.set_chunks(chunk_bytes=chunk)
            for u in SWEEP_IN_FLIGHT:
                for occ in SWEEP_WORKGROUPS_PER_CU:
                    for seg in SWEEP_SEGMENTS:
                        t = self.time_us(steps=steps, in_flight=u, workgroups_per_cu=occ, segments=seg)
                        if best is None or t < best["us"]:
                            best = {"us": t, "in_flight": u, "workgroups_per_cu": occ,
                                    "segments": seg, "chunk_bytes": chunk}
        return best

    def time_with_output_us(self, setting: dict, out, steps: int = 10) -> float:
        """The probe at ``setting`` (a result of ``best_time_us``) when it also fills ``out``
        once per launch: rows fetched and an output of that size written."""
        self.set_chunks(chunk_bytes=setting["chunk_bytes"])
        return self.time_us(steps=steps, in_flight=setting["in_flight"],
                            workgroups_per_cu=setting["workgroups_per_cu"],
                            segments=setting["segments"], out=out)
