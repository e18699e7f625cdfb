"""ctypes bindings of a generated ``librecom.so`` (``recom_*`` in ``include/recflex_hip.h``).

Stands where the reference calls ``torch.ops.load_library(librecom_path)`` and
``torch.ops.recom.{process,get_max_concurrent_blocks,get_gpu_pointers_array}``
(``RecFlex/rec_modules.py:71-72,82-94``).  Each ``RecomLib`` owns its own ``dlopen`` handle, so
any number of emitted kernels can be used in one process.
"""

import ctypes
import os
from typing import List

_I32P = ctypes.POINTER(ctypes.c_int32)


class RecomInfo(ctypes.Structure):
    _fields_ = [
        ("abi_version", ctypes.c_int32),
        ("num_features", ctypes.c_int32),
        ("embed_dim_sum", ctypes.c_int32),
        ("block_threads", ctypes.c_int32),
        ("occupancy", ctypes.c_int32),
        ("num_bodies", ctypes.c_int32),
        ("timing", ctypes.c_int32),
        ("tile_bytes", ctypes.c_int32),
        ("static_binding", ctypes.c_int32),
        ("num_candidates", ctypes.c_int32),
        ("xcd_segments", ctypes.c_int32),
        ("outliers", ctypes.c_int32),
        ("static_workspace", ctypes.c_int32),
        ("reserved", ctypes.c_int32 * 3),
    ]


class RecomLaunchInfo(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in (
        "compute_units", "occupancy", "dyn_lds_bytes", "natural_occupancy", "api_occupancy",
        "num_vgprs", "static_lds_bytes", "lds_bytes_per_cu", "padded_api_occupancy")] + \
        [("reserved", ctypes.c_int32 * 3)]

    def as_dict(self):
        return {n: getattr(self, n) for n, _ in self._fields_ if n != "reserved"}


class RecomProcessArgs(ctypes.Structure):
    _fields_ = [
        ("d_embed_table_ptrs", ctypes.c_void_p),
        ("d_io_ptrs", ctypes.c_void_p),
        ("d_arg_buffers", ctypes.c_void_p),
        ("d_arg_buffer_offsets", ctypes.c_void_p),
        ("d_output", ctypes.c_void_p),
        ("batch", ctypes.c_int32),
        ("tile_bytes", ctypes.c_int32),
        ("grid_blocks", ctypes.c_int32),
        ("xcd_segments", ctypes.c_int32),
        ("d_schedule_choice", ctypes.c_void_p),
        ("d_times", ctypes.c_void_p),
        ("stream", ctypes.c_void_p),
        ("output_row_stride", ctypes.c_int64),
        ("d_workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_int64),
        ("start_event", ctypes.c_void_p),
        ("stop_event", ctypes.c_void_p),
        ("d_lookup_counts", ctypes.c_void_p),
    ]


RECOM_ABI_VERSION = 6
RECOM_STATIC_WORKSPACE_MAX_BYTES = 32 * 1024 * 1024
RECOM_ESTATIC_WORKSPACE = -5
EXPORTED_SYMBOLS = ("recom_get_info", "recom_get_feature_tables", "recom_get_candidate_counts",
                    "recom_get_launch_info", "recom_get_workspace_bytes",
                    "recom_get_max_concurrent_blocks", "recom_process",
                    "recom_process_static_workspace")


class RecomError(RuntimeError):
    def __init__(self, func: str, code: int):
        super().__init__(f"{func} failed with hipError_t {code}")
        self.code = code


class RecomLib:
    def __init__(self, path: str):
        if not os.path.exists(path):
            raise FileNotFoundError(f"{path} does not exist; build it first (the HIP library is "
                                    "required, there is no fallback path)")
        self.path = os.path.abspath(path)
        self.lib = ctypes.CDLL(self.path)
        for name in EXPORTED_SYMBOLS:
            if not hasattr(self.lib, name):
                raise RecomError(f"{path}: missing symbol {name}", -1)
        self.lib.recom_get_info.restype = ctypes.c_int
        self.lib.recom_get_info.argtypes = [ctypes.POINTER(RecomInfo)]
        self.lib.recom_get_feature_tables.restype = ctypes.c_int
        self.lib.recom_get_feature_tables.argtypes = [_I32P, _I32P, _I32P, _I32P]
        self.lib.recom_get_max_concurrent_blocks.restype = ctypes.c_int
        self.lib.recom_get_max_concurrent_blocks.argtypes = [_I32P]
        self.lib.recom_process.restype = ctypes.c_int
        self.lib.recom_process.argtypes = [ctypes.POINTER(RecomProcessArgs)]
        self.lib.recom_process_static_workspace.restype = ctypes.c_int
        self.lib.recom_process_static_workspace.argtypes = [ctypes.POINTER(RecomProcessArgs)]

        self.info = RecomInfo()
        rc = self.lib.recom_get_info(ctypes.byref(self.info))
        if rc != 0:
            raise RecomError("recom_get_info", rc)
        if self.info.abi_version != RECOM_ABI_VERSION:
            raise RecomError(f"{path}: ABI version {self.info.abi_version} != {RECOM_ABI_VERSION}", -1)
        f = self.info.num_features
        arrs = [(ctypes.c_int32 * f)() for _ in range(4)]
        rc = self.lib.recom_get_feature_tables(*arrs)
        if rc != 0:
            raise RecomError("recom_get_feature_tables", rc)
        self.embed_dims: List[int] = list(arrs[0])
        self.embed_dim_offsets: List[int] = list(arrs[1])
        self.dtypes: List[int] = list(arrs[2])
        self.row_strides: List[int] = list(arrs[3])
        self.lib.recom_get_candidate_counts.restype = ctypes.c_int
        self.lib.recom_get_candidate_counts.argtypes = [_I32P]
        counts = (ctypes.c_int32 * f)()
        rc = self.lib.recom_get_candidate_counts(counts)
        if rc != 0:
            raise RecomError("recom_get_candidate_counts", rc)
        self.candidate_counts: List[int] = list(counts)
        self.lib.recom_get_workspace_bytes.restype = ctypes.c_int
        self.lib.recom_get_workspace_bytes.argtypes = [ctypes.POINTER(ctypes.c_int64)]
        nbytes = ctypes.c_int64(0)
        rc = self.lib.recom_get_workspace_bytes(ctypes.byref(nbytes))
        if rc != 0:
            raise RecomError("recom_get_workspace_bytes", rc)
        self.workspace_bytes: int = nbytes.value
        self._workspaces = {}

    @property
    def num_features(self) -> int:
        return self.info.num_features

    @property
    def embed_dim_sum(self) -> int:
        return self.info.embed_dim_sum

    def get_launch_info(self) -> RecomLaunchInfo:
        out = RecomLaunchInfo()
        self.lib.recom_get_launch_info.restype = ctypes.c_int
        self.lib.recom_get_launch_info.argtypes = [ctypes.POINTER(RecomLaunchInfo)]
        rc = self.lib.recom_get_launch_info(ctypes.byref(out))
        if rc != 0:
            raise RecomError("recom_get_launch_info", rc)
        return out

    def get_max_concurrent_blocks(self) -> int:
        out = ctypes.c_int32(0)
        rc = self.lib.recom_get_max_concurrent_blocks(ctypes.byref(out))
        if rc != 0:
            raise RecomError("recom_get_max_concurrent_blocks", rc)
        return out.value

    def default_workspace(self) -> int:
        """Address of a zeroed workspace of ``workspace_bytes`` on the current device, allocated
        on first use and kept for the life of this handle (0 if the library needs none).
        Launches of this handle that may overlap on different streams must not share it: pass
        ``workspace=`` to ``process`` for those."""
        if self.workspace_bytes == 0:
            return 0
        import torch
        dev = torch.cuda.current_device()
        if dev not in self._workspaces:
            self._workspaces[dev] = torch.zeros((self.workspace_bytes + 3) // 4, dtype=torch.int32,
                                                device=torch.device("cuda", dev))
            torch.cuda.current_stream().synchronize()
        return self._workspaces[dev].data_ptr()

    def process(self, table_ptrs: int, output: int, batch: int, *, io_ptrs: int = 0,
                arg_buffers: int = 0, arg_buffer_offsets: int = 0, tile_bytes: int = 0,
                grid_blocks: int = 0, xcd_segments: int = 0, schedule_choice: int = 0,
                times: int = 0, stream: int = 0, output_row_stride: int = 0,
                workspace: int = 0, workspace_bytes: int = 0,
                static_workspace: bool = False, start_event: int = 0, stop_event: int = 0,
                lookup_counts: int = 0) -> None:
        """All pointer arguments are raw device addresses (``tensor.data_ptr()``).  Without a
        ``workspace``, a library that needs one uses ``default_workspace()``.
        ``start_event`` / ``stop_event``: ``hipEvent_t`` handles that receive the begin and end of
        the fused kernel's own dispatch.
        ``lookup_counts``: device int32[F], the lookups of each feature in this batch as far as
        the caller knows (a hint that spares the binding a scattered read per feature).
        ``static_workspace=True`` calls ``recom_process_static_workspace`` instead: no workspace
        is passed or allocated, the library uses its own static device array."""
        if static_workspace:
            args = RecomProcessArgs(table_ptrs or None, io_ptrs or None, arg_buffers or None,
                                    arg_buffer_offsets or None, output or None, batch, tile_bytes,
                                    grid_blocks, xcd_segments, schedule_choice or None,
                                    times or None, stream or None, output_row_stride, None, 0,
                                    start_event or None, stop_event or None, lookup_counts or None)
            rc = self.lib.recom_process_static_workspace(ctypes.byref(args))
            if rc == RECOM_ESTATIC_WORKSPACE:
                raise RecomError(f"recom_process_static_workspace: the library needs "
                                 f"{self.workspace_bytes} bytes of workspace, its static array holds "
                                 f"at most {RECOM_STATIC_WORKSPACE_MAX_BYTES};", rc)
            if rc != 0:
                raise RecomError("recom_process_static_workspace", rc)
            return
        if not workspace and self.workspace_bytes:
            workspace, workspace_bytes = self.default_workspace(), self.workspace_bytes
        args = RecomProcessArgs(table_ptrs or None, io_ptrs or None, arg_buffers or None,
                                arg_buffer_offsets or None, output or None, batch, tile_bytes,
                                grid_blocks, xcd_segments, schedule_choice or None, times or None,
                                stream or None, output_row_stride, workspace or None,
                                workspace_bytes, start_event or None, stop_event or None,
                                lookup_counts or None)
        rc = self.lib.recom_process(ctypes.byref(args))
        if rc != 0:
            raise RecomError("recom_process", rc)
