"""ctypes bindings of the CPU text front end (``recom_host_*`` in ``include/recflex_hip.h``).

``RecomHost`` stands where the reference has the generated pybind module ``recom_host``
(``RecFlex/code_emitter/codegen.py:90-218``): ``preprocess(raw_data, max_concurrent_blocks)``
takes the ``List[F][B]`` of sample lines and returns a 7-tuple in the reference's order
``(data_buffer_offsets, output_offsets, extra_buffer_offsets, task_mapping, task_tiles, data,
scala_data)``.  Differences, all consequences of the device-side thread binding:
``task_mapping`` is empty and ``task_tiles`` is zero (tiles are decided on the GPU),
``extra_buffer_offsets`` is all zero (no schedule needs scratch memory), ``data`` holds numpy
int32 arrays ``[offsets_0, indices_0, offsets_1, indices_1, ...]`` instead of Python lists, and
inside the packed buffer a feature's offsets come first, then its indices.
"""

import ctypes
import os
from typing import List, Sequence, Tuple

import numpy as np

_I32P = ctypes.POINTER(ctypes.c_int32)
_I64P = ctypes.POINTER(ctypes.c_int64)

_ERRORS = {-1: "invalid argument", -2: "output capacity too small",
           -3: "text holds a different number of lines than expected",
           -4: "index does not fit in int32"}


class RecomHostError(RuntimeError):
    pass


def _declare(lib: ctypes.CDLL) -> None:
    lib.recom_host_parse_lines.restype = ctypes.c_int
    lib.recom_host_parse_lines.argtypes = [ctypes.c_char_p, ctypes.c_int64, ctypes.c_int32, _I32P,
                                           ctypes.c_int64, _I32P, _I64P]
    lib.recom_host_max_indices.restype = ctypes.c_int64
    lib.recom_host_max_indices.argtypes = [ctypes.c_int64]
    lib.recom_host_alignmem.restype = ctypes.c_int64
    lib.recom_host_alignmem.argtypes = [ctypes.c_int64]
    lib.recom_host_packed_size.restype = ctypes.c_int64
    lib.recom_host_packed_size.argtypes = [ctypes.c_int32, ctypes.c_int64]
    lib.recom_host_pack.restype = ctypes.c_int
    lib.recom_host_pack.argtypes = [ctypes.c_int32, ctypes.c_int32, ctypes.POINTER(_I32P),
                                    ctypes.POINTER(_I32P), _I64P, ctypes.c_void_p, ctypes.c_int64, _I64P]


def default_host_lib_path() -> str:
    from recflex_amd.code_emitter.build_basic import BasicBuilder
    return BasicBuilder().host_lib_path()


class RecomHost:
    """Loads ``librecflex_host.so`` (model independent) or a generated ``recom_host.so``
    (which also knows the model's feature count)."""

    def __init__(self, path: str = None):
        self.path = path or default_host_lib_path()
        if not os.path.exists(self.path):
            raise FileNotFoundError(
                f"{self.path} is not built; run recflex_amd.code_emitter.build_basic.BasicBuilder().build()")
        self.lib = ctypes.CDLL(self.path)
        _declare(self.lib)
        self.num_features = None
        if hasattr(self.lib, "recom_host_num_features"):
            self.lib.recom_host_num_features.restype = ctypes.c_int32
            self.num_features = int(self.lib.recom_host_num_features())
        self._knows_dims = hasattr(self.lib, "recom_host_output_row_bytes")
        if self._knows_dims:
            self.lib.recom_host_output_row_bytes.restype = ctypes.c_int64
            self.lib.recom_host_output_row_bytes.argtypes = [ctypes.c_int32]

    # -------------------------------------------------------------------------------------

    def parse_lines(self, lines: Sequence[str]) -> Tuple[np.ndarray, np.ndarray]:
        """Sample lines of one feature -> (indices int32[L], offsets int32[B+1])."""
        text = "\n".join(lines).encode()
        n_lines = len(lines)
        cap = int(self.lib.recom_host_max_indices(len(text)))
        indices = np.empty(max(cap, 1), dtype=np.int32)
        offsets = np.empty(n_lines + 1, dtype=np.int32)
        n = ctypes.c_int64(0)
        rc = self.lib.recom_host_parse_lines(text, len(text), n_lines,
                                             indices.ctypes.data_as(_I32P), cap,
                                             offsets.ctypes.data_as(_I32P), ctypes.byref(n))
        if rc != 0:
            raise RecomHostError(f"recom_host_parse_lines: {_ERRORS.get(rc, rc)}")
        return indices[:n.value].copy(), offsets

    def alignmem(self, nbytes: int) -> int:
        return int(self.lib.recom_host_alignmem(nbytes))

    def pack(self, offsets: List[np.ndarray], indices: List[np.ndarray]) -> Tuple[np.ndarray, np.ndarray]:
        """Per-feature arrays -> (packed int32 buffer, int64 byte offsets [F+1])."""
        num_feats = len(offsets)
        assert len(indices) == num_feats
        if num_feats == 0:
            return np.zeros(0, dtype=np.int32), np.zeros(1, dtype=np.int64)
        batch = len(offsets[0]) - 1
        offs = [np.ascontiguousarray(o, dtype=np.int32) for o in offsets]
        idxs = [np.ascontiguousarray(i, dtype=np.int32) for i in indices]
        for o in offs:
            if len(o) != batch + 1:
                raise ValueError("all features must have the same batch size")
        counts = np.array([len(i) for i in idxs], dtype=np.int64)
        total = sum(int(self.lib.recom_host_packed_size(batch, int(c))) for c in counts)
        dst = np.empty(total // 4, dtype=np.int32)
        byte_offsets = np.zeros(num_feats + 1, dtype=np.int64)
        off_ptrs = (_I32P * num_feats)(*[o.ctypes.data_as(_I32P) for o in offs])
        idx_ptrs = (_I32P * num_feats)(*[i.ctypes.data_as(_I32P) for i in idxs])
        rc = self.lib.recom_host_pack(num_feats, batch, off_ptrs, idx_ptrs,
                                      counts.ctypes.data_as(_I64P), dst.ctypes.data_as(ctypes.c_void_p),
                                      total, byte_offsets.ctypes.data_as(_I64P))
        if rc != 0:
            raise RecomHostError(f"recom_host_pack: {_ERRORS.get(rc, rc)}")
        return dst, byte_offsets

    # -------------------------------------------------------------------------------------

    def preprocess(self, raw_data: List[List[str]], max_concurrent_blocks: int = 0):
        num_feats = len(raw_data)
        if self.num_features is not None and num_feats != self.num_features:
            raise ValueError(f"this host library was generated for {self.num_features} features, "
                             f"got {num_feats}")
        data: List[np.ndarray] = []
        scala_data: List[int] = []
        offsets, indices = [], []
        for lines in raw_data:
            idx, off = self.parse_lines(lines)
            offsets.append(off)
            indices.append(idx)
            data.extend([off, idx])
            scala_data.extend([len(idx), len(off) - 1])   # num_inputs, num_segments
        self.packed, byte_offsets = self.pack(offsets, indices)
        data_buffer_offsets = byte_offsets.tolist()
        # byte offsets of each feature's slab of pooled output (prefix sum of batch * dim * 4,
        # reference: codegen.py:144-147); the generic library does not know the dims and
        # reports zeros, FeatPreprocess then sizes the output from the model's dims
        output_offsets = [0]
        for f, o in enumerate(offsets):
            row_bytes = int(self.lib.recom_host_output_row_bytes(f)) if self._knows_dims else 0
            output_offsets.append(output_offsets[-1] + (len(o) - 1) * row_bytes)
        extra_buffer_offsets = [0] * (num_feats + 1)
        task_mapping: List[Tuple[int, int]] = []
        task_tiles = [0] * num_feats
        return (data_buffer_offsets, output_offsets, extra_buffer_offsets, task_mapping,
                task_tiles, data, scala_data)
