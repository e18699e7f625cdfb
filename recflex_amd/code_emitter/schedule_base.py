"""Interface between the fused-kernel emitter and the per-feature schedule templates.

Mirrors ``RecFlex/code_emitter/schedule_base.py:17-87`` (``InputStats``, ``MetaData``,
``ScheduleVars``, ``PreprocessVars``, ``ScheduleBase`` and its method names) so that schedule
templates written against the reference interface keep their shape.  What differs is what the
emitted strings talk to: a schedule body here is HIP for gfx950 that sums the bags
``[bag_begin, bag_end)`` of one feature, given the feature's int32 ``indices`` / ``offsets``
arrays, instead of CUDA that decodes a packed argument buffer for block ``task_bid``.
"""

from abc import ABC, abstractmethod
from typing import List, NamedTuple, Tuple


# Schedules that split a bag over several workgroups: the granularity by which such a schedule
# announces itself to the run-time binding (rfx::kSplitGran) and the slots of a feature's
# workspace region (rfx::kBindMaxSplitTiles)
SPLIT_GRANULARITY = -1
SPLIT_MAX_TILES = 2048


class InputStats(NamedTuple):
    # field names as in the reference (including the spelling of ``minmum``)
    mean: float
    var: float
    maximum: float
    minmum: float


_DTYPE_IDS = {"float": 0, "half": 1, "int8": 2}
_DTYPE_ALIASES = {
    "float": "float", "float32": "float", "fp32": "float", "f32": "float",
    "half": "half", "float16": "half", "fp16": "half", "f16": "half",
    "int8": "int8", "i8": "int8", "uint8": "int8", "u8": "int8",
}


def canonical_data_type(name: str) -> str:
    try:
        return _DTYPE_ALIASES[name.strip().lower()]
    except KeyError:
        raise ValueError(f"unknown table data type {name!r}; expected one of {sorted(_DTYPE_ALIASES)}")


class MetaData(NamedTuple):
    """Static description of one feature's table (reference: schedule_base.py:23-25).

    ``data_type`` is ``"float"`` (fp32 rows), ``"half"`` (fp16 rows, fp32 accumulate) or
    ``"int8"`` (row = ``embed_dim`` unsigned 8-bit codes, fp16 scale, fp16 bias, row stride
    rounded up to 16 bytes; value = code * scale + bias).
    """
    embed_dim: int
    data_type: str = "float"

    @property
    def dtype_id(self) -> int:
        return _DTYPE_IDS[canonical_data_type(self.data_type)]

    @property
    def elem_bytes(self) -> int:
        return (4, 2, 1)[self.dtype_id]

    @property
    def payload_bytes(self) -> int:
        return self.embed_dim * self.elem_bytes

    @property
    def row_stride(self) -> int:
        """Bytes between consecutive table rows."""
        if self.dtype_id == 2:
            return (self.payload_bytes + 4 + 15) // 16 * 16
        return self.payload_bytes

    @property
    def row_bytes(self) -> int:
        """Algorithmic bytes fetched per lookup (payload, plus scale and bias for int8)."""
        return self.payload_bytes + (4 if self.dtype_id == 2 else 0)

    @property
    def vec_bytes(self) -> int:
        """Bytes one lane moves per load: the widest of 16/8/4 dividing the payload."""
        p = self.payload_bytes
        if p % 4 != 0:
            raise ValueError(f"row payload of {p} bytes (dim {self.embed_dim}, {self.data_type}) "
                             "is not a whole number of 4-byte words")
        return 16 if p % 16 == 0 else (8 if p % 8 == 0 else 4)

    @property
    def row_vectors(self) -> int:
        return self.payload_bytes // self.vec_bytes

    @property
    def elems_per_vector(self) -> int:
        return self.vec_bytes // self.elem_bytes


class ScheduleVars(NamedTuple):
    """Names visible inside an emitted schedule body (reference: schedule_base.py:28-40)."""
    embed_table: str = "d_embed_table"       # const char *, base of this feature's table
    shmem: str = "s"                         # char *, the workgroup's LDS union
    stage: str = "stage"                     # rfx::f32x4 *, LDS staging of team outputs (or null)
    indices: str = "d_indices"               # const int *, this feature's lookups
    offsets: str = "d_offsets"               # const int *, [batch + 1]
    output: str = "d_output"                 # float *, [batch, EMBED_DIM_SUM]
    embed_dim_offset: str = "embed_dim_offset"
    EMBED_DIM_SUM: str = "EMBED_DIM_SUM"
    out_row_stride: str = "out_row_stride"   # floats between output rows (EMBED_DIM_SUM if dense)
    BLOCK_THREADS: str = "BLOCK_THREADS"
    bag_begin: str = "bag_begin"             # this tile sums bags [bag_begin, bag_end)
    bag_end: str = "bag_end"
    out_vec: str = "OUT_VEC"                 # widest aligned output store in floats (4, 2 or 1)
    # schedules that split a bag over workgroups: this tile is part split_part of split_parts of
    # bag bag_begin (split_parts <= 1: a plain bag range); split_region = the feature's floats
    # of the caller's workspace (null if no schedule of the feature splits)
    # int: bags of more lookups than this were found ahead of the kernel and run as tiles of
    # their own, the body must leave them alone (INT_MAX when there are none)
    skip_long: str = "skip_longer_than"
    # int: 1 if this batch holds exactly as many lookups of the feature as bags (every bag may
    # have exactly one lookup; a body for such bags can fetch indices[bag] ahead of the bag's
    # offsets and check afterwards), else 0
    one_per_bag: str = "one_per_bag"
    split_part: str = "split_part"
    split_parts: str = "split_parts"
    split_region: str = "split_region"
    # rfx::MidBagQueue * (null in a build without outlier tiles): where a team leaves a bag
    # beyond its schedule's reach for whichever wavefront of the workgroup has time, under the
    # feature's number feat_id
    mid_queue: str = "mid_queue"
    feat_id: str = "feat_id"


class PreprocessVars(NamedTuple):
    """Names visible inside an emitted host preprocess snippet (reference: schedule_base.py:43-51)."""
    raw_data: str = "raw_data"
    raw_data_len: str = "raw_data_len"
    num_lines: str = "num_lines"
    indices: str = "indices"
    indices_capacity: str = "indices_capacity"
    offsets: str = "offsets"
    num_inputs_ref: str = "num_inputs_ref"


class ScheduleBase(ABC):
    def __init__(self, meta_data: MetaData, block_threads: int):
        self.meta: MetaData = meta_data
        self.block_threads = block_threads
        self.sched_vars: ScheduleVars = ScheduleVars()
        self.pre_vars: PreprocessVars = PreprocessVars()

    @abstractmethod
    def EmitScheduleBody(self, params: NamedTuple) -> str:
        pass

    @abstractmethod
    def EmitShmemType(self, params: NamedTuple) -> str:
        pass

    def NeedsOutputStage(self, params: NamedTuple) -> bool:
        """True if the body writes through the kernel's ``rfx::TeamStage`` LDS buffer."""
        return False

    @abstractmethod
    def TileGranularity(self, params: NamedTuple) -> int:
        """Bags one workgroup of this schedule covers per pass; tiles are multiples of it."""

    def LongBagThreshold(self, params: NamedTuple) -> int:
        """Bags of more lookups than this are outliers for the schedule.  A library emitted with
        ``outliers=True`` gives those of them that carry at least a tile's traffic to several
        workgroups and tells the body which to skip (``skip_long``).  0: the schedule takes bags
        of any length and ignores that."""
        return 0

    def WorkspaceFloats(self, params: NamedTuple) -> int:
        """Floats of the caller's workspace this schedule needs for its feature (0 = none).  A
        schedule that needs some must return the split granularity from ``TileGranularity``."""
        return 0

    @abstractmethod
    def GenParamCandidates(self, stats: InputStats = None) -> List:
        pass

    def UsedArgCounts(self) -> Tuple[int, int]:
        # data vectors: offsets, indices; scalars: num_inputs, num_segments
        # (same counts as the reference's bag schedules, warp_per_sample.py:78-81)
        return 2, 2

    def EmitHostPreprocess(self, params: NamedTuple) -> str:
        """All schedules read the same (indices, offsets) form, so one host snippet serves all."""
        v = self.pre_vars
        return (f"  return recom_host_parse_lines({v.raw_data}, {v.raw_data_len}, {v.num_lines},\n"
                f"                                {v.indices}, {v.indices_capacity}, {v.offsets},\n"
                f"                                {v.num_inputs_ref});\n")

    def EmitHeaders(self) -> List[str]:
        return ['"rfx_schedules.hip.h"']

    def EmitPrepropHeaders(self) -> List[str]:
        return ['"recflex_hip.h"']
