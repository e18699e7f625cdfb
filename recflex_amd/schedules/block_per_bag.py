"""Block-per-bag and split-bag schedule templates.

``BlockPerBagSchedule`` emits a call to ``rfx::block_bags``
(``csrc/include/rfx_schedules.hip.h``): the whole workgroup sums one bag at a time, the bag's
indices are staged in LDS with coalesced loads, the lookup lanes of a wavefront are combined
with the cross-lane butterfly and the wavefronts through LDS.

``SplitBagSchedule`` emits ``rfx::split_bags``: when a batch holds few, very long bags -- the
mean bag carries more than a tile's traffic and the feature has at most 2048 / parts bags --
the run-time binding gives every bag ``parts`` workgroups; each sums its share like
``block_bags``, leaves its partial sums in the caller's workspace and the one that finishes
last adds them in part order and writes the output.  On any other batch it is ``block_bags``.
It has the role of the reference's schedules for long or skewed bags,
``MultiBlockPerSampleSchedule`` (examples/schedules/multi_block_per_sample.py) and
``ReduceByKeySchedule`` (examples/schedules/reduce_by_key.py), without their atomics onto an
uninitialised output, with a fixed summation order, and without a workgroup ever waiting for
another one.
"""

from typing import List, NamedTuple

from recflex_amd.code_emitter.schedule_base import (ScheduleBase, InputStats, SPLIT_GRANULARITY,
                                                    SPLIT_MAX_TILES)
from .team import next_pow2, _pow2_upto, MAX_ACC_FLOATS, MAX_INFLIGHT_DWORDS


class BlockPerBagParams(NamedTuple):
    lanes_x: int            # column lanes (<= 64); block_threads / lanes_x lookup lanes
    items_per_thread: int   # lookups in flight per lane
    chunk: int              # indices staged in LDS at a time (multiple of block_threads)


class BlockPerBagSchedule(ScheduleBase):
    def _check(self, p: BlockPerBagParams) -> None:
        if p.lanes_x < 1 or p.lanes_x > 64 or p.lanes_x & (p.lanes_x - 1):
            raise ValueError(f"lanes_x={p.lanes_x} must be a power of two <= 64")
        if self.block_threads % 64:
            raise ValueError("block_threads must hold whole wavefronts")
        if p.chunk < self.block_threads or p.chunk % self.block_threads:
            raise ValueError(f"chunk={p.chunk} must be a multiple of block_threads={self.block_threads}")
        if p.items_per_thread < 1:
            raise ValueError("items_per_thread must be >= 1")

    def _storage(self, p: BlockPerBagParams) -> str:
        m = self.meta
        return (f"rfx::BlockBagStorage<{self.sched_vars.BLOCK_THREADS}, {m.dtype_id}, {m.embed_dim}, "
                f"{p.lanes_x}, {p.chunk}>")

    def EmitScheduleBody(self, params: BlockPerBagParams) -> str:
        self._check(params)
        v = self.sched_vars
        m = self.meta
        return f'''
  rfx::block_bags<{v.BLOCK_THREADS}, {m.dtype_id}, {m.embed_dim}, {params.lanes_x},
                  {params.items_per_thread}, {params.chunk}>(
      *reinterpret_cast<{self._storage(params)} *>({v.shmem}),
      {v.embed_table}, {v.indices}, {v.offsets}, {v.output},
      {v.out_row_stride}, {v.embed_dim_offset}, {v.bag_begin}, {v.bag_end});
'''

    def EmitShmemType(self, params: BlockPerBagParams) -> str:
        self._check(params)
        return self._storage(params)

    def TileGranularity(self, params: BlockPerBagParams) -> int:
        return 1

    def GenParamCandidates(self, stats: InputStats = None) -> List[BlockPerBagParams]:
        m = self.meta
        out = []
        vmax = next_pow2(m.row_vectors)
        for x in _pow2_upto(min(64, vmax)):
            vpl = -(-m.row_vectors // x)
            if vpl > 4 or vpl * m.elems_per_vector > MAX_ACC_FLOATS:
                continue
            if x * 4 < min(64, vmax):   # keep to the widest few column splits
                continue
            for items in (1, 2, 4):
                if items * vpl * m.vec_bytes // 4 > MAX_INFLIGHT_DWORDS:
                    continue
                out.append(BlockPerBagParams(x, items, 4 * self.block_threads))
        return out


class SplitBagSchedule(BlockPerBagSchedule):
    def EmitScheduleBody(self, params: BlockPerBagParams) -> str:
        self._check(params)
        v = self.sched_vars
        m = self.meta
        return f'''
  rfx::split_bags<{v.BLOCK_THREADS}, {m.dtype_id}, {m.embed_dim}, {params.lanes_x},
                  {params.items_per_thread}, {params.chunk}>(
      *reinterpret_cast<{self._storage(params)} *>({v.shmem}),
      {v.embed_table}, {v.indices}, {v.offsets}, {v.output},
      {v.out_row_stride}, {v.embed_dim_offset}, {v.bag_begin}, {v.bag_end},
      {v.split_part}, {v.split_parts}, {v.split_region});
'''

    def TileGranularity(self, params: BlockPerBagParams) -> int:
        return SPLIT_GRANULARITY

    def WorkspaceFloats(self, params: BlockPerBagParams) -> int:
        return SPLIT_MAX_TILES * (self.meta.embed_dim + 1)
