"""The six schedule class names of the reference, so that its ``schedule_config.txt`` files
(e.g. examples/models/test/schedule_config.txt:1-6 of the reference) resolve unchanged.

Each name keeps the role it has in the reference and draws its candidates from the gfx950
templates:

=============================  ==========================================================
``OneHotSchedule``             bags of one lookup: the row-copy template (``OneHotBagSchedule``),
                               no lookup lanes, several bags in flight per team
``OneHotMultiBlockSchedule``   same (the reference variant differs only in its block count,
                               which the run-time binding decides here)
``WarpPerSampleSchedule``      X column lanes, serial lookups, no cross-lane reduction
``OneBlockMultiSampleSchedule``X x Y lanes with a cross-lane reduction over Y
``MultiBlockPerSampleSchedule``split-bag: several workgroups per bag when a batch holds few,
                               very long bags, block-per-bag otherwise
``ReduceByKeySchedule``        split-bag
=============================  ==========================================================
"""

from typing import List

from recflex_amd.code_emitter.schedule_base import InputStats
from .team import (TeamScheduleBase, TeamParams, fits_registers, next_pow2, _pow2_upto,
                   passes_for, MAX_ACC_FLOATS, OneHotBagSchedule, OneHotBagParams)
from .block_per_bag import SplitBagSchedule, BlockPerBagParams


def _vpp(meta, vpl: int) -> int:
    return vpl if vpl * meta.elems_per_vector <= MAX_ACC_FLOATS else passes_for(vpl, meta)[-1]


class _GenericTeam(TeamScheduleBase):
    def team_params(self, params: TeamParams) -> TeamParams:
        return TeamParams(*params)


class OneHotSchedule(OneHotBagSchedule):
    pass


class OneHotMultiBlockSchedule(OneHotBagSchedule):
    pass


class WarpPerSampleSchedule(_GenericTeam):
    def GenParamCandidates(self, stats: InputStats = None) -> List[TeamParams]:
        m = self.meta
        out = []
        for x in _pow2_upto(min(64, next_pow2(m.row_vectors))):
            vpl = -(-m.row_vectors // x)
            if vpl > 8:
                continue
            for items in (1, 2, 4, 8):
                p = TeamParams(x, 1, items, 1, _vpp(m, vpl))
                if fits_registers(m, p):
                    out.append(p)
        return out


class OneBlockMultiSampleSchedule(_GenericTeam):
    def GenParamCandidates(self, stats: InputStats = None) -> List[TeamParams]:
        m = self.meta
        out = []
        for x in _pow2_upto(min(32, next_pow2(m.row_vectors))):
            vpl = -(-m.row_vectors // x)
            if vpl > 4:
                continue
            for y in (2, 4, 8, 16, 32, 64):
                if x * y > 64:
                    continue
                for items in (1, 2, 4, 8):
                    p = TeamParams(x, y, items, 1, _vpp(m, vpl))
                    if fits_registers(m, p):
                        out.append(p)
        return out


class MultiBlockPerSampleSchedule(SplitBagSchedule):
    pass


class ReduceByKeySchedule(SplitBagSchedule):
    pass


# parameter tuple names of the reference, for scripts that import them
OneHotParams = OneHotBagParams
OneHotMultiBlockParams = OneHotBagParams
WarpPerSampleParams = TeamParams
OneBlockMultiSampleParams = TeamParams
MultiBlockPerSampleParams = BlockPerBagParams
ReduceByKeyParams = BlockPerBagParams
