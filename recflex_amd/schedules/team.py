"""Thread-, sub-wavefront- and wavefront-per-bag schedule templates for 64-lane wavefronts.

All three emit a call to ``rfx::team_bags`` (``csrc/include/rfx_schedules.hip.h``): a bag is
summed by a team of ``X * Y`` lanes, ``X`` lanes across the row's 16-byte vectors and ``Y``
lanes across the bag's lookups (combined with a DPP / ds_swizzle / permlane butterfly).

Reference counterparts: ``WarpPerSampleSchedule`` (examples/schedules/warp_per_sample.py:24-113,
X lanes x serial lookups), ``OneBlockMultiSampleSchedule``
(examples/schedules/one_block_multi_sample.py:25-125, X x Y lanes with a shared-memory tree) and
``OneHotSchedule`` (examples/schedules/one_hot.py:22-92, bags of exactly one lookup).
"""

from typing import List, NamedTuple

from recflex_amd.code_emitter.schedule_base import ScheduleBase, InputStats, MetaData

# dwords of row data a lane may hold in flight (U * UB * VPP * vec_bytes / 4) and accumulator
# floats per lane (UB * VPP * elems_per_vector); keeps candidates inside the VGPR budget of
# four or more wavefronts per SIMD
MAX_INFLIGHT_DWORDS = 64
MAX_ACC_FLOATS = 64


def next_pow2(n: int) -> int:
    p = 1
    while p < n:
        p *= 2
    return p


def _pow2_upto(n: int) -> List[int]:
    out, p = [], 1
    while p <= n:
        out.append(p)
        p *= 2
    return out


class TeamParams(NamedTuple):
    """lanes_x * lanes_y lanes per bag; items_per_thread lookups x bags_per_team bags x
    vectors_per_pass row vectors in flight per lane."""
    lanes_x: int
    lanes_y: int
    items_per_thread: int
    bags_per_team: int
    vectors_per_pass: int


class ThreadPerBagParams(NamedTuple):
    items_per_thread: int
    bags_per_thread: int
    vectors_per_pass: int


class SubWavefrontPerBagParams(NamedTuple):
    lanes_x: int
    lanes_y: int
    items_per_thread: int
    bags_per_team: int
    vectors_per_pass: int


class WavefrontPerBagParams(NamedTuple):
    lanes_x: int
    items_per_thread: int
    vectors_per_pass: int


def fits_registers(meta: MetaData, p: TeamParams) -> bool:
    dwords = p.items_per_thread * p.bags_per_team * p.vectors_per_pass * meta.vec_bytes // 4
    accs = p.bags_per_team * p.vectors_per_pass * meta.elems_per_vector
    return dwords <= MAX_INFLIGHT_DWORDS and accs <= MAX_ACC_FLOATS


def passes_for(vpl: int, meta: MetaData) -> List[int]:
    """Choices of vectors-per-pass for a lane that owns ``vpl`` row vectors."""
    out = []
    for vpp in _pow2_upto(vpl):
        if vpl % vpp == 0 and vpp * meta.elems_per_vector <= MAX_ACC_FLOATS:
            out.append(vpp)
    if vpl not in out and vpl * meta.elems_per_vector <= MAX_ACC_FLOATS:
        out.append(vpl)
    return out or [1]


class TeamScheduleBase(ScheduleBase):
    """Common emission for every team size up to one wavefront."""

    def team_params(self, params: NamedTuple) -> TeamParams:
        raise NotImplementedError

    def _check(self, p: TeamParams) -> None:
        team = p.lanes_x * p.lanes_y
        if team < 1 or team > 64 or team & (team - 1):
            raise ValueError(f"team of {team} lanes is not a power of two <= 64")
        if self.block_threads % 64 or self.block_threads % team:
            raise ValueError(f"block_threads={self.block_threads} must hold whole wavefronts and teams")
        vpl = -(-self.meta.row_vectors // p.lanes_x)
        if not 1 <= p.vectors_per_pass <= vpl:
            raise ValueError(f"vectors_per_pass={p.vectors_per_pass} outside [1, {vpl}]")
        if min(p.items_per_thread, p.bags_per_team) < 1:
            raise ValueError("items_per_thread and bags_per_team must be >= 1")

    def EmitScheduleBody(self, params: NamedTuple) -> str:
        p = self.team_params(params)
        self._check(p)
        v = self.sched_vars
        m = self.meta
        return f'''
  rfx::team_bags<{v.BLOCK_THREADS}, {m.dtype_id}, {m.embed_dim}, {p.lanes_x}, {p.lanes_y},
                 {p.items_per_thread}, {p.bags_per_team}, {p.vectors_per_pass}, {v.out_vec}>(
      {v.stage},
      {v.embed_table}, {v.indices}, {v.offsets}, {v.output},
      {v.out_row_stride}, {v.embed_dim_offset}, {v.bag_begin}, {v.bag_end}, {v.skip_long},
      {v.mid_queue}, {v.feat_id});
'''

    def LongBagThreshold(self, params: NamedTuple) -> int:
        """rfx::long_bag_threshold(U, Y): more than sixteen dependent rounds of the team."""
        p = self.team_params(params)
        return max(64, 16 * p.items_per_thread * p.lanes_y)

    def EmitShmemType(self, params: NamedTuple) -> str:
        return "char"

    def NeedsOutputStage(self, params: NamedTuple) -> bool:
        """fp16 / int8 teams stage their output through the kernel's ``TeamStage`` LDS buffer."""
        return self.meta.elems_per_vector > 4

    def TileGranularity(self, params: NamedTuple) -> int:
        p = self.team_params(params)
        return self.block_threads // (p.lanes_x * p.lanes_y) * p.bags_per_team


class ThreadPerBagSchedule(TeamScheduleBase):
    """One lane per bag: the lane walks its bag and loads whole rows."""

    def team_params(self, params: ThreadPerBagParams) -> TeamParams:
        return TeamParams(1, 1, params.items_per_thread, params.bags_per_thread, params.vectors_per_pass)

    def GenParamCandidates(self, stats: InputStats = None) -> List[ThreadPerBagParams]:
        m = self.meta
        out = []
        if m.payload_bytes > 256:      # rows this long always want several lanes
            return out
        for vpp in passes_for(m.row_vectors, m):
            for bags in (1, 2, 4):
                for items in (1, 2, 4):
                    p = ThreadPerBagParams(items, bags, vpp)
                    if fits_registers(m, self.team_params(p)):
                        out.append(p)
        return out


class SubWavefrontPerBagSchedule(TeamScheduleBase):
    """2..32 lanes per bag."""

    def team_params(self, params: SubWavefrontPerBagParams) -> TeamParams:
        return TeamParams(*params)

    def GenParamCandidates(self, stats: InputStats = None) -> List[SubWavefrontPerBagParams]:
        m = self.meta
        out = []
        vmax = next_pow2(m.row_vectors)
        for x in _pow2_upto(min(32, vmax)):
            vpl = -(-m.row_vectors // x)
            if vpl > 8:
                continue
            for y in (1, 2, 4, 8, 16):
                team = x * y
                if team < 2 or team > 32:
                    continue
                vpp = vpl if vpl * m.elems_per_vector <= MAX_ACC_FLOATS else passes_for(vpl, m)[-1]
                for items in (1, 2, 4, 8):
                    for bags in ((1, 2, 4) if y == 1 else (1,)):
                        if bags > 1 and items > 2:
                            continue
                        p = SubWavefrontPerBagParams(x, y, items, bags, vpp)
                        if fits_registers(m, TeamParams(*p)):
                            out.append(p)
        return out


class WavefrontPerBagSchedule(TeamScheduleBase):
    """A whole 64-lane wavefront per bag: X column lanes x 64/X lookup lanes."""

    def team_params(self, params: WavefrontPerBagParams) -> TeamParams:
        return TeamParams(params.lanes_x, 64 // params.lanes_x, params.items_per_thread, 1,
                          params.vectors_per_pass)

    def GenParamCandidates(self, stats: InputStats = None) -> List[WavefrontPerBagParams]:
        m = self.meta
        out = []
        vmax = next_pow2(m.row_vectors)
        for x in _pow2_upto(min(64, vmax)):
            vpl = -(-m.row_vectors // x)
            if vpl > 8:
                continue
            vpp = vpl if vpl * m.elems_per_vector <= MAX_ACC_FLOATS else passes_for(vpl, m)[-1]
            for items in (1, 2, 4, 8):
                p = WavefrontPerBagParams(x, items, vpp)
                if fits_registers(m, self.team_params(p)):
                    out.append(p)
        return out


class OneHotBagParams(NamedTuple):
    lanes_x: int
    bags_per_team: int


class OneHotBagSchedule(ScheduleBase):
    """Bags of at most one lookup: ``rfx::onehot_bags``, X column lanes per bag, ``bags_per_team``
    bags (and row loads) in flight per team, the index fetched together with the bag's offsets
    when the batch holds exactly one lookup per bag.  A wavefront whose pass holds a longer bag
    runs that pass through ``rfx::team_bags``, so the schedule is right for any input and fast
    for the input it is meant for.

    Reference counterpart: ``OneHotSchedule`` / ``OneHotMultiBlockSchedule``
    (examples/schedules/one_hot.py:22-92, one_hot_multi_block.py), whose kernel takes the bag
    length of 1 for granted."""

    # row vectors a lane holds in flight at most (bags_per_team x vectors per lane)
    MAX_VECTORS_IN_FLIGHT = 16

    def _check(self, p: OneHotBagParams) -> None:
        x = p.lanes_x
        if x < 1 or x > 64 or x & (x - 1):
            raise ValueError(f"lanes_x={x} is not a power of two <= 64")
        if self.block_threads % 64:
            raise ValueError(f"block_threads={self.block_threads} must hold whole wavefronts")
        if p.bags_per_team < 1:
            raise ValueError("bags_per_team must be >= 1")

    def EmitScheduleBody(self, params: OneHotBagParams) -> str:
        self._check(params)
        v = self.sched_vars
        m = self.meta
        return f'''
  rfx::onehot_bags<{v.BLOCK_THREADS}, {m.dtype_id}, {m.embed_dim}, {params.lanes_x},
                   {params.bags_per_team}, {v.out_vec}>(
      {v.stage},
      {v.embed_table}, {v.indices}, {v.offsets}, {v.output},
      {v.out_row_stride}, {v.embed_dim_offset}, {v.bag_begin}, {v.bag_end}, {v.skip_long},
      {v.one_per_bag});
'''

    def EmitShmemType(self, params: OneHotBagParams) -> str:
        return "char"

    def NeedsOutputStage(self, params: OneHotBagParams) -> bool:
        # the general routine behind it stages fp16 / int8 outputs through LDS
        return self.meta.elems_per_vector > 4

    def LongBagThreshold(self, params: OneHotBagParams) -> int:
        return 64           # rfx::long_bag_threshold(2, 1) of the general routine behind it

    def TileGranularity(self, params: OneHotBagParams) -> int:
        return self.block_threads // params.lanes_x * params.bags_per_team

    def GenParamCandidates(self, stats: InputStats = None) -> List[OneHotBagParams]:
        m = self.meta
        out = []
        for x in _pow2_upto(min(64, next_pow2(m.row_vectors))):
            vpl = -(-m.row_vectors // x)
            if vpl > 8:
                continue
            for bags in (1, 2, 4, 8):
                if bags * vpl <= self.MAX_VECTORS_IN_FLIGHT:
                    out.append(OneHotBagParams(x, bags))
        return out

    def default_params(self) -> OneHotBagParams:
        """Two row vectors per lane where the row has four or more, two bags per team: four row
        loads in flight per lane (measured on 26 features x 4 096 bags of 256-byte rows: 8 lanes
        x 2 bags 8.2 us, 8 x 4 8.7 us, 16 lanes x 2, 4 or 8 bags 12 us and more)."""
        v = self.meta.row_vectors
        x = min(64, next_pow2(v))
        if v >= 4:
            x //= 2
        return OneHotBagParams(x, 2)
