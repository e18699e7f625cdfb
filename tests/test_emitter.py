"""Code emitter and schedule templates (host logic only: what is emitted, not how it runs)."""

import json
import os
import re

import pytest

from recflex_amd.code_emitter import CodeEmitter, MetaData, ScheduleBase
from recflex_amd.schedules import (SCHEDULE_MAPPING, BlockPerBagParams, BlockPerBagSchedule,
                                   SubWavefrontPerBagParams, SubWavefrontPerBagSchedule,
                                   ThreadPerBagSchedule, WavefrontPerBagParams,
                                   WavefrontPerBagSchedule, default_schedule, schedule_from_config)
from recflex_amd.schedules.team import fits_registers


def test_metadata_row_formats():
    m = MetaData(64)
    assert (m.data_type, m.row_stride, m.row_bytes, m.vec_bytes, m.row_vectors, m.elems_per_vector) == \
        ("float", 256, 256, 16, 16, 4)
    m = MetaData(128, "half")
    assert (m.row_stride, m.row_bytes, m.vec_bytes, m.row_vectors, m.elems_per_vector) == (256, 256, 16, 16, 8)
    m = MetaData(128, "int8")
    assert (m.row_stride, m.row_bytes, m.vec_bytes, m.row_vectors, m.elems_per_vector) == (144, 132, 16, 8, 16)
    m = MetaData(6)
    assert (m.vec_bytes, m.row_vectors) == (8, 3)
    with pytest.raises(ValueError):
        MetaData(3, "int8").vec_bytes
    with pytest.raises(ValueError):
        MetaData(8, "bfloat16").dtype_id


def test_reference_schedule_names_resolve():
    """The class names used by the reference's schedule_config.txt files."""
    for name in ("OneHotSchedule", "OneHotMultiBlockSchedule", "WarpPerSampleSchedule",
                 "OneBlockMultiSampleSchedule", "MultiBlockPerSampleSchedule", "ReduceByKeySchedule",
                 "ThreadPerBagSchedule", "SubWavefrontPerBagSchedule", "WavefrontPerBagSchedule",
                 "BlockPerBagSchedule"):
        cls = SCHEDULE_MAPPING[name]
        assert issubclass(cls, ScheduleBase)
        cands = cls(MetaData(16), 256).GenParamCandidates()
        assert len(cands) > 0
        assert len(set(cands)) == len(cands)


@pytest.mark.parametrize("dt,dim", [("float", 8), ("float", 128), ("half", 16), ("half", 256),
                                    ("int8", 128), ("float", 12)])
def test_candidates_are_valid_and_emit(dt, dim):
    meta = MetaData(dim, dt)
    total = 0
    for cls in (ThreadPerBagSchedule, SubWavefrontPerBagSchedule, WavefrontPerBagSchedule, BlockPerBagSchedule):
        sched = cls(meta, 256)
        for p in sched.GenParamCandidates():
            body = sched.EmitScheduleBody(p)          # raises on invalid parameters
            assert "rfx::" in body
            g = sched.TileGranularity(p)
            assert g >= 1 and 256 % g == 0 or g % 256 == 0 or g > 0
            if cls is not BlockPerBagSchedule:
                tp = sched.team_params(p)
                assert fits_registers(meta, tp)
                assert tp.lanes_x * tp.lanes_y <= 64
            total += 1
    assert 4 <= total <= 200


def test_invalid_params_rejected():
    meta = MetaData(64)
    with pytest.raises(ValueError):
        SubWavefrontPerBagSchedule(meta, 256).EmitScheduleBody(SubWavefrontPerBagParams(3, 1, 1, 1, 1))
    with pytest.raises(ValueError):
        SubWavefrontPerBagSchedule(meta, 256).EmitScheduleBody(SubWavefrontPerBagParams(16, 8, 1, 1, 1))
    with pytest.raises(ValueError):
        WavefrontPerBagSchedule(meta, 256).EmitScheduleBody(WavefrontPerBagParams(16, 1, 5))
    with pytest.raises(ValueError):
        BlockPerBagSchedule(meta, 256).EmitScheduleBody(BlockPerBagParams(16, 1, 1000))


def _emitter(dims_types, sched_fn=None):
    fs = []
    for d, t, pf in dims_types:
        fs.append(default_schedule(MetaData(d, t), pf, 256))
    return CodeEmitter(fs)


def test_body_dedup_and_tables():
    """Identical (LDS type, body) pairs are emitted once (codegen.py:233-243)."""
    em = _emitter([(32, "float", 4), (32, "float", 4), (64, "float", 4), (32, "float", 4), (32, "half", 4)])
    id_map, bodies = em.dedup()
    assert id_map == {0: 0, 1: 0, 2: 2, 3: 0, 4: 4} and bodies == [0, 2, 4]
    src = em.emit_kernel(occupancy=4)
    assert len(re.findall(r"void ProcessFeat\d+\(", src)) == 3
    assert "constexpr int NUM_FEATS = 5;" in src and "constexpr int EMBED_DIM_SUM = 192;" in src
    assert "__launch_bounds__(BLOCK_THREADS, 4)" in src
    m = re.search(r"c_embed_dim_offsets\[\] = \{\s*([\d,\s]+)\}", src)
    assert [int(v) for v in m.group(1).split(",")] == [0, 32, 64, 128, 160, 192]
    m = re.search(r"c_cand_func_ids\[\] = \{\s*([\d,\s]+)\}", src)
    assert [int(v) for v in m.group(1).split(",")] == [0, 0, 2, 0, 4]
    m = re.search(r"c_cand_begin\[\] = \{\s*([\d,\s]+)\}", src)
    assert [int(v) for v in m.group(1).split(",")] == [0, 1, 2, 3, 4, 5]
    # bytes per lookup = row bytes + int32 index; per bag = fp32 output slice + one offset
    m = re.search(r"c_lookup_bytes\[\] = \{\s*([\d,\s]+)\}", src)
    assert [int(v) for v in m.group(1).split(",")] == [132, 132, 260, 132, 68]
    m = re.search(r"c_bag_bytes\[\] = \{\s*([\d,\s]+)\}", src)
    assert [int(v) for v in m.group(1).split(",")] == [132, 132, 260, 132, 132]


def test_candidate_lists_share_bodies_across_features():
    """A tuning build carries every candidate of every feature; features with the same dim and
    element type share all their bodies."""
    from recflex_amd.schedules import WarpPerSampleSchedule, OneHotSchedule
    metas = [MetaData(16), MetaData(16), MetaData(32)]
    cands = []
    for m in metas:
        c = []
        for cls in (OneHotSchedule, WarpPerSampleSchedule):
            s = cls(m, 256)
            c.extend((s, p) for p in s.GenParamCandidates())
        cands.append(c)
    em = CodeEmitter(None, feat_candidates=cands)
    assert [len(c) for c in em.feat_candidates] == [len(c) for c in cands]
    id_map, bodies = em.dedup()
    n16, n32 = len(cands[0]), len(cands[2])
    assert len(bodies) <= n16 + n32
    for i in range(n16):
        assert id_map[n16 + i] == id_map[i]         # feature 1 reuses feature 0's bodies
    src = em.emit_kernel(occupancy=4, timing=True)
    assert f"constexpr int NUM_CANDIDATES = {2 * n16 + n32};" in src
    m = re.search(r"c_cand_begin\[\] = \{\s*([\d,\s]+)\}", src)
    assert [int(v) for v in m.group(1).split(",")] == [0, n16, 2 * n16, 2 * n16 + n32]
    assert em.feat_schedules[0] == cands[0][0]
    ser = em.serialize_candidates()
    assert len(ser) == 3 and len(ser[2]) == n32


def test_output_vector_width_follows_column_alignment():
    assert _emitter([(32, "float", 4), (64, "float", 4)]).out_vec() == 4
    assert _emitter([(6, "float", 4), (64, "float", 4)]).out_vec() == 2
    assert _emitter([(3, "float", 4), (64, "float", 4)]).out_vec() == 1


def test_emit_variants_and_file_update(tmp_path):
    em = _emitter([(32, "float", 4), (128, "int8", 50)])
    f = tmp_path / "process.hip"
    em.emit(str(f), occupancy=2, timing=True)
    src = f.read_text()
    assert "TIMING = true" in src and "s_memtime" in src and "s_ticks[feat_idx] +=" in src
    assert "atomicAdd(&d_times[f]" in src
    assert 'extern "C" int recom_process' in src and 'extern "C" int recom_get_info' in src
    mtime = f.stat().st_mtime_ns
    em.emit(str(f), occupancy=2, timing=True)            # unchanged -> not rewritten
    assert f.stat().st_mtime_ns == mtime
    em.emit(str(f), occupancy=2, timing=False, fixed_task_block_nums=[3, 9])
    src = f.read_text()
    assert "STATIC_BINDING = true" in src and "c_fixed_task_block_nums" in src
    em.emit(str(f), inline=False)
    assert "__noinline__ void ProcessFeat0" in f.read_text()
    h = tmp_path / "preprocess.cpp"
    em.emit_host(str(h))
    hsrc = h.read_text()
    assert "recom_host_preprocess_feat" in hsrc and hsrc.count("static int PreprocFeat") == 1
    c = tmp_path / "CMakeLists.txt"
    em.emit_cmake_list(str(c), code_fname="process.hip", host_fname="preprocess.cpp")
    csrc = c.read_text()
    assert "--offload-arch=gfx950" in csrc and "-packed-fp32-ops" in csrc and "librecom.so" in csrc


def test_serialize_round_trip(tmp_path):
    em = _emitter([(32, "float", 1), (128, "half", 40), (128, "int8", 300), (256, "float", 900)])
    cfg = em.serialize_config()
    assert [c["schedule"] for c in cfg] == [type(s).__name__ for s, _ in em.feat_schedules]
    p = tmp_path / "schedule.json"
    em.dump_key(str(p))
    back = json.loads(p.read_text())
    for entry, (sched, params) in zip(back, em.feat_schedules):
        s2, p2 = schedule_from_config(entry, sched.meta, 256)
        assert type(s2) is type(sched) and p2 == params
    from recflex_amd.model_build import load_feat_schedules
    fs = load_feat_schedules(str(p))
    assert [p for _, p in fs] == [p for _, p in em.feat_schedules]
    assert [s.meta for s, _ in fs] == [s.meta for s, _ in em.feat_schedules]


def test_default_schedule_covers_all_templates():
    kinds = set()
    for dt in ("float", "half", "int8"):
        for dim in (8, 16, 32, 64, 128, 256):
            for pf in (1, 4, 30, 120, 800):
                if dt == "int8" and dim < 16:
                    continue
                s, p = default_schedule(MetaData(dim, dt), pf)
                s.EmitScheduleBody(p)
                kinds.add(type(s).__name__)
    # bags of 512 lookups and more get the whole workgroup (and several, when the batch is small)
    assert kinds >= {"SubWavefrontPerBagSchedule", "WavefrontPerBagSchedule", "SplitBagSchedule"}
    s, p = default_schedule(MetaData(64, "float"), 800)
    assert type(s).__name__ == "SplitBagSchedule" and s.TileGranularity(p) == -1
    assert s.WorkspaceFloats(p) == 2048 * 65 and "rfx::split_bags<" in s.EmitScheduleBody(p)


def test_split_bag_schedules_get_workspace_regions():
    """Features with a split-bag candidate get a region of 2048 * (D + 1) floats of the caller's
    workspace each, in feature order; the kernel takes the workspace pointer only then, and the
    reference names for long bags resolve to the split-bag schedule."""
    from recflex_amd.schedules import (SplitBagSchedule, MultiBlockPerSampleSchedule,
                                       ReduceByKeySchedule)
    assert issubclass(MultiBlockPerSampleSchedule, SplitBagSchedule)
    assert issubclass(ReduceByKeySchedule, SplitBagSchedule)
    fs = [default_schedule(MetaData(32), 4), default_schedule(MetaData(64), 900),
          default_schedule(MetaData(16, "half"), 2), default_schedule(MetaData(128, "int8"), 5000)]
    em = CodeEmitter(fs)
    regions, total = em.split_regions()
    assert regions == [-1, 0, -1, 2048 * 65] and total == 2048 * (65 + 129)
    src = em.emit_kernel(occupancy=4)
    assert f"SPLIT_BYTES = {total * 4}LL" in src and "c_split_region[feat_idx]" in src
    assert "rfx::split_bags<" in src and "bind_tiles<NUM_FEATS, BLOCK_THREADS, HAS_SPLIT," in src
    m = re.search(r"c_cand_gran\[\] = \{\s*([-\d,\s]+)\}", src)
    gran = [int(v) for v in m.group(1).split(",")]
    assert gran[1] == -1 and gran[3] == -1 and gran[0] > 0 and gran[2] > 0
    plain = CodeEmitter(fs[:1]).emit_kernel(occupancy=4)
    assert "SPLIT_BYTES = 0LL" in plain and "c_split_region" not in plain


def test_outlier_tiles_are_emitted_on_request():
    """outliers=True: a kernel that lists the bags beyond each feature's threshold (its
    schedule's reach, and at least 128 KiB of traffic), one block-wide body per (element type,
    dim), the list and its partial sums in the workspace.  Nothing of it otherwise."""
    fs = [default_schedule(MetaData(32), 4), default_schedule(MetaData(128), 1),
          default_schedule(MetaData(32), 30), default_schedule(MetaData(64, "half"), 900)]
    em = CodeEmitter(fs)
    thr, keys, body_of = em.long_bag_tables()
    # 132-byte lookups: 993 lookups make 128 KiB; 516-byte lookups: 255; the split-bag feature
    # takes bags of any length itself
    assert thr == [993, 255, 993, 0] and keys == [(0, 32), (0, 128)] and body_of == [0, 1, 0, -1]
    assert all(t >= s.LongBagThreshold(p) for t, (s, p) in zip(thr[:3], fs[:3]))
    src = em.emit_kernel(occupancy=4, outliers=True)
    assert "#define RFX_OUTLIERS 1" in src and "OutlierKnl" in src and "MAX_LONG_DIM = 128" in src
    assert src.count("rfx::split_part<") == 2 and "rfx::outliers_done(d_outliers)" in src
    assert "c_long_thr[feat_idx]" in src
    plain = em.emit_kernel(occupancy=4)
    assert "#define RFX_OUTLIERS 0" in plain and "OutlierKnl" not in plain and "c_long_thr" not in plain
    with pytest.raises(AssertionError):
        em.emit_kernel(occupancy=4, outliers=True, timing=True)


def _table(src: str, name: str):
    import re
    body = re.search(r"\b" + name + r"\[\] = \{(.*?)\};", src, re.S).group(1)
    return [int(v) for v in body.replace("\n", " ").split(",") if v.strip()]


def test_tile_order_permutes_the_kernels_tables_and_nothing_the_host_sees():
    """tile_order: inside the kernel a feature's number is its place in the tile space -- every
    per-feature table is emitted in that order, the output columns stay where the model has
    them, and what the caller passes per feature is found through c_ext_feat.  The identity and
    no order at all emit the same source; the host-side description of the library does not
    move."""
    fs = [default_schedule(MetaData(32), 4), default_schedule(MetaData(128), 1),
          default_schedule(MetaData(8), 30), default_schedule(MetaData(64, "half"), 900)]
    em = CodeEmitter(fs)
    plain = em.emit_kernel(occupancy=4)
    assert em.emit_kernel(occupancy=4, tile_order=[0, 1, 2, 3]) == plain
    assert "c_ext_feat" not in plain and "#define RFX_TILE_ORDER 0" in plain
    order = [2, 0, 3, 1]
    src = em.emit_kernel(occupancy=4, tile_order=order)
    assert "#define RFX_TILE_ORDER 1" in src and _table(src, "c_ext_feat") == order
    for name in ("c_cand_func_ids", "c_cand_gran", "c_embed_dims", "c_lookup_bytes", "c_bag_bytes"):
        assert _table(src, name) == [_table(plain, name)[f] for f in order], name
    offs = _table(plain, "c_embed_dim_offsets")
    assert offs == [0, 32, 160, 168, 232]
    assert _table(src, "c_embed_dim_offsets") == [offs[f] for f in order] + [232]
    assert _table(src, "c_split_region") == [_table(plain, "c_split_region")[f] for f in order]
    assert "d_lookup_counts, c_ext_feat}" in src and "d_lookup_counts, nullptr}" in plain
    assert em.emit_process_func(occupancy=4) == CodeEmitter(fs).emit_process_func(occupancy=4)
    with pytest.raises(AssertionError):
        em.emit_kernel(occupancy=4, tile_order=[0, 1, 2, 2])
    with pytest.raises(AssertionError):
        em.emit_kernel(occupancy=4, tile_order=order, timing=True)


def test_drawn_tail_takes_its_ticket_counters_from_the_workspace():
    """drawn_tail=N: the last N passes of the tile walk are drawn; the ticket counters live in
    the workspace where an outlier list would (never both), and the kernel that clears a static
    workspace clears them."""
    fs = [default_schedule(MetaData(32), 4), default_schedule(MetaData(128), 1)]
    em = CodeEmitter(fs)
    src = em.emit_kernel(occupancy=4, drawn_tail=2) + em.emit_process_func(occupancy=4)
    assert "#define RFX_DRAWN_TAIL 2" in src and "using OutlierSpace = rfx::TailTickets;" in src
    assert "rfx::draw_tail_ticket(d_tickets, xcd)" in src and "rfx::tail_tickets_done(d_tickets)" in src
    assert "sizeof(rfx::TailTickets) / 4" in src
    plain = em.emit_kernel(occupancy=4)
    assert "#define RFX_DRAWN_TAIL 0" in plain and "draw_tail_ticket" not in plain
    with pytest.raises(AssertionError):
        em.emit_kernel(occupancy=4, drawn_tail=2, outliers=True)


def test_launch_bounds_carry_wavefronts_per_simd_not_workgroups_per_cu():
    """hipcc reads the second argument of __launch_bounds__ as wavefronts per SIMD: a build of
    64-thread workgroups at 20 per CU has to ask for 5, one of 128-thread workgroups at 6 for 3."""
    from recflex_amd.code_emitter.codegen import waves_per_simd
    from recflex_amd.tuning.tuner import Tuner
    assert [waves_per_simd(o, 256) for o in (1, 2, 4, 5, 8, 12)] == [1, 2, 4, 5, 8, 8]
    assert waves_per_simd(20, 64) == 5 and waves_per_simd(16, 64) == 4 and waves_per_simd(6, 128) == 3
    assert waves_per_simd(1, 64) == 1 and waves_per_simd(2, 512) == 4
    assert Tuner.vgpr_budget(5) == 96 and Tuner.vgpr_budget(4) == 128 and Tuner.vgpr_budget(6) == 80
    assert Tuner.vgpr_budget(20, 64) == 96 and Tuner.vgpr_budget(6, 128) == 168
    fs = [default_schedule(MetaData(32, "float"), 4, 64)]
    src = CodeEmitter(fs).emit_kernel(occupancy=20)
    assert "constexpr int BLOCK_THREADS = 64;" in src and "__launch_bounds__(BLOCK_THREADS, 5)" in src


def test_binding_once_per_launch_is_the_default_only_where_every_workgroup_cannot_bind():
    """Up to ``BIND_ONCE_MIN_FEATS`` features every workgroup binds for itself -- unless its
    tables (12 bytes per feature and the prefix sum's second level) would not fit into LDS beside
    the other workgroups of the CU at the build's occupancy."""
    from recflex_amd.code_emitter.codegen import BIND_ONCE_MIN_FEATS, binds_once_by_default
    assert BIND_ONCE_MIN_FEATS == 3072
    assert not binds_once_by_default(1000, 4) and not binds_once_by_default(2500, 4)
    assert not binds_once_by_default(2500) and not binds_once_by_default(3000, 4)
    assert binds_once_by_default(3072, 4) and not binds_once_by_default(3072, 3)     # 41 KB of LDS
    assert binds_once_by_default(3073, 3) and binds_once_by_default(10000, 1)
    assert binds_once_by_default(2500, 5) and not binds_once_by_default(2000, 5)
    assert binds_once_by_default(1500, 8) and not binds_once_by_default(1000, 8)



def test_models_derived_from_a_tuned_schedule_keep_the_plain_walk_where_they_must():
    """A tuned schedule file may carry a tile order and a drawn end; the timing build, the
    frozen-binding build and the outlier builds made from the same file go with neither (the
    emitter refuses the combination), so they are emitted with the plain walk."""
    from recflex_amd import prebuilt
    tuned = prebuilt.model_spec("c3_tuned").emit_kwargs
    assert tuned.get("drawn_tail") and tuned.get("tile_order")
    for name in ("c3_tuned_ticks", "c3_tuned_static", "c3_skew", "c3_skew_plain"):
        kw = prebuilt.model_spec(name).emit_kwargs
        assert "drawn_tail" not in kw and "tile_order" not in kw, name
        assert kw.get("tile_bytes") == tuned.get("tile_bytes") and kw.get("xcd_segments") == tuned.get("xcd_segments")
    for name in ("c4_tuned", "c5_tuned", "refa_tuned", "reff4_tuned"):
        kw = prebuilt.model_spec(name).emit_kwargs
        assert kw.get("drawn_tail", 0) > 0 and not kw.get("outliers"), name
