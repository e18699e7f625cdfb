"""No-GPU checks of the boundary: every symbol that include/recflex_hip.h declares is exported by
the libraries that implement it, the ctypes struct layouts match the header, the HIP attribute
numbers used by hip_helper match the installed header, and the text-format readers behave like
the reference's."""

import ctypes
import os
import re

import numpy as np
import pytest

from helpers import ROOT, oracle
from recflex_amd import prebuilt
from recflex_amd.code_emitter.build_basic import BasicBuilder
from recflex_amd.librecom import RecomInfo, RecomLib, RecomProcessArgs, EXPORTED_SYMBOLS

HEADER = os.path.join(ROOT, "include", "recflex_hip.h")


def _declared_functions():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return re.findall(r"\b(recom_[a-z_]+)\s*\(", src)


def test_header_declares_what_the_loaders_bind():
    names = set(_declared_functions())
    assert set(EXPORTED_SYMBOLS) <= names
    assert {"recom_host_parse_lines", "recom_host_pack", "recom_host_alignmem",
            "recom_host_packed_size", "recom_host_max_indices"} <= names


def test_generated_library_exports_every_gpu_symbol():
    """Loads a prebuilt librecom.so (no device needed for dlopen and the static queries)."""
    path = prebuilt.ensure_built("c1")
    lib = ctypes.CDLL(path)
    for name in _declared_functions():
        if not name.startswith("recom_host_"):
            assert hasattr(lib, name), f"{path} lacks {name}"
    r = RecomLib(path)
    assert r.num_features == 4 and r.embed_dim_sum == 128 and r.info.block_threads == 256
    assert r.embed_dims == [32] * 4 and r.embed_dim_offsets == [0, 32, 64, 96]
    assert r.dtypes == [0] * 4 and r.row_strides == [128] * 4
    assert r.info.timing == 0 and r.info.static_binding == 0 and r.info.tile_bytes == 0    # 0: tiles sized per batch


def test_host_library_exports_every_host_symbol():
    lib = ctypes.CDLL(BasicBuilder().build())
    for name in _declared_functions():
        if name.startswith("recom_host_"):
            assert hasattr(lib, name), name


def test_ctypes_structs_match_header_layout():
    # recom_info: 11 named int32 + 5 reserved; recom_process_args: 5 pointers, 4 int32,
    # 3 pointers, an int64, a pointer and an int64 on LP64
    assert ctypes.sizeof(RecomInfo) == 16 * 4
    assert ctypes.sizeof(RecomProcessArgs) == 5 * 8 + 4 * 4 + 3 * 8 + 8 + 8 + 8 + 2 * 8 + 8
    assert RecomProcessArgs.d_lookup_counts.offset == 120
    assert RecomProcessArgs.output_row_stride.offset == 80
    assert RecomProcessArgs.d_workspace.offset == 88 and RecomProcessArgs.workspace_bytes.offset == 96
    assert RecomProcessArgs.start_event.offset == 104 and RecomProcessArgs.stop_event.offset == 112
    assert RecomProcessArgs.batch.offset == 40 and RecomProcessArgs.d_schedule_choice.offset == 56
    assert RecomProcessArgs.d_times.offset == 64
    src = open(HEADER).read()
    fields = re.search(r"typedef struct recom_process_args \{(.*?)\} recom_process_args;", src, re.S).group(1)
    fields = re.sub(r"/\*.*?\*/", "", fields, flags=re.S)
    names = re.findall(r"(\w+);", fields)
    assert names == [n for n, _ in RecomProcessArgs._fields_]
    assert r"int recom_get_candidate_counts" in src
    fields = re.search(r"typedef struct recom_info \{(.*?)\} recom_info;", src, re.S).group(1)
    fields = re.sub(r"/\*.*?\*/", "", fields, flags=re.S)
    names = [n.split("[")[0] for n in re.findall(r"int32_t (\w+(?:\[\d+\])?);", fields)]
    assert names == [n for n, _ in RecomInfo._fields_]


def test_process_rejects_bad_arguments_without_a_device():
    """Argument validation happens before any HIP call: hipErrorInvalidValue (1)."""
    r = RecomLib(prebuilt.ensure_built("c1"))
    assert r.lib.recom_process(None) == 1
    a = RecomProcessArgs()
    assert r.lib.recom_process(ctypes.byref(a)) == 1
    a = RecomProcessArgs(d_embed_table_ptrs=8, d_io_ptrs=8, d_output=8, batch=-1)
    assert r.lib.recom_process(ctypes.byref(a)) == 1
    a = RecomProcessArgs(d_embed_table_ptrs=8, d_io_ptrs=8, d_output=8, batch=4, d_times=8)
    assert r.lib.recom_process(ctypes.byref(a)) == 1         # timers on a non-timing build
    a = RecomProcessArgs(d_embed_table_ptrs=8, d_io_ptrs=8, d_output=16, batch=0)
    assert r.lib.recom_process(ctypes.byref(a)) == 0         # empty batch: nothing to launch
    # output rows: a stride below the row length, one that breaks the 16-byte stores of a
    # library whose sum of dims is a multiple of 4, a misaligned base
    assert r.embed_dim_sum % 4 == 0
    for bad in ({"output_row_stride": r.embed_dim_sum - 4}, {"output_row_stride": r.embed_dim_sum + 2},
                {"d_output": 24}):
        kw = dict(d_embed_table_ptrs=8, d_io_ptrs=8, d_output=16, batch=0)
        kw.update(bad)
        assert r.lib.recom_process(ctypes.byref(RecomProcessArgs(**kw))) == 1, bad
    a = RecomProcessArgs(d_embed_table_ptrs=8, d_io_ptrs=8, d_output=16, batch=0,
                         output_row_stride=r.embed_dim_sum + 64)
    assert r.lib.recom_process(ctypes.byref(a)) == 0


def test_split_bag_library_wants_its_workspace():
    """A library with a schedule that splits bags over workgroups reports the workspace it needs
    (2048 slots of D floats and 2048 counters per such feature) and refuses a launch without
    it, before any HIP call; other libraries need none."""
    assert RecomLib(prebuilt.ensure_built("c1")).workspace_bytes == 0
    r = RecomLib(prebuilt.ensure_built("longbags"))
    dims = r.embed_dims
    assert r.workspace_bytes == sum(2048 * (d + 1) * 4 for d in dims)
    ok = dict(d_embed_table_ptrs=8, d_io_ptrs=8, d_output=16, batch=0)
    assert r.lib.recom_process(ctypes.byref(RecomProcessArgs(**ok))) == 1
    assert r.lib.recom_process(ctypes.byref(RecomProcessArgs(
        d_workspace=256, workspace_bytes=r.workspace_bytes - 1, **ok))) == 1
    assert r.lib.recom_process(ctypes.byref(RecomProcessArgs(
        d_workspace=264, workspace_bytes=r.workspace_bytes, **ok))) == 1        # misaligned
    assert r.lib.recom_process(ctypes.byref(RecomProcessArgs(
        d_workspace=256, workspace_bytes=r.workspace_bytes, **ok))) == 0        # empty batch


def test_missing_library_fails_loudly():
    with pytest.raises(FileNotFoundError):
        RecomLib("/nonexistent/librecom.so")
    from recflex_amd import rec_modules
    saved = rec_modules._current_lib
    rec_modules._current_lib = None
    try:
        with pytest.raises(RuntimeError):
            rec_modules.FeatEmbed("cpu", table_shapes=[(4, 4)])
    finally:
        rec_modules._current_lib = saved


def test_hip_attribute_numbers_match_installed_header():
    hdr = "/opt/rocm/include/hip/hip_runtime_api.h"
    if not os.path.exists(hdr):
        pytest.skip("no ROCm headers")
    src = open(hdr).read()
    body = re.search(r"typedef enum hipDeviceAttribute_t \{(.*?)\} hipDeviceAttribute_t;", src, re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    body = re.sub(r"//[^\n]*", "", body)
    names, val = {}, -1
    for item in body.split(","):
        item = item.strip()
        if not item:
            continue
        if "=" in item:
            n, v = [x.strip() for x in item.split("=")]
            val = int(v, 0) if re.fullmatch(r"(0x)?[0-9a-fA-F]+", v) else eval(v, {}, dict(names))
        else:
            n, val = item, val + 1
        names[n] = val
    from recflex_amd import hip_helper as h
    assert names["hipDeviceAttributeMultiprocessorCount"] == h.HIP_DEVICE_ATTRIBUTE_MULTIPROCESSOR_COUNT
    assert names["hipDeviceAttributeMaxThreadsPerMultiProcessor"] == h.HIP_DEVICE_ATTRIBUTE_MAX_THREADS_PER_MULTIPROCESSOR
    assert names["hipDeviceAttributeComputeCapabilityMajor"] == h.HIP_DEVICE_ATTRIBUTE_COMPUTE_CAPABILITY_MAJOR
    assert names["hipDeviceAttributeComputeCapabilityMinor"] == h.HIP_DEVICE_ATTRIBUTE_COMPUTE_CAPABILITY_MINOR
    assert names["hipDeviceAttributeMaxSharedMemoryPerMultiprocessor"] == h.HIP_DEVICE_ATTRIBUTE_MAX_SHARED_MEMORY_PER_MULTIPROCESSOR
    assert names["hipDeviceAttributeWallClockRate"] == h.HIP_DEVICE_ATTRIBUTE_WALL_CLOCK_RATE
    assert names["hipDeviceAttributeClockRate"] == h.HIP_DEVICE_ATTRIBUTE_CLOCK_RATE


# ------------------------------------------------------------------------------------ text formats

def test_parse_configs(tmp_path):
    from recflex_amd.parser import parse_schedule_types, parse_table_dtypes, parse_table_shapes
    from recflex_amd.schedules import SCHEDULE_MAPPING
    t = tmp_path / "table_config.txt"
    t.write_text("1024,16\n4096,32,half\n100,128,int8\n")
    assert parse_table_shapes(str(t)) == [(1024, 16), (4096, 32), (100, 128)]
    assert parse_table_dtypes(str(t)) == ["float", "half", "int8"]
    s = tmp_path / "schedule_config.txt"
    s.write_text("OneHotSchedule\nReduceByKeySchedule,OneBlockMultiSampleSchedule,WarpPerSampleSchedule\nNoSuch\n")
    types = parse_schedule_types(str(s), SCHEDULE_MAPPING)
    assert [[c.__name__ if c else None for c in row] for row in types] == [
        ["OneHotSchedule"], ["ReduceByKeySchedule", "OneBlockMultiSampleSchedule", "WarpPerSampleSchedule"],
        [None]]


def test_parse_raw_data_batches_layout_and_sampling():
    """Batch k = the line range given by the running sum of the batch sizes; sampled batch ids
    follow the legacy numpy stream (parser.py:34-62)."""
    from recflex_amd.parser import parse_raw_data_batches
    from recflex_amd.utils import get_data_fnames
    d = os.path.join(ROOT, "tests", "golden", "model_test", "data")
    fnames = get_data_fnames(d)
    assert len(fnames) == 6
    sizes = [int(l) for l in open(os.path.join(d, "batch_sizes.txt")).read().split()]
    offs = np.cumsum([0] + sizes)
    ids = oracle.sample_batch_ids_legacy(len(sizes), 3, seed=0)
    fm = parse_raw_data_batches(os.path.join(d, "batch_sizes.txt"), fnames, 3, seed=0, feat_major=True)
    bm = parse_raw_data_batches(os.path.join(d, "batch_sizes.txt"), fnames, 3, seed=0, feat_major=False)
    assert len(fm) == 6 and len(fm[0]) == 3 and len(bm) == 3 and len(bm[0]) == 6
    lines4 = open(fnames[4]).read().splitlines()
    for i, b in enumerate(ids):
        assert fm[4][i] == lines4[offs[b]:offs[b + 1]] == bm[i][4]
        assert len(fm[4][i]) == sizes[b]
    # all batches when more are asked for than exist
    assert len(parse_raw_data_batches(os.path.join(d, "batch_sizes.txt"), fnames, 128)[0]) == len(sizes)


def test_rocprof_stats_reader(tmp_path):
    from recflex_amd.parser import parse_knl_total_time, parse_knl_calls_and_average, parse_first_knl_total_time
    p = tmp_path / "report_kernel_stats.csv"
    p.write_text('"Name","Calls","TotalDurationNs","AverageNs","Percentage","MinNs","MaxNs","StdDev"\n'
                 '"FusedKnl",10,1500000,150000.0,75.0,140000,160000,5000.0\n'
                 '"other_kernel",3,500000,166666.7,25.0,1,2,3.0\n')
    assert parse_knl_total_time("FusedKnl", str(tmp_path / "report")) == 1500000
    assert parse_knl_total_time("FusedKnl", str(p)) == 1500000
    assert parse_knl_calls_and_average("FusedKnl", str(tmp_path)) == (10, 150000.0)
    assert parse_first_knl_total_time(str(tmp_path)) == 1500000
    with pytest.raises(FileNotFoundError):
        parse_knl_total_time("FusedKnl", str(tmp_path / "nothing_here"))


def test_gather_probe_chunks_cover_every_lookup_once():
    from benchaid.gather_probe import make_chunks, CHUNK_LOOKUPS
    lookups = [2500, 0, 10, 1024]
    vectors = [2, 9, 64, 1]
    chunks = make_chunks(lookups, vectors)
    assert chunks.dtype == np.int32 and chunks.shape[1] == 4
    for f, n in enumerate(lookups):
        mine = chunks[chunks[:, 0] == f]
        assert mine[:, 2].sum() == n and (mine[:, 2] <= CHUNK_LOOKUPS).all() and (mine[:, 2] > 0).all()
        assert list(mine[:, 1]) == list(range(0, n, CHUNK_LOOKUPS))
        assert all(1 << int(l) >= min(vectors[f], 64) for l in mine[:, 3])
    assert make_chunks([0, 0], [1, 1]).shape == (0, 4)
    by_bytes = make_chunks(lookups, vectors, chunk_bytes=16384)
    for f, n in enumerate(lookups):
        mine = by_bytes[by_bytes[:, 0] == f]
        assert mine[:, 2].sum() == n
        if n:
            assert mine[0, 2] == min(n, max(32, min(4096, 16384 // (16 * vectors[f]))))
