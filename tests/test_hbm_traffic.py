"""The record of counter-measured HBM traffic that bench.py reports: two rocprofv3 ``--pmc`` csv
files (FETCH_SIZE, WRITE_SIZE) become bytes per launch, scaled by a copy of known size in the same
run, and the figure is handed out only for the library it was measured on."""

import os

import pytest

from benchaid import hbm_traffic
from recflex_amd import prebuilt

HEADER = ('"Correlation_Id","Dispatch_Id","Agent_Id","Queue_Id","Process_Id","Thread_Id","Grid_Size",'
          '"Kernel_Id","Kernel_Name","Workgroup_Size","LDS_Block_Size","Scratch_Size","VGPR_Count",'
          '"Accum_VGPR_Count","SGPR_Count","Counter_Name","Counter_Value","Start_Timestamp","End_Timestamp"')


def _csv(path, counter, rows):
    lines = [HEADER]
    for i, (name, value) in enumerate(rows):
        lines.append(f'{i},{i},"Agent 1",1,10,10,327680,3,"{name}",256,1536,0,48,0,80,"{counter}",{value},1,2')
    path.write_text("\n".join(lines) + "\n")
    return str(path)


def test_record_scales_by_the_copy_and_is_keyed_to_the_library(tmp_path, monkeypatch):
    monkeypatch.setattr(hbm_traffic, "RECORD_PATH", str(tmp_path / "hbm_traffic.json"))
    model = "c1"
    prebuilt.ensure_built(model)
    assert hbm_traffic.recorded_traffic_bytes(model) is None          # nothing recorded yet
    copy_bytes = 1 << 20
    # the copy reads 1 MiB: the fetch counter shows 512 (units of 2 KiB), the write counter 1024
    fetch = _csv(tmp_path / "f_counter_collection.csv", "FETCH_SIZE",
                 [("CalibrationCopyKnl", 512), ("__amd_rocclr_copyBuffer", 70000), ("FusedKnl", 100),
                  ("FusedKnl", 300), ("other", 9999)])
    write = _csv(tmp_path / "w_counter_collection.csv", "WRITE_SIZE",
                 [("CalibrationCopyKnl", 1024), ("FusedKnl", 50), ("FusedKnl", 50)])
    rec = hbm_traffic.record(model, fetch, write, copy_bytes)
    assert rec["fetch_bytes_per_unit"] == 2048 and rec["write_bytes_per_unit"] == 1024
    assert rec["read_bytes"] == 200 * 2048 and rec["written_bytes"] == 50 * 1024
    assert rec["bytes"] == 200 * 2048 + 50 * 1024 and rec["dispatches"] == [2, 2]
    assert hbm_traffic.recorded_traffic_bytes(model) == rec["bytes"]
    assert hbm_traffic.recorded_traffic_bytes("c2") is None
    # the library changes (another emitted source): the record no longer applies
    monkeypatch.setattr(hbm_traffic, "library_key", lambda m: "something else")
    assert hbm_traffic.recorded_traffic_bytes(model) is None


def test_record_needs_both_kernels_in_the_counter_file(tmp_path, monkeypatch):
    monkeypatch.setattr(hbm_traffic, "RECORD_PATH", str(tmp_path / "hbm_traffic.json"))
    prebuilt.ensure_built("c1")
    only_fused = _csv(tmp_path / "a_counter_collection.csv", "FETCH_SIZE", [("FusedKnl", 1)])
    both = _csv(tmp_path / "b_counter_collection.csv", "WRITE_SIZE", [("FusedKnl", 1), ("CalibrationCopyKnl", 4)])
    twice = _csv(tmp_path / "c_counter_collection.csv", "FETCH_SIZE",
                 [("FusedKnl", 1), ("CalibrationCopyKnl", 4), ("CalibrationCopyKnl", 4)])
    with pytest.raises(ValueError, match="calibrate"):
        hbm_traffic.record("c1", only_fused, both, 4096)
    with pytest.raises(ValueError, match="exactly one"):
        hbm_traffic.record("c1", twice, both, 4096)
    with pytest.raises(ValueError, match="FETCH_SIZE"):
        hbm_traffic.record("c1", both, both, 4096)
    assert not os.path.exists(hbm_traffic.RECORD_PATH)


def test_committed_records_name_known_models():
    for model, rec in hbm_traffic.load_records().items():
        assert model in prebuilt.model_names() and rec["bytes"] > 0 and len(rec["key"]) == 24
