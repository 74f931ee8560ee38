"""`roofline.traffic` of bench.py comes from a counter record that names the kernel sources it was taken from: a record
from other sources, or for another tile, is not reported (host-side logic only; no GPU)."""
import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402

HEADER = ("Correlation_Id,Dispatch_Id,Agent_Id,Queue_Id,Process_Id,Thread_Id,Grid_Size,Kernel_Id,Kernel_Name,Workgroup_Size,"
          "LDS_Block_Size,Scratch_Size,VGPR_Count,Accum_VGPR_Count,SGPR_Count,Counter_Name,Counter_Value,Start_Timestamp,End_Timestamp\n")
CAL = "void at::native::vectorized_elementwise_kernel<4, at::native::CUDAFunctorOnSelf_add<int>, std::array<char*, 2ul> >(int)"
GEMM = "void tnx::gemm_tile_kernel<tnx::TagBF16, tnx::TileCfg<tnx::TagBF16, 256, 256, 64, 4, 2>, true, false, false, false>(tnx::GemmParams)"
TILE = {"block_m": 256, "block_n": 256, "block_k": 64, "group_m": 8, "num_stages": 2, "num_warps": 4, "superblock": 1}


def counter_csv(path, counter, calibration, kernel_values):
    rows = [f'1,1,"Agent 1",1,1,1,{1 << 24},5,"{CAL}",256,0,0,8,0,32,"{counter}",{calibration},10,20\n']
    rows += [f'{i + 2},{i + 2},"Agent 1",1,1,1,262144,9,"{GEMM}",256,131072,224,256,256,100,"{counter}",{v},30,40\n'
             for i, v in enumerate(kernel_values)]
    rows.append(f'99,99,"Agent 1",1,1,1,4096,3,"some_other_kernel",256,0,0,8,0,32,"{counter}",5.0,50,60\n')
    with open(path, "w") as f:
        f.write(HEADER + "".join(rows))
    return str(path)


def test_record_is_built_from_two_counter_files_and_refused_when_stale(tmp_path, monkeypatch):
    monkeypatch.setattr(bench, "TRAFFIC_RECORD", str(tmp_path / "c2_hbm_traffic.json"))
    assert bench.recorded_traffic(TILE) == (None, "no counter record (profiles/c2_hbm_traffic.json)")
    # the 2^28-byte calibration pass reads 131072 KiB on FETCH_SIZE (factor 2) and 262144 KiB on WRITE_SIZE (factor 1)
    fetch = counter_csv(tmp_path / "fetch.csv", "FETCH_SIZE", 131072.0, [789000.0, 790000.0])
    write = counter_csv(tmp_path / "write.csv", "WRITE_SIZE", 262144.0, [187000.0, 188000.0])
    rec = bench.write_traffic_record(fetch, write, TILE)
    assert (rec["fetch_kib"], rec["fetch_scale"], rec["write_kib"], rec["write_scale"]) == (789500.0, 2.0, 187500.0, 1.0)
    assert rec["kernel_source_sha256"] == bench.kernel_source_hash() and rec["dispatches"] == [2, 2]
    nbytes, note = bench.recorded_traffic(TILE)
    assert nbytes == int((789500.0 * 2.0 + 187500.0) * 1024) == rec["bytes_per_launch"] and "c2_hbm_traffic.json" in note
    # another tile: not this record's kernel
    assert bench.recorded_traffic(dict(TILE, num_warps=8))[0] is None
    # other kernel sources: the record is stale and says so instead of being reported
    stale = dict(rec, kernel_source_sha256="0" * 64)
    with open(bench.TRAFFIC_RECORD, "w") as f:
        json.dump(stale, f)
    nbytes, note = bench.recorded_traffic(TILE)
    assert nbytes is None and "other kernel sources" in note
    with pytest.raises(SystemExit):                                   # a counter file without the kernel's rows
        bench.write_traffic_record(write, write, TILE)


def test_committed_record_names_committed_sources():
    """The record in profiles/ must describe the kernel sources of this tree, or bench.py reports no traffic."""
    path = os.path.join(ROOT, "profiles", "c2_hbm_traffic.json")
    with open(path) as f:
        rec = json.load(f)
    assert set(rec["kernel_sources"]) == set(bench.KERNEL_SOURCES)
    assert rec["kernel_source_sha256"] == bench.kernel_source_hash(), "re-run the two --pmc passes and bench.py --traffic-from"
    assert rec["bytes_per_launch"] > rec["algorithmic_bytes"] == 3 * 8192 * 8192 * 2
