"""Host-side pieces of the measurement harness (CPU): the counter-dump reader behind the HBM traffic figure and
the check that ties that figure to the kernel sources it was measured on."""
from __future__ import annotations

import json
from pathlib import Path

from latent_bounded_interfaces_amd import benchmarks

HEADER = ('"Correlation_Id","Dispatch_Id","Agent_Id","Queue_Id","Process_Id","Thread_Id","Grid_Size","Kernel_Id",'
          '"Kernel_Name","Workgroup_Size","LDS_Block_Size","Scratch_Size","VGPR_Count","Accum_VGPR_Count","SGPR_Count",'
          '"Counter_Name","Counter_Value","Start_Timestamp","End_Timestamp"\n')


def _dump(folder: Path, counter: str, rows):
    folder.mkdir()
    lines = [HEADER]
    for i, (kernel, value) in enumerate(rows, start=1):
        lines.append(f'{i},{i},"Agent 1",1,1,1,64,1,"{kernel}",256,0,0,4,0,16,"{counter}",{value},0,1\n')
    (folder / "p_counter_collection.csv").write_text("".join(lines))


def test_traffic_from_counter_dumps_and_staleness(tmp_path, monkeypatch):
    kernel = "void lbi::scan_mfma_kernel<float, 256, 32, 64, true, 0>(float const*)"
    # FETCH_SIZE counts half a KiB per KiB moved, WRITE_SIZE one; the first copy is the calibration copy
    _dump(tmp_path / "f", "FETCH_SIZE", [("__amd_rocclr_copyBuffer", 512.0), (kernel, 1000.0), (kernel, 1100.0),
                                        ("__amd_rocclr_copyBuffer", 7.0)])
    _dump(tmp_path / "w", "WRITE_SIZE", [("__amd_rocclr_copyBuffer", 1024.0), (kernel, 3000.0), (kernel, 3000.0)])
    pkg = tmp_path / "pkg"
    (pkg / "csrc").mkdir(parents=True)
    (pkg / "csrc" / "k.hip").write_text("kernel v1")
    monkeypatch.setattr(benchmarks, "PACKAGE_DIR", pkg)
    record = benchmarks.pmc_traffic(str(tmp_path / "f"), str(tmp_path / "w"), kernel="scan_mfma_kernel<float, 256, 32, 64, true, 0>",
                                    copy_kernel="__amd_rocclr_copyBuffer", copy_bytes=1024 * 1024, sources=["csrc/k.hip"])
    assert record["dispatches_averaged"] == 2
    assert record["fetch_scale"] == 2.0 and record["write_scale"] == 1.0
    assert record["traffic_bytes"] == int((1050.0 * 2.0 + 3000.0) * 1024)
    path = tmp_path / "t.json"
    path.write_text(json.dumps(record))
    name = "scan_mfma_kernel<float, 256, 32, 64, true, 0>"
    assert benchmarks.load_traffic(path, name) == record["traffic_bytes"]
    assert benchmarks.load_traffic(path, "scan_split_kernel") is None          # another kernel
    assert benchmarks.load_traffic(tmp_path / "missing.json", name) is None
    (pkg / "csrc" / "k.hip").write_text("kernel v2")                             # the source moved on
    assert benchmarks.load_traffic(path, name) is None


def test_committed_traffic_record_names_the_bench_kernel():
    import bench

    record = json.loads(Path(bench.SCAN_TRAFFIC_JSON).read_text())
    assert record["kernel"] == bench.SCAN_KERNEL
    assert set(record["sources"]) == {"csrc/lbi_scan.hip", "csrc/lbi_common.h"}
    # algorithmic bytes of the workload are 4.320e9: a figure far from it would be a unit slip
    assert 4.2e9 < record["traffic_bytes"] < 4.6e9


def test_flop_and_byte_formulas():
    # one shared Q K^T plus four products per direction over the causal triangle
    assert benchmarks.algorithmic_flops(4, 16, 4096, 128, 16, True) == 4 * 16 * (4096 * 4097 / 2) * 2 * 128 * 65
    assert benchmarks.algorithmic_flops(1, 1, 8, 4, 2, False) == 64 * 2 * 4 * 9
    assert benchmarks.algorithmic_bytes(8, 8, 128, 64, 4, 2) == 8 * 8 * 128 * 64 * 2 * 19
