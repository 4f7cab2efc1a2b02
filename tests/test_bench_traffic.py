"""bench_traffic.py: kernel-name classification, counter-file parsing and the staleness check (no GPU needed)."""
import json
import os

import bench_traffic as BT


def test_kernel_families():
    assert BT.family("void amoe::fwd256_kernel<unsigned short, 1, true, true, true, false>(amoe::RowsParams)") == "fwd"
    assert BT.family("void amoe::bwdx256_kernel<unsigned short, true, false, false, 128>(amoe::RowsParams)") == "xgrad"
    assert BT.family("void amoe::gemm_wgrad_kernel<unsigned short>(amoe::WgradParams)") == "wgrad"
    assert BT.family("void amoe::wgrad256_kernel<unsigned short>(amoe::WgradParams)") == "wgrad"
    assert BT.family("void amoe::wgrad_reduce_kernel<unsigned short>(amoe::WgradParams)") is None
    assert BT.family("void amoe::gemm_rows_kernel<float, true, 2, false>(amoe::RowsParams)") == "xgrad"
    assert BT.family("void amoe::gemm_rows_kernel<float, false, 1, false>(amoe::RowsParams)") == "fwd"
    assert BT.family("void amoe::head_reduce_kernel<unsigned short>(...)") is None


def _counter_file(tmp_path, name, counter, values):
    d = tmp_path / name / "vm"
    d.mkdir(parents=True)
    rows = ["Dispatch_Id,Kernel_Name,Counter_Name,Counter_Value"]
    i = 0
    rows.append(f"{i},__amd_rocclr_copyBuffer,{counter},{values['copy']}")
    for step in range(2):
        for kern, role_vals in (("void amoe::fwd256_kernel<unsigned short, 1>(p)", ("fwd_up", "fwd_down")),
                                ("void amoe::bwdx256_kernel<unsigned short, true>(p)", ("xgrad_down", "xgrad_up")),
                                ("void amoe::gemm_wgrad_kernel<unsigned short>(p)", ("wgrad_down", "wgrad_up"))):
            for role in role_vals:
                i += 1
                rows.append(f'{i},"{kern}",{counter},{values[role] + step}')
                i += 1
                rows.append(f'{i},"{kern}",OTHER_COUNTER,7')
    (d / "1_counter_collection.csv").write_text("\n".join(rows) + "\n")
    return str(tmp_path / name)


def test_counter_runs_become_bytes_per_launch(tmp_path, monkeypatch):
    roles = ["fwd_up", "fwd_down", "xgrad_down", "xgrad_up", "wgrad_down", "wgrad_up"]
    fetch = dict({r: 1000 * (i + 1) for i, r in enumerate(roles)}, copy=131072)     # a copy reads half its bytes
    write = dict({r: 100 * (i + 1) for i, r in enumerate(roles)}, copy=262144)
    fdir = _counter_file(tmp_path, "fetch", "FETCH_SIZE", fetch)
    wdir = _counter_file(tmp_path, "write", "WRITE_SIZE", write)
    out = tmp_path / "traffic.json"
    monkeypatch.setattr(BT, "traffic_file", lambda config: str(out))
    monkeypatch.setattr("sys.argv", ["bench_traffic.py", fdir, wdir, "--config", "cX"])
    BT.main()
    rec = json.loads(out.read_text())
    assert rec["copy_calibration"]["fetch_scale"] == 2.0 and rec["copy_calibration"]["write_scale"] == 1.0
    # the first step is left out of the average: the second step's readings are value + 1
    assert rec["launches"]["xgrad_up"]["read_bytes"] == (4000 + 1) * 1024 * 2.0
    assert rec["launches"]["wgrad_down"]["write_bytes"] == (500 + 1) * 1024 * 1.0
    assert rec["source_digest"] == BT.source_digest()
    got, note = BT.load_traffic("cX")
    assert note is None and got["fwd_up"] == (1000 + 1) * 2048.0 + (100 + 1) * 1024.0
    rec["source_digest"] = "0" * 64
    out.write_text(json.dumps(rec))
    got, note = BT.load_traffic("cX")
    assert got is None and "changed" in note


def test_recorded_traffic_file_is_well_formed():
    path = BT.traffic_file("c3")
    assert os.path.exists(path)
    with open(path) as fh:
        rec = json.load(fh)
    assert set(rec["launches"]) == {"fwd_up", "fwd_down", "xgrad_down", "xgrad_up", "wgrad_down", "wgrad_up"}
    assert all(v["total_bytes"] > 1e8 for v in rec["launches"].values())
