"""Host-side profile summarizers against small hand-made rocprofv3 counter tables (no GPU)."""

import csv
import json

import pytest

from causal_trainer_dev_amd import rocprof_issue, rocprof_traffic

FIELDS = ["Dispatch_Id", "Kernel_Name", "Counter_Name", "Counter_Value"]


def _write(folder, rows):
    sub = folder / "host" / "1234_counter_collection.csv"
    sub.parent.mkdir(parents=True, exist_ok=True)
    with open(sub, "w", newline="") as handle:
        writer = csv.DictWriter(handle, fieldnames=FIELDS)
        writer.writeheader()
        for dispatch, kernel, counter, value in rows:
            writer.writerow({"Dispatch_Id": dispatch, "Kernel_Name": kernel, "Counter_Name": counter,
                             "Counter_Value": value})
    return str(folder)


def test_kernel_names_are_reduced_to_the_plain_identifier():
    short = rocprof_traffic._short
    assert short("_ZN2ct15attn_dkv_kernelILi128EEEvNS_10AttnParamsE") == "attn_dkv_kernel"
    assert short("void ct::attn_fwd_kernel<128, 4>(ct::AttnParams)") == "attn_fwd_kernel"
    assert short("ct_calibration_copy_kernel(char const*, char*, long)") == "ct_calibration_copy_kernel"


def test_traffic_is_scaled_by_the_copy_kernel_of_known_size(tmp_path, capsys):
    copy = "ct_calibration_copy_kernel(char const*, char*, long)"
    dkv = "_ZN2ct15attn_dkv_kernelILi128EEEvNS_10AttnParamsE"
    # a counter with two instances per dispatch (summed), two dispatches per kernel (averaged)
    fetch = _write(tmp_path / "f", [
        (1, copy, "FETCH_SIZE", 300.0), (1, copy, "FETCH_SIZE", 200.0),
        (2, dkv, "FETCH_SIZE", 100.0), (2, dkv, "FETCH_SIZE", 150.0),
        (3, dkv, "FETCH_SIZE", 350.0), (3, dkv, "WRITE_SIZE", 9e9),  # other counters are ignored
    ])
    write = _write(tmp_path / "w", [
        (1, copy, "WRITE_SIZE", 250.0),
        (2, dkv, "WRITE_SIZE", 50.0),
        (3, dkv, "WRITE_SIZE", 150.0),
    ])
    out = tmp_path / "out"
    assert rocprof_traffic.main([fetch, write, "1000", "--out", str(out), "--command", "cmd"]) == 0
    summary = json.loads((out / "traffic.json").read_text())
    assert summary["bytes_per_fetch_size_unit"] == pytest.approx(2.0)  # 1000 bytes / 500 units
    assert summary["bytes_per_write_size_unit"] == pytest.approx(4.0)  # 1000 bytes / 250 units
    entry = summary["kernels"]["attn_dkv_kernel"]
    assert entry["dispatches"] == 2
    assert entry["fetch_bytes"] == pytest.approx(2.0 * (250.0 + 350.0) / 2)
    assert entry["write_bytes"] == pytest.approx(4.0 * (50.0 + 150.0) / 2)
    assert "ct_calibration_copy_kernel" not in summary["kernels"]
    text = (out / "traffic_bench_attention_cutce.txt").read_text()
    assert "command: cmd" in text and "attn_dkv_kernel" in text
    assert capsys.readouterr().out == text


def test_traffic_needs_the_copy_kernel(tmp_path):
    dkv = "_ZN2ct15attn_dkv_kernelILi128EEEvNS_10AttnParamsE"
    fetch = _write(tmp_path / "f", [(1, dkv, "FETCH_SIZE", 1.0)])
    write = _write(tmp_path / "w", [(1, dkv, "WRITE_SIZE", 1.0)])
    with pytest.raises(SystemExit, match="calibration copy kernel"):
        rocprof_traffic.main([fetch, write, "1000", "--out", str(tmp_path / "o")])
    with pytest.raises(SystemExit, match="no counter_collection.csv"):
        rocprof_traffic.read_counter(str(tmp_path / "missing"), "FETCH_SIZE")


def test_issue_shares_follow_the_counter_units(tmp_path):
    fwd = "void ct::attn_fwd_kernel<128, 4>(ct::AttnParams)"
    rows_a, rows_b = [], []
    for dispatch in (1, 2):
        # two wavefronts per SIMD: SIMD time = 4 * 1000 / 2 = 2000 cycles
        rows_a += [(dispatch, fwd, "SQ_WAVE_CYCLES", 1000.0),
                   (dispatch, fwd, "SQ_VALU_MFMA_BUSY_CYCLES", 800.0),  # 40 % of 2000
                   (dispatch, fwd, "SQ_ACTIVE_INST_VALU", 300.0),      # 1200 cycles incl. the MFMAs' own issue
                   (dispatch, fwd, "SQ_ACTIVE_INST_LDS", 50.0),        # 200 cycles = 10 %
                   (dispatch, fwd, "SQ_WAIT_INST_ANY", 400.0),         # 1600 / 2 wavefronts = 40 %
                   (dispatch, fwd, "SQ_WAIT_INST_LDS", 100.0)]         # 10 %
        rows_b += [(dispatch, fwd, "SQ_INSTS_MFMA", 25.0),
                   (dispatch, fwd, "SQ_INSTS_VALU", 150.0),            # 125 other than MFMA: 5.0 per MFMA
                   (dispatch, fwd, "SQ_INSTS_LDS", 50.0),              # 2.0 per MFMA
                   (dispatch, fwd, "SQ_INSTS_SALU", 75.0)]             # 3.0 per MFMA
    counters = rocprof_issue.read_counters([_write(tmp_path / "a", rows_a), _write(tmp_path / "b", rows_b)])
    assert counters["attn_fwd_kernel"]["SQ_WAVE_CYCLES"] == pytest.approx(1000.0)  # mean over the dispatches
    lines = rocprof_issue.summarize(counters)
    assert len(lines) == 2  # header + the one kernel present
    cells = lines[1].replace("|", " ").replace(",", " ").split()
    assert cells[0] == "attn_fwd_kernel"
    shares = [float(c.rstrip("%")) for c in cells[1:6]]
    # VALU share: 1200 cycles scaled by the non-MFMA fraction of the VALU instructions (125 / 150) = 1000 = 50 %
    assert shares == pytest.approx([40.0, 50.0, 10.0, 40.0, 10.0])
    assert [float(c) for c in cells[6:9]] == pytest.approx([5.0, 2.0, 3.0])


def test_issue_summary_skips_kernels_without_counters():
    assert len(rocprof_issue.summarize({"attn_dq_kernel": {"SQ_INSTS_MFMA": 1.0}})) == 1
