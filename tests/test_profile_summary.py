"""Host-only checks of the rocprofv3 CSV condenser (dscuda_amd/harness/profile_summary.py):
the figures quoted from profiles/ come out of it, so its arithmetic is pinned on
small hand-made files whose answers can be read off."""

import csv

from dscuda_amd.harness import profile_summary

KERNEL = "void dscuda::(anonymous namespace)::attention_forward_pingpong_kernel<192, 128>(float*, int)"


def write_counters(path, rows):
    fields = ["Kernel_Name", "Counter_Name", "Counter_Value", "Start_Timestamp", "End_Timestamp"]
    with open(path, "w", newline="") as handle:
        writer = csv.DictWriter(handle, fieldnames=fields)
        writer.writeheader()
        for row in rows:
            writer.writerow(dict(zip(fields, row)))


def test_short_name_strips_namespaces_and_arguments():
    assert profile_summary.short_name(KERNEL) == "attention_forward_pingpong_kernel<192, 128>"


def test_counter_means_durations_and_clock(tmp_path):
    # 10 launches: the first five take 800 us at 1.5 GHz, the last five 600 us at 2.0 GHz;
    # GRBM_GUI_ACTIVE is summed over 8 dies
    rows = []
    for launch in range(10):
        duration = 800_000 if launch < 5 else 600_000
        clock = 1.5 if launch < 5 else 2.0
        start = 1_000_000_000 + launch * 1_000_000
        rows.append((KERNEL, "GRBM_GUI_ACTIVE", 8 * clock * duration, start, start + duration))
    rows.append(("void other_kernel(int)", "GRBM_GUI_ACTIVE", 1.0, 0, 10))
    path = tmp_path / "t_counter_collection.csv"
    write_counters(path, rows)
    lines = profile_summary.counter_averages(path, ["dscuda"])
    text = "\n".join(lines)
    assert "other_kernel" not in text
    assert lines[0] == "attention_forward_pingpong_kernel<192, 128>"
    assert "(mean of 10 dispatches)" in lines[1]
    mean_cycles = (5 * 8 * 1.5 * 800_000 + 5 * 8 * 2.0 * 600_000) / 10
    assert f"{mean_cycles:18.1f}" in lines[1]
    assert "first 5 launches 800.0 us, second half (5 launches) 600.0 us" in text
    assert "first launches 1.50 GHz, second half 2.00 GHz" in text


def test_few_dispatches_report_one_mean_duration(tmp_path):
    rows = [(KERNEL, "FETCH_SIZE", 100.0 + launch, 0, 2_000 * (launch + 1)) for launch in range(3)]
    path = tmp_path / "x_counter_collection.csv"
    write_counters(path, rows)
    lines = profile_summary.counter_averages(path, [])
    assert "FETCH_SIZE" in lines[1] and f"{101.0:18.1f}" in lines[1]
    assert lines[-1].strip() == "dispatch duration: 4.0 us (mean of 3)"


def test_kernel_stats_table(tmp_path):
    path = tmp_path / "t_kernel_stats.csv"
    with open(path, "w", newline="") as handle:
        writer = csv.DictWriter(handle, fieldnames=["Name", "Calls", "AverageNs", "MinNs", "MaxNs", "Percentage"])
        writer.writeheader()
        writer.writerow({"Name": KERNEL, "Calls": 4, "AverageNs": 650_000, "MinNs": 640_000, "MaxNs": 700_000,
                         "Percentage": 91.5})
        writer.writerow({"Name": "void unrelated(int)", "Calls": 1, "AverageNs": 1, "MinNs": 1, "MaxNs": 1,
                         "Percentage": 0.1})
    lines = profile_summary.kernel_stats(path, ["dscuda"])
    assert len(lines) == 2
    assert lines[1].split()[-5:] == ["4", "650.0", "640.0", "700.0", "91.50"]


def test_bench_reads_the_committed_forward_profile():
    """bench.py takes roofline.traffic and profiled_kernel_ms from the forward's summary under profiles/: the line
    it wants is the machine-readable one, not one of the counter lines that start with the same kernel name."""
    import bench
    traffic, microseconds = bench.profiled_figures("mla_prefill_forward_S4096_H128", "attention_forward_pingpong_kernel")
    assert traffic is not None and 5e8 < traffic < 1e10
    assert microseconds is not None and 300.0 < microseconds < 2000.0
    assert bench.profiled_figures("no_such_case", "attention_forward_pingpong_kernel") == (None, None)
