"""Host-side checks of the rocprofv3 capture driver: the extraction arithmetic on synthetic rocprofv3 CSV
files (calibration by the copy case, settled durations, matrix-pipe utilisation and clock from the counters),
the pass definitions against the hardware's counter-block limits, and the raw-dump comparator."""

import csv

import numpy as np

from dscuda_amd.profiler import capture, compare_dumps

TRACE_HEADER = ["Kind", "Agent_Id", "Queue_Id", "Stream_Id", "Thread_Id", "Dispatch_Id", "Kernel_Id", "Kernel_Name",
                "Correlation_Id", "Start_Timestamp", "End_Timestamp", "LDS_Block_Size", "Scratch_Size", "VGPR_Count",
                "Accum_VGPR_Count", "SGPR_Count", "Workgroup_Size_X", "Workgroup_Size_Y", "Workgroup_Size_Z",
                "Grid_Size_X", "Grid_Size_Y", "Grid_Size_Z"]
COUNTER_HEADER = ["Correlation_Id", "Dispatch_Id", "Agent_Id", "Queue_Id", "Process_Id", "Thread_Id", "Grid_Size",
                  "Kernel_Id", "Kernel_Name", "Workgroup_Size", "LDS_Block_Size", "Scratch_Size", "VGPR_Count",
                  "Accum_VGPR_Count", "SGPR_Count", "Counter_Name", "Counter_Value", "Start_Timestamp", "End_Timestamp"]
KERNEL = "void dscuda::(anonymous namespace)::attention_forward_pingpong_kernel<192, 128>(__hip_bfloat16*, float*)"


def _write(path, header, rows):
    path.parent.mkdir(parents=True, exist_ok=True)
    with open(path, "w", newline="") as handle:
        writer = csv.writer(handle, quoting=csv.QUOTE_NONNUMERIC)
        writer.writerow(header)
        writer.writerows(rows)


def _trace_rows(name, durations_ns):
    rows, clock = [], 1000
    for index, duration in enumerate(durations_ns):
        rows.append(["KERNEL_DISPATCH", "Agent 1", 1, 0, 7, index + 1, 5, name, index + 1, clock, clock + duration,
                     155648, 0, 219, 0, 96, 512, 1, 1, 131072, 1, 1])
        clock += duration + 10
    return rows


def _counter_rows(name, counter, values, duration_ns):
    rows, clock = [], 5000
    for index, value in enumerate(values):
        rows.append([index + 1, index + 1, "Agent 1", 1, 9, 9, 131072, 5, name, 512, 155648, 0, 219, 0, 96, counter,
                     float(value), clock, clock + duration_ns])
        clock += duration_ns + 10
    return rows


def test_extraction_on_synthetic_rocprof_output(tmp_path):
    out, profiles = tmp_path / "out", tmp_path / "profiles"
    copy = "__amd_rocclr_copyBuffer"
    # calibration: the 1 GiB copy reads as 524288 KiB fetched (factor 2) and 1048576 KiB written (factor 1)
    _write(out / "copy_1GiB" / "fetch" / "x_counter_collection.csv", COUNTER_HEADER,
           _counter_rows(copy, "FETCH_SIZE", [524288.0] * 6, 400000))
    _write(out / "copy_1GiB" / "write" / "x_counter_collection.csv", COUNTER_HEADER,
           _counter_rows(copy, "WRITE_SIZE", [1048576.0] * 6, 400000))
    _write(out / "copy_1GiB" / "time" / "x_kernel_trace.csv", TRACE_HEADER, _trace_rows(copy, [400000] * 6))
    stem = "mla_prefill_forward_S4096_H128"
    # eight launches: four cold at 760 us, four settled at 640 us
    _write(out / stem / "time" / "x_kernel_trace.csv", TRACE_HEADER, _trace_rows(KERNEL, [760000] * 4 + [640000] * 4))
    _write(out / stem / "fetch" / "x_counter_collection.csv", COUNTER_HEADER,
           _counter_rows(KERNEL, "FETCH_SIZE", [500000.0] * 4, 640000))
    _write(out / stem / "write" / "x_counter_collection.csv", COUNTER_HEADER,
           _counter_rows(KERNEL, "WRITE_SIZE", [200000.0] * 4, 640000))
    # counter pass: 620 us at 2.0 GHz -> 1.24e6 cycles per die, matrix pipe busy 50 %
    cycles = 620e-6 * 2.0e9
    rows = (_counter_rows(KERNEL, "GRBM_GUI_ACTIVE", [cycles * 8] * 4, 620000) +
            _counter_rows(KERNEL, "SQ_VALU_MFMA_BUSY_CYCLES", [0.5 * cycles * 1024] * 4, 620000) +
            _counter_rows(KERNEL, "SQ_LDS_BANK_CONFLICT", [0.0] * 4, 620000))
    _write(out / stem / "mfma" / "x_counter_collection.csv", COUNTER_HEADER, rows)

    capture.main(["metric", "quick", "extract", "--out", str(out), "--profiles", str(profiles), "--only", stem])

    factors = capture.calibration(out)
    assert abs(factors[0] - 2.0) < 1e-9 and abs(factors[1] - 1.0) < 1e-9
    row, = capture.extract_case(next(c for c in capture.metric_cases("quick") if c.stem == stem), out, factors)
    assert row["kernel"] == "attention_forward_pingpong_kernel<192, 128>"
    assert row["launches"] == 8 and abs(row["time_us"] - 640.0) < 1e-9 and abs(row["first_us"] - 736.0) < 1e-9
    assert abs(row["read_mb"] - 500000 * 2 * 1024 / 1e6) < 1e-6 and abs(row["write_mb"] - 200000 * 1024 / 1e6) < 1e-6
    assert abs(row["mfma_pct"] - 50.0) < 1e-6 and abs(row["clock_ghz"] - 2.0) < 1e-6
    assert (row["vgpr"], row["scratch"], row["lds"]) == (438, 0, 155648)   # VGPR_Count is in units of two
    text = (profiles / f"{stem}.md").read_text()
    assert "attention_forward_pingpong_kernel<192, 128> :: time_us = 640.000 ; fabric_bytes = 1228800000" in text
    assert (profiles / "capture_metric.md").is_file()


def test_counter_passes_fit_the_counter_blocks():
    limits = {"SQ_": 8, "TCC_": 4, "TCP_": 4, "TA_": 2, "TD_": 2, "GRBM_": 2}
    derived = {"FETCH_SIZE": ("TCC_", 3), "WRITE_SIZE": ("TCC_", 2)}
    for name, arguments in capture.PASSES.items():
        if "--pmc" not in arguments:
            assert "--kernel-trace" in arguments
            continue
        # a counter pass never carries a trace domain next to --pmc
        assert not any(flag in arguments for flag in ("--kernel-trace", "--stats", "--sys-trace", "--hip-trace"))
        used = dict.fromkeys(limits, 0)
        for counter in arguments[1:]:
            if counter in derived:
                block, count = derived[counter]
                used[block] += count
            else:
                block = next(prefix for prefix in limits if counter.startswith(prefix))
                used[block] += 1
        for block, count in used.items():
            assert count <= limits[block], (name, block, count)


def test_program_follows_the_separator_directly():
    for family in capture.FAMILIES.values():
        for case in [capture.copy_case()] + family("full"):
            command = capture.rocprof_command("fetch", "/tmp/x", case.counter_command)
            program = command[command.index("--") + 1]
            assert program.endswith(("python3", "python")) or "/build/benchmark_" in program, program


def test_dump_comparator(tmp_path):
    generator = np.random.default_rng(0)
    values = generator.standard_normal(2 * 8 * 4 * 16).astype(np.float32)
    (tmp_path / "a.bin").write_bytes(values.tobytes())
    (tmp_path / "b.bin").write_bytes((values + np.float32(1e-3)).tobytes())
    (tmp_path / "c.bin").write_bytes((values + np.float32(0.5)).tobytes())
    assert compare_dumps.main([str(tmp_path / "a.bin"), str(tmp_path / "b.bin"), "2", "8", "4", "16"]) == 0
    assert compare_dumps.main([str(tmp_path / "a.bin"), str(tmp_path / "c.bin"), "2", "8", "4", "16"]) == 1
    assert compare_dumps.main([str(tmp_path / "a.bin"), str(tmp_path / "b.bin"), "2", "8", "4", "17"]) == 2
    worst, rms, passed = compare_dumps.compare(tmp_path / "a.bin", tmp_path / "b.bin", values.size, 2.5e-2)
    assert abs(worst - 1e-3) < 1e-6 and abs(rms - 1e-3) < 1e-6 and passed
