"""The record bench.py prints last must stay small enough for a reader that keeps only a short tail
of stdout, and must carry the contract's keys.  No GPU: the formatter runs on a synthetic record of the
size a full run produces."""
import io
import json
import os
import sys
from contextlib import redirect_stderr, redirect_stdout

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def _synthetic_full(with_cpu=True):
    rows = []
    for _, test, metric in bench.FRAC_KEYS:
        rows.append({"test": test, "metric": metric, "value": 123456.78, "unit": "tflops", "us_per_launch": 12345.67,
                     "peak": 10100.0, "frac": 0.98765, "shape": "8192x8192x8192", "sclk_mhz": 2399.0, "watts": 1399.6,
                     "ppt_residency": 0.8741})
    # rows without a peak and rows the compact record leaves out
    rows.append({"test": "kernel_launch_latency", "metric": "roundtrip", "value": 9.47, "unit": "us", "us_per_launch": 9.47})
    for i in range(80):
        rows.append({"test": f"mfma_kind{i}", "metric": f"mfma_kind{i} distinct operands per chain", "value": 1.0,
                     "unit": "tflops", "us_per_launch": 1.0, "peak": 2500.0, "frac": 0.5})
    cpu = None
    if with_cpu:
        fig = {"ST": 12345.67, "MT": 123456.78, "unit": "GB/s", "iters_ST": 10, "iters_MT": 100}
        cpu = {"value": 516.12, "unit": "GB/s", "cores": 16, "kind": "reference", "pinned_workers": 16,
               "sample": "x" * 600, "reference": {"isa": "avx512", "global_memory_bandwidth read": fig,
                                                  "single_precision_compute float": fig},
               "port": {"global_memory_bandwidth float4": fig, **{f"family {i}": fig for i in range(20)}}}
    return {"metric": "MFMA TFLOPS/TOPS per dtype (dense, 2:4) + HBM GB/s, as % of MI355X peak",
            "value": 7457.12, "unit": "GB/s", "n_gpus": 1, "steps": 300, "warmup": 100, "ms_per_step": 0.57612,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": "w" * 200, "buffer_bytes": 1 << 32, "threads": 65536, "pct_of_peak": 93.21},
            "roofline": {"bound": "hbm", "achieved": 7444.11, "peak": 8000.0, "unit": "GB/s", "frac": 0.9305,
                         "traffic": 4295176192, "kernel_us": 576.95, "algorithmic_bytes": 1 << 32},
            "cpu_baseline": cpu, "rows": rows, "rows_file": "some/dir/bench_rows.json"}


def test_compact_line_is_small_and_complete():
    full = _synthetic_full()
    text = json.dumps(bench.compact_line(full), separators=(",", ":"))
    assert len(text.encode()) < 2000, len(text)
    line = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "fracs"):
        assert key in line, key
    assert line["config"]["workload"] and "model" not in line["config"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel_us", "algorithmic_bytes"):
        assert key in line["roofline"], key
    for key in ("value", "unit", "cores", "kind", "sample", "ST", "MT"):
        assert key in line["cpu_baseline"], key
    for key in ("mfma_fp16", "mfma_bf16", "mfma_fp8", "mfma_mxfp4", "mfma_int8", "smfmac_fp16", "smfmac_int8",
                "gemm_bf16_seeded"):
        assert key in line["fracs"], key
    assert line["launch_roundtrip_us"] == 9.47
    assert line["mfma_operands"] == "one set per wave"
    assert line["below_target_mhz_w"] == {}          # every synthetic row is above its target


def test_compact_line_names_the_held_clock_of_rows_below_target():
    full = _synthetic_full()
    for r in full["rows"]:
        r["frac"] = 0.5                    # everything below target: the largest the record can get
    text = json.dumps(bench.compact_line(full), separators=(",", ":"))
    assert len(text.encode()) < 2000, len(text)
    held = json.loads(text)["below_target_mhz_w"]
    assert held["smfmac_fp16"] == [2399, 1400] and held["mfma_fp16_32x32x16"] == [2399, 1400] and len(held) == 16
    assert [k for k in held if not k.startswith(("mfma", "smfmac"))] == ["gemm_bf16_seeded"]


def test_emit_prints_the_compact_record_last(tmp_path):
    full = _synthetic_full(with_cpu=False)
    out, err = io.StringIO(), io.StringIO()
    rows_file = tmp_path / "rows.json"
    with redirect_stdout(out), redirect_stderr(err):
        bench.emit(full, str(rows_file))
    lines = out.getvalue().splitlines()
    assert len(lines) == 1 and len(lines[-1].encode()) < 2000
    assert json.loads(lines[-1])["cpu_baseline"] is None
    # the full record, every row of it, is in the file; the rows are listed for a human on stderr
    assert len(json.loads(rows_file.read_text())["rows"]) == len(full["rows"])
    assert err.getvalue().count("\n") == len(full["rows"])


def test_traffic_figure_is_the_committed_profile():
    """`roofline.traffic` is a measured figure carried as a constant: it must be the one the committed counter
    summary derives, so that a changed kernel with a stale profile (or the other way round) fails here."""
    import re
    text = open(os.path.join(ROOT, "profiles", "hbm_float4_read_4GiB_traffic.md")).read()
    m = re.search(r"=\s*\*\*(\d+) bytes\*\*", text)
    assert m, "no scaled traffic figure in the profile"
    assert int(m.group(1)) == bench.TRAFFIC_BYTES_PER_LAUNCH
    # and the figure follows from the table's own rows: each counter (KiB per dispatch) scaled by what it reads for the
    # copy kernel of known size (1 GiB each way)
    kib = {(k, c): float(v) for k, c, v in re.findall(r"\| (copy_kernel|global_bandwidth_kernel<float4, 6>)[^|]*\| (FETCH_SIZE|WRITE_SIZE) \| \d+ \| ([\d.]+) \|", text)}
    read = kib[("global_bandwidth_kernel<float4, 6>", "FETCH_SIZE")] * (1048576.0 / kib[("copy_kernel", "FETCH_SIZE")]) * 1024
    written = kib[("global_bandwidth_kernel<float4, 6>", "WRITE_SIZE")] * (1048576.0 / kib[("copy_kernel", "WRITE_SIZE")]) * 1024
    assert abs(read + written - bench.TRAFFIC_BYTES_PER_LAUNCH) <= 64        # the table prints two decimals of a KiB
    assert 0.999 <= (1 << 32) / bench.TRAFFIC_BYTES_PER_LAUNCH <= 1.0         # the read kernel fetches what it must and no more
    # the profile names the grid it measured; it is the grid the headline launches
    assert "65536 threads" in text and bench.HEADLINE_BLOCKS_PER_CU * 256 * 256 == 65536


def test_headline_grid_is_the_parity_tested_one():
    """One 256-thread workgroup per CU: bench.py's headline launch, the host layer's default, and the grid the
    4 GiB GPU parity test runs first."""
    assert bench.HEADLINE_BLOCKS_PER_CU == 1
    header = open(os.path.join(ROOT, "clpeak_amd", "host", "mi355_peak.h")).read()
    assert "bwBlocksPerCU = 1;" in header
    gpu_test = open(os.path.join(ROOT, "tests", "test_gpu_basic.py")).read()
    assert "for blocks_per_cu in (1, 8):" in gpu_test


def test_metrics_table_fields_are_read_where_the_driver_puts_them(tmp_path):
    """bench.py reads the driver's metrics table (gpu_metrics, format 1.8) at fixed offsets: a table built here with known
    values in those places must come back as those values, a table of another revision as None, and the difference of two
    snapshots as residencies (share of the accumulation cycles) and mean power (energy counter over firmware time)."""
    import struct

    def table(rev, energy_units, acc, residencies, fw_ticks, clocks):
        b = bytearray(3872)
        struct.pack_into("<HBB", b, 0, 3872, 1, rev)
        struct.pack_into("<Q", b, 24, energy_units)
        struct.pack_into("<I", b, 40, acc)
        struct.pack_into("<5I", b, 44, *residencies)
        struct.pack_into("<Q", b, 288, fw_ticks)
        struct.pack_into("<8H", b, 296, *clocks)
        return bytes(b)

    tel = bench._Telemetry.__new__(bench._Telemetry)
    path = tmp_path / "gpu_metrics"
    tel.metrics = str(path)
    path.write_bytes(table(8, 1_000_000, 0xfffffff0, (0, 0xffffff00, 3, 4, 5), 10_000_000_000, range(1700, 1708)))
    a = tel.snapshot()
    assert a["acc"] == 0xfffffff0 and a["ppt"] == 0xffffff00 and a["prochot"] == 0 and a["hbm_thm"] == 5
    assert a["gfxclk"] == list(range(1700, 1708)) and abs(a["fw_s"] - 100.0) < 1e-9 and abs(a["energy_j"] - 15.259) < 1e-6
    # two seconds later: 2000 accumulation cycles (the 32-bit counters wrap), the package limiter active in 500 of them, 2800 J
    units = 1_000_000 + int(round(2800.0 / 15.259e-6))
    path.write_bytes(table(8, units, (0xfffffff0 + 2000) & 0xffffffff, (0, (0xffffff00 + 500) & 0xffffffff, 3, 4, 5),
                           10_000_000_000 + 200_000_000, range(1800, 1808)))
    d = bench._Telemetry.between(a, tel.snapshot())
    assert d["ppt_residency"] == 0.25 and d["prochot_residency"] == 0.0 and d["socket_thm_residency"] == 0.0
    assert abs(d["watts_energy_counter"] - 1400.0) < 0.2 and d["gfxclk_mhz_per_xcd"] == list(range(1800, 1808))
    path.write_bytes(table(7, 1, 2, (3, 4, 5, 6, 7), 8, range(8)))
    assert tel.snapshot() is None                      # another revision: other offsets, not guessed at
    assert bench._Telemetry.between(a, None) == {}
    tel.metrics = str(tmp_path / "absent")
    assert tel.snapshot() is None


def test_every_name_the_gpu_only_code_uses_exists():
    """Most of bench.py, the C-ABI mirror and the smoke test run only on a GPU box; a name that a function reads and
    nothing defines (a line lost in an edit) would show there at the earliest, in a child process perhaps not at all.
    Every name a function takes from the module must be bound at module level or be a builtin."""
    import builtins
    import symtable
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for rel in ("bench.py", "__graft_entry__.py", os.path.join("clpeak_amd", "capi.py"), os.path.join("clpeak_amd", "workloads.py"),
                os.path.join("tests", "vendor_parity_child.py")):
        path = os.path.join(root, rel)
        top = symtable.symtable(open(path).read(), path, "exec")
        bound = {s.get_name() for s in top.get_symbols() if s.is_assigned() or s.is_imported() or s.is_namespace()} | {"__file__", "__name__"}
        missing = []

        def walk(table):
            for child in table.get_children():
                for s in child.get_symbols():
                    if s.is_referenced() and s.is_global() and not s.is_assigned() and s.get_name() not in bound \
                            and not hasattr(builtins, s.get_name()):
                        missing.append((child.get_name(), s.get_name()))
                walk(child)
        walk(top)
        assert missing == [], (rel, missing)
