"""The two text-table tools that turn rocprofv3 CSV output into what profiles/ holds, on small synthetic inputs."""
import importlib.util
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent


def load(name):
    spec = importlib.util.spec_from_file_location(name, ROOT / "gemm-zoo_amd" / "bench" / f"{name}.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def run_main(mod, argv, capsys):
    old = sys.argv
    sys.argv = [mod.__name__] + argv
    try:
        assert mod.main() == 0
    finally:
        sys.argv = old
    return capsys.readouterr().out


def test_pmc_table_means_and_levels(tmp_path, capsys):
    d = tmp_path / "run"
    d.mkdir()
    rows = ["Kernel_Name,Counter_Name,Counter_Value"]
    rows += [f"kern_a,FETCH_SIZE,{v}" for v in (100, 101, 200, 202, 201)]
    rows += ["kern_a,WRITE_SIZE,50", "fill_kernel,FETCH_SIZE,7"]
    (d / "x_counter_collection.csv").write_text("\n".join(rows) + "\n")
    out = run_main(load("pmc_table"), [str(d), "--levels"], capsys)
    assert "kern_a" in out and "fill_kernel" not in out            # the default --skip list
    line = next(l for l in out.splitlines() if "FETCH_SIZE" in l)
    assert "161" in line and "min 100" in line and "max 202" in line and "(5 dispatches)" in line
    levels = [l.split() for l in out.splitlines() if l.strip().startswith("level")]
    assert [(float(l[1].replace(",", "")), int(l[3])) for l in levels] == [(100.5, 2), (201.0, 3)]
    out = run_main(load("pmc_table"), [str(d), "--skip", ""], capsys)
    assert "fill_kernel" in out


def test_trace_table_cuts_runs_and_windows(tmp_path, capsys):
    d = tmp_path / "trace"
    d.mkdir()
    rows = ["Kernel_Name,Start_Timestamp,End_Timestamp"]
    t = 0
    def add(name, n, dur):
        nonlocal t
        for _ in range(n):
            rows.append(f"{name},{t},{t + dur}")
            t += dur + 10
    add("kern_a", 6, 1000)          # first leg: 1 us each
    add("gz::fill_kernel", 1, 50)   # does not end a run
    add("kern_a", 4, 1000)
    add("kern_b", 3, 5000)
    add("kern_a", 5, 3000)          # second leg of kern_a: 3 us each
    (d / "x_kernel_trace.csv").write_text("\n".join(rows) + "\n")
    out = run_main(load("trace_table"), [str(d), "--min-run", "3", "--window", "1:4"], capsys)
    lines = [l for l in out.splitlines() if l.strip()]
    assert len(lines) == 3
    assert lines[0].startswith("kern_a") and " 10  mean      1.00" in lines[0] and "mean      1.00 over 3" in lines[0]
    assert lines[1].startswith("kern_b") and "  3  mean      5.00" in lines[1]
    assert lines[2].startswith("kern_a") and "  5  mean      3.00" in lines[2]
