"""The size-halving sweep in the shape of the reference's ``__main__`` benchmarks
(triton_reduce_scatter.py:213-240): its line format on the CPU, the sweep itself on the GPU."""
import os
import subprocess
import sys

import pytest

from tccl_amd import harness

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_line_format_round_trip():
    assert harness.parse_line("tccl_amd 4096 0.681 GB/s  (HBM 5.4 GB/s, 6.0 us)") == ("tccl_amd", 4096, 0.681)
    assert harness.parse_line("torch 536870912 123.456 GB/s  (4348.7 us)") == ("torch", 536870912, 123.456)
    assert harness.parse_line("expired waits: 0") is None
    assert harness.parse_line("") is None


def test_plot_from_lines(tmp_path):
    pytest.importorskip("matplotlib")
    lines = [f"tccl_amd {2048 << i} {1.5 * (i + 1):.3f} GB/s  (x)" for i in range(8)]
    lines += [f"torch {2048 << i} {0.5 * (i + 1):.3f} GB/s  (x)" for i in range(8)]
    out = tmp_path / "curve.png"
    harness.plot(lines, str(out), "test")
    assert out.stat().st_size > 2000
    assert out.read_bytes()[:8] == b"\x89PNG\r\n\x1a\n"


@pytest.mark.gpu
@pytest.mark.parametrize("op", ["all_reduce", "reduce_scatter", "all_gather", "double_tree", "double_tree_pipelined",
                                "two_shot_world"])
def test_sweep_runs_and_prints_the_reference_columns(op, tmp_path):
    """``python -m tccl_amd.harness <op>``: every line is ``name bytes rate``, sizes halve from
    the maximum down to 2,048 elements, rates are finite and positive; with --compare there is a
    torch line per size, and --plot writes a picture."""
    png = tmp_path / f"{op}.png"
    cmd = [sys.executable, "-m", "tccl_amd.harness", op, "--max-elems", str(1 << 20), "--compare", "--plot", str(png)]
    proc = subprocess.run(cmd, cwd=ROOT, capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    recs = [harness.parse_line(ln) for ln in proc.stdout.splitlines()]
    ours = [r for r in recs if r and r[0] == "tccl_amd"]
    theirs = [r for r in recs if r and r[0] == "torch"]
    assert len(ours) == 10                                     # 2^20 ... 2^11 elements
    assert [r[1] for r in ours] == sorted((r[1] for r in ours), reverse=True)
    assert ours[0][1] == 2 * (1 << 20) and ours[-1][1] == 2 * 2048
    assert all(0 < r[2] < 1e5 for r in ours)
    if op in ("all_reduce", "reduce_scatter", "all_gather"):
        assert [r[1] for r in theirs] == [r[1] for r in ours]
        assert all(0 < r[2] < 1e5 for r in theirs)
    if op in ("double_tree_pipelined", "two_shot_world"):
        assert "expired waits: 0" in proc.stdout
    assert png.exists() and png.read_bytes()[:4] == b"\x89PNG"


@pytest.mark.gpu
def test_bench_prints_a_stamp_table_for_one_operation():
    """``python bench.py --only c1 --stamps``: the measurement build of the library (every kernel with
    per-workgroup time stamps) loads, runs the operation through the same entry points, and the table
    it prints holds the 512 workgroups of the W=8 x 8 MiB launch with times that make sense."""
    cmd = [sys.executable, os.path.join(ROOT, "bench.py"), "--only", "c1", "--stamps", "--steps", "3", "--warmup", "8"]
    proc = subprocess.run(cmd, cwd=ROOT, capture_output=True, text=True, timeout=150)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    out = proc.stdout
    assert "512 workgroups stamped" in out and "last store acked" in out
    rows = [ln.split() for ln in out.splitlines() if ln.startswith("all ")]
    assert len(rows) == 1
    numbers = [float(v) for v in rows[0] if v.replace(".", "").isdigit()]
    start_max, first_data, last_load, last_store = numbers[1], numbers[2], numbers[4], numbers[7]
    assert start_max < first_data < last_load < last_store < 100.0          # microseconds after the first workgroup started


@pytest.mark.gpu
@pytest.mark.parametrize("op", ["all_reduce", "reduce_scatter", "all_gather", "two_shot", "double_tree", "auto"])
def test_sweep_with_a_process_per_rank(op):
    """The same sweep started once per rank, as the reference's benchmarks are started by torchrun: 4 processes,
    every call one launch per rank; rank 0 prints the reference's columns."""
    cmd = [sys.executable, "-m", "tccl_amd.launch", "--nproc-per-node", "4", "--module", "tccl_amd.harness", op,
           "--max-elems", str(1 << 20)]
    proc = subprocess.run(cmd, cwd=ROOT, capture_output=True, text=True, timeout=150)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    recs = [harness.parse_line(ln) for ln in proc.stdout.splitlines()]
    recs = [r for r in recs if r is not None]
    assert [r[1] for r in recs] == [2 * ((1 << 20) >> i) for i in range(10)], proc.stdout
    assert all(r[0] == "tccl_amd" and 0 < r[2] < float("inf") for r in recs)


@pytest.mark.gpu
def test_barrier_timeline_with_a_process_per_rank():
    """``benchlib/ipc_forms.py --timeline`` with 3 processes: every rank stamps the GPU's wall clock before and
    after each barrier launch; the table rank 0 prints has a line per round with one arrival per rank, the
    first of them 0, and every rank leaves a barrier after the last has arrived."""
    cmd = [sys.executable, "-m", "tccl_amd.launch", "--nproc-per-node", "3", os.path.join(ROOT, "benchlib", "ipc_forms.py"),
           "--timeline"]
    proc = subprocess.run(cmd, cwd=ROOT, capture_output=True, text=True, timeout=150)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    rows = [ln.split("|") for ln in proc.stdout.splitlines() if ln[:6].strip().isdigit()]
    assert len(rows) == 32, proc.stdout
    for _, arrivals, left, lasted in rows:
        arrivals = [float(v) for v in arrivals.split()]
        assert len(arrivals) == 3 and min(arrivals) == 0.0
        assert float(left) >= max(arrivals) and 0 < float(lasted) < 1e5
    assert "mean arrival after the round's first" in proc.stdout
