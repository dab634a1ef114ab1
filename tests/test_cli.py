"""bin/spmm_test, the C++ harness over SPMM_ACCEL (counterpart of main.cu)."""
import re
import subprocess
from pathlib import Path

import numpy as np
import pytest

import helpers
from oracle import partition_oracle as po

ROOT = Path(__file__).resolve().parent.parent
EXE = ROOT / "iccad-accel-gcn_amd" / "bin" / "spmm_test"


def write_graph(tmp, name, seed, n_long=3):
    """<name>.config/.new_indptr/.new_indices in upstream's layout (degree-sorted
    rows, raw int32), the same matrix in its own row order as <name>.graph.ptrdump /
    .graph.edgedump (main.cu:64-65), plus the matching <name>.block4."""
    g0 = helpers.graph_from_degrees(helpers.degree_mix(seed=seed, n_long=n_long), seed=seed)
    n = g0.n_rows
    # square adjacency, as upstream assumes (vin has v_num rows)
    g0.indices[:] = g0.indices % n
    perm = po.degree_sort(g0.indptr)
    sip, six, _ = po.permute_csr(g0.indptr, g0.indices, g0.values, perm)
    graphs, meta = tmp / "graphs", tmp / "block_level_meta"
    graphs.mkdir(exist_ok=True)
    meta.mkdir(exist_ok=True)
    (graphs / f"{name}.config").write_text("")
    sip.astype("<i4").tofile(graphs / f"{name}.new_indptr")
    six.astype("<i4").tofile(graphs / f"{name}.new_indices")
    g0.indptr.astype("<i4").tofile(graphs / f"{name}.graph.ptrdump")
    g0.indices.astype("<i4").tofile(graphs / f"{name}.graph.edgedump")
    po.partition_closed_form(sip).astype("<i4").tofile(meta / f"{name}.block4")
    return graphs, meta


def test_cli_without_gpu_says_so(pkg):
    if pkg.device_count() > 0:
        pytest.skip("a GPU is present")
    assert EXE.exists(), "spmm_test was not built"
    r = subprocess.run([str(EXE), "g", "16"], capture_output=True, text=True)
    assert r.returncode == 3 and "no GPU" in r.stderr


@pytest.mark.gpu
def test_operator_error_paths(gpu):
    """bin/operator_check: a refused launch is reported by do_test and nothing more is
    launched, the operator computes again afterwards, a host pointer is refused, values
    rewritten between two calls are picked up."""
    exe = EXE.parent / "operator_check"
    assert exe.exists(), "operator_check was not built"
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count("ok:") == 5 and "FAIL" not in r.stdout


@pytest.mark.gpu
def test_cli_check_and_timing(gpu, tmp_path):
    graphs, meta = write_graph(tmp_path, "mix", seed=11)
    r = subprocess.run([str(EXE), "--graphs", str(graphs), "--meta", str(meta), "mix", "60"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "validation pass!" in r.stdout
    m = re.search(r"^0/0 mix 60 accel ([0-9.eE+-]+)$", r.stdout, re.M)    # main.cu:161-167 line format
    assert m and 0 < float(m.group(1)) < 1e6


@pytest.mark.gpu
def test_cli_refuses_stale_metadata(gpu, tmp_path):
    graphs, meta = write_graph(tmp_path, "mix", seed=12)
    b = np.fromfile(meta / "mix.block4", dtype="<i4")
    b[2] += 1
    b.tofile(meta / "mix.block4")
    r = subprocess.run([str(EXE), "--graphs", str(graphs), "--meta", str(meta), "mix", "32"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "metadata differs" in r.stderr


@pytest.mark.gpu
def test_cli_sweep_mode(gpu, tmp_path):
    for i, name in enumerate(("a", "b")):
        graphs, meta = write_graph(tmp_path, name, seed=20 + i, n_long=1)
    # sweep = every *.config, dims 16..128 (main.cu:12,195-219); without a metadata
    # directory the operator builds everything itself
    r = subprocess.run([str(EXE), "--graphs", str(graphs), "--meta", str(tmp_path / "none")],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    lines = re.findall(r"^(\d)/2 (\w) (\d+) accel ([0-9.eE+-]+)$", r.stdout, re.M)
    assert len(lines) == 2 * 113
    assert {(l[0], l[1]) for l in lines} == {("1", "a"), ("2", "b")}
    assert [int(l[2]) for l in lines[:113]] == list(range(16, 129))


@pytest.mark.gpu
def test_cli_saved_state_is_loaded_by_the_next_run(gpu, tmp_path):
    graphs, meta = write_graph(tmp_path, "mix", seed=13)
    cmd = [str(EXE), "--graphs", str(graphs), "--meta", str(meta), "--save-state", "mix", "48"]
    first = subprocess.run(cmd, capture_output=True, text=True, timeout=120)
    assert first.returncode == 0, first.stdout + first.stderr
    assert (meta / "mix.accelstate").exists() and "loaded from saved state" not in first.stderr
    second = subprocess.run(cmd, capture_output=True, text=True, timeout=120)
    assert second.returncode == 0, second.stdout + second.stderr
    assert "loaded from saved state" in second.stderr and "validation pass!" in second.stdout
    # a state that belongs to another graph is a stale cache entry: recomputed, not an error
    graphs2, meta2 = write_graph(tmp_path, "other", seed=14)
    (meta / "mix.accelstate").rename(meta2 / "other.accelstate")
    third = subprocess.run([str(EXE), "--graphs", str(graphs2), "--meta", str(meta2), "other", "48"],
                           capture_output=True, text=True, timeout=120)
    assert third.returncode == 0, third.stdout + third.stderr
    assert "loaded from saved state" not in third.stderr and "validation pass!" in third.stdout


@pytest.mark.gpu
def test_cli_natural_order_input(gpu, tmp_path):
    """--natural reads <g>.graph.ptrdump / .graph.edgedump (main.cu:64-65) and gives that CSR
    to the operator, which sorts it itself: the same validation passes through both inputs,
    and the .block4 file written for the sorted rows still describes the partition."""
    graphs, meta = write_graph(tmp_path, "mix", seed=15)
    base = [str(EXE), "--graphs", str(graphs), "--meta", str(meta)]
    for extra in ([], ["--natural"]):
        r = subprocess.run(base + extra + ["mix", "40"], capture_output=True, text=True, timeout=120)
        assert r.returncode == 0, r.stdout + r.stderr
        assert "validation pass!" in r.stdout and re.search(r"^0/0 mix 40 accel ", r.stdout, re.M)
    # unsorted input has a real permutation to save: the next run takes the order from the file
    cmd = base + ["--natural", "--save-state", "mix", "40"]
    first = subprocess.run(cmd, capture_output=True, text=True, timeout=120)
    assert first.returncode == 0 and "loaded from saved state" not in first.stderr
    assert (meta / "mix.accelstate").stat().st_size > 4 * (np.fromfile(graphs / "mix.graph.ptrdump", "<i4").size - 1)
    second = subprocess.run(cmd, capture_output=True, text=True, timeout=120)
    assert second.returncode == 0, second.stdout + second.stderr
    assert "loaded from saved state" in second.stderr and "validation pass!" in second.stdout
    # the state of the natural order does not fit the pre-sorted files: ignored, recomputed
    third = subprocess.run(base + ["--save-state", "mix", "40"], capture_output=True, text=True, timeout=120)
    assert third.returncode == 0, third.stdout + third.stderr
    assert "loaded from saved state" not in third.stderr and "validation pass!" in third.stdout
    missing = subprocess.run(base + ["--natural", "nosuch", "40"], capture_output=True, text=True, timeout=120)
    assert missing.returncode != 0


@pytest.mark.gpu
def test_upstream_shaped_driver_runs_on_a_dataset_in_upstreams_layout(gpu, tmp_path):
    """The driver of tests/cases (written like main.cu: data.h readers, `string` before its
    using-directive, the nine-argument constructor, do_test(false/true, dim), util.h's clock)
    reads ../graphs/<g>.* relative to its working directory (main.cu:10), as upstream does,
    checks the operator against a host loop and prints upstream's timing line, for the
    pre-sorted files and for the graph's own order."""
    exe = EXE.parent / "upstream_shaped_caller"
    assert exe.exists(), "upstream_shaped_caller was not built"
    graphs, meta = write_graph(tmp_path, "mix", seed=16)
    build = tmp_path / "build"
    build.mkdir()
    for extra in ([], ["natural"]):
        r = subprocess.run([str(exe), "mix", "24"] + extra, cwd=build, capture_output=True, text=True, timeout=120)
        assert r.returncode == 0, r.stdout + r.stderr
        assert "validation pass!" in r.stdout and re.search(r"^0/0 mix 24 accel [0-9.eE+-]+$", r.stdout, re.M)
    r = subprocess.run([str(exe), "nosuch", "24"], cwd=build, capture_output=True, text=True, timeout=120)
    assert r.returncode == 1 and "cannot read" in r.stdout


@pytest.mark.gpu
def test_bench_line_on_the_small_workload(gpu, tmp_path):
    """bench.py end to end on the CPU-runnable workload, with every optional section: one JSON
    line with the metric, the roofline and cpu_baseline objects, a passing parity check, the
    strided run, both comparison baselines and the dense product of the layer."""
    import json
    import sys
    r = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--workload", "cfg1", "--steps", "3", "--warmup", "2",
                        "--ld", "64", "--dense-k", "48", "--compare-rocsparse", "--compare-neighbor-partition",
                        "--cache-dir", str(tmp_path)], capture_output=True, text=True, timeout=600, cwd=str(ROOT))
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, "exactly one line on stdout"
    d = json.loads(lines[0])
    assert d["metric"].startswith("SpMM GFLOP/s") and d["unit"] == "GFLOP/s" and d["n_gpus"] == 1
    assert d["steps"] == 3 and d["warmup"] == 2 and d["dtype"] == "f32" and d["vs_baseline"] is None
    assert d["value"] > 0 and d["ms_per_step"] > 0 and "cfg1" in d["config"]["workload"]
    roof = d["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and 0 < roof["frac"] < 1
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert roof["algorithmic_bytes"] == d["config"]["nnz"] * 8 + 2 * d["config"]["rows"] * d["config"]["N"] * 4
    assert d["cpu_baseline"]["kind"] == "port" and d["cpu_baseline"]["cores"] == 1 and d["cpu_baseline"]["value"] > 0
    assert d["parity"]["ok"] and d["parity"]["rows_checked"] == d["config"]["rows"]
    assert d["config"]["strided"]["ld"] == 64 and d["config"]["strided"]["kernel_ms_avg"] > 0
    layer = d["config"]["gcn_layer"]
    assert layer["K"] == 48 and layer["dense_ok"] and layer["layer_ms"] > 0 and layer["dense_ms"] > 0
    assert d["rocsparse"]["best_ms"] > 0 and d["neighbor_partition"]["ms"] > 0
    # more than one GPU is refused with a message
    r2 = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                        timeout=120, cwd=str(ROOT))
    assert r2.returncode != 0 and "one GPU" in (r2.stdout + r2.stderr)
