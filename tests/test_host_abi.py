"""CPU-side checks of the C ABI: the library loads, exports every symbol the
header declares, its explicit host routines match the oracle and the golden
files, errors are reported as status codes, and nothing computes on the CPU in
place of the GPU."""
import ctypes as C
import re
from pathlib import Path

import numpy as np
import pytest

import block4_codec
import helpers
from oracle import partition_oracle as po

ROOT = Path(__file__).resolve().parent.parent


def declared_symbols():
    text = (ROOT / "include" / "accel_gcn.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(accel_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(pkg):
    names = declared_symbols()
    assert len(names) >= 24
    L = pkg.lib()
    for n in names:
        assert hasattr(L, n), f"{n} is declared in include/accel_gcn.h but not exported"
    assert set(names) == set(pkg._lib.SIGNATURES), "Python binding and header disagree"
    assert L.accel_version() >= 100


def test_cpp_operator_symbols_present(pkg):
    import subprocess
    out = subprocess.run(["nm", "-DC", "--defined-only", str(pkg._lib.LIB_PATH)],
                         capture_output=True, text=True, check=True).stdout
    assert "SPMM_ACCEL::do_test(bool, int)" in out
    assert "SPMM_ACCEL::run(int)" in out


@pytest.mark.parametrize("name", block4_codec.names())
def test_host_partition_reproduces_golden(pkg, name):
    golden = block4_codec.load(name)
    indptr = po.indptr_from_degrees(po.degrees_from_block4(golden))
    got = pkg.block_level_partition.partition(indptr, backend="host")
    assert got.tobytes() == golden.tobytes()


@pytest.mark.parametrize("seed", range(5))
def test_host_partition_on_unsorted_rows(pkg, seed):
    deg = helpers.degree_mix(seed=seed, n_long=6)
    indptr = po.indptr_from_degrees(deg)
    assert np.array_equal(pkg.block_level_partition.partition(indptr, backend="host"),
                          po.partition_walk(indptr))


def test_host_partition_sizing_call(pkg):
    ip = po.indptr_from_degrees([5, 5, 400])
    n = C.c_int64(-1)
    rc = pkg.lib().accel_partition_host(ip.ctypes.data_as(C.POINTER(C.c_int32)), 3, None, 0, C.byref(n))
    assert rc == 0 and n.value == 3


@pytest.mark.parametrize("seed", range(3))
def test_host_degree_sort(pkg, seed):
    deg = np.random.default_rng(seed).integers(0, 30, size=5000)
    indptr = po.indptr_from_degrees(deg)
    assert np.array_equal(pkg.block_level_partition.degree_sort(indptr), po.degree_sort(indptr))


def test_host_routines_reject_bad_input(pkg):
    L, lib = pkg.lib(), pkg._lib
    n = C.c_int64(0)
    out = np.zeros(16, dtype=np.int32)
    bad = np.array([0, 3, 2, 5], dtype=np.int32)
    p = lambda a: a.ctypes.data_as(C.POINTER(C.c_int32))
    assert L.accel_partition_host(None, 3, p(out), 4, C.byref(n)) == lib.ERR_ARG
    assert "bad argument" in lib.last_error()
    assert L.accel_partition_host(p(bad), 3, p(out), 4, C.byref(n)) == lib.ERR_CSR
    assert "decreases" in lib.last_error()
    assert L.accel_partition_host(p(np.array([1, 2], dtype=np.int32)), 1, p(out), 4, C.byref(n)) == lib.ERR_CSR
    assert L.accel_degree_sort_host(p(bad), 3, p(out)) == lib.ERR_CSR
    assert L.accel_degree_sort_host(p(bad), -1, p(out)) == lib.ERR_ARG


def test_raw_file_round_trip(pkg, tmp_path):
    blp = pkg.block_level_partition
    golden = block4_codec.load("pubmed")
    f = tmp_path / "pubmed.block4"
    blp.write_block4(f, golden)
    assert f.read_bytes() == golden.tobytes()             # raw little-endian int32, interleaved
    assert np.array_equal(blp.read_raw_i32(f).reshape(-1, 4), golden)
    with pytest.raises(pkg.AccelError) as e:
        blp.read_raw_i32(tmp_path / "missing.block4")
    assert e.value.status == pkg._lib.ERR_IO
    (tmp_path / "odd").write_bytes(b"12345")
    with pytest.raises(pkg.AccelError) as e:
        blp.read_raw_i32(tmp_path / "odd")
    assert e.value.status == pkg._lib.ERR_IO


def test_stage_writes_reference_layout_with_host_backend(pkg, tmp_path):
    """File naming and layout of the stage (block_level_partition.py:26-32,105-106)."""
    graphs = tmp_path / "graphs"
    graphs.mkdir()
    golden = block4_codec.load("arxiv")
    indptr = po.indptr_from_degrees(po.degrees_from_block4(golden))
    (graphs / "arxiv.config").write_text("")
    indptr.astype("<i4").tofile(graphs / "arxiv.new_indptr")
    done = pkg.block_level_partition.run_stage(graphs, tmp_path / "meta", backend="host", verbose=False)
    assert done == {"arxiv": golden.shape[0]}
    assert (tmp_path / "meta" / "arxiv.block4").read_bytes() == golden.tobytes()


def test_operator_argument_errors_need_no_gpu(pkg):
    L, lib = pkg.lib(), pkg._lib
    h = C.c_void_p()
    ip = np.array([0, 1], dtype=np.int32)
    assert L.accel_create(None, None, None, 1, 1, 1, 0, C.byref(h)) == lib.ERR_ARG
    assert L.accel_create(ip.ctypes.data, None, None, 1, 1, 1, 0, C.byref(h)) == lib.ERR_ARG
    assert L.accel_create(ip.ctypes.data, ip.ctypes.data, ip.ctypes.data, -1, 1, 1, 0, C.byref(h)) == lib.ERR_ARG
    assert L.accel_create(ip.ctypes.data, ip.ctypes.data, ip.ctypes.data, 1, 1, 1, 7, C.byref(h)) == lib.ERR_ARG
    assert L.accel_run(None, None, None, 4, None) == lib.ERR_ARG
    assert L.accel_preprocess(None) == lib.ERR_ARG
    assert L.accel_destroy(None) == lib.OK


def test_no_cpu_fallback_without_a_gpu(pkg):
    """Where there is no device, every GPU entry point must say so."""
    if pkg.device_count() > 0:
        pytest.skip("a GPU is present")
    lib = pkg._lib
    g = helpers.graph_from_degrees([1, 2, 3], n_cols=8)
    with pytest.raises(pkg.AccelError) as e:
        pkg.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols)
    assert e.value.status == lib.ERR_HIP and "no CPU fallback" in e.value.message
    with pytest.raises(pkg.AccelError) as e:
        pkg.block_level_partition.partition(g.indptr, backend="gpu")
    assert e.value.status == lib.ERR_HIP
    with pytest.raises(pkg.AccelError):
        pkg.DeviceBuffer(16)


def test_product_does_not_import_the_oracle():
    for f in list((ROOT / "iccad-accel-gcn_amd").rglob("*.py")) + list((ROOT / "iccad-accel-gcn_amd" / "csrc").iterdir()):
        if f.is_file():
            text = f.read_text(errors="ignore")
            assert "oracle" not in text.lower(), f"{f} mentions the oracle"


def test_binding_refuses_host_arrays_as_dense_operands(pkg):
    """run/run_epilogue/time take device memory; a numpy array (a host address) or an
    object that says it is too small is refused before anything reaches the library."""
    L = pkg._lib
    with pytest.raises(pkg.AccelError) as e:
        L.dev_ptr(np.zeros(8, np.float32), 32, "X")
    assert e.value.status == L.ERR_ARG and "host" in e.value.message

    class FakeTensor:
        def __init__(self, n, cuda):
            self.n, self.is_cuda = n, cuda
        def data_ptr(self):
            return 0x1000
        def numel(self):
            return self.n
        def element_size(self):
            return 4

    with pytest.raises(pkg.AccelError):
        L.dev_ptr(FakeTensor(8, False), 32, "X")          # a CPU tensor
    with pytest.raises(pkg.AccelError):
        L.dev_ptr(FakeTensor(7, True), 32, "Y")           # too small
    assert L.dev_ptr(FakeTensor(8, True), 32, "Y").value == 0x1000
    assert L.dev_ptr(None, 4, "bias") is None
    assert L.dev_ptr(0x2000, 1 << 40, "X").value == 0x2000  # raw addresses are the library's to check


def test_upstream_shaped_caller_compiles_against_the_headers(pkg, tmp_path):
    """A driver with the shape of upstream's main.cu (`string` named before its own
    using-directive, main.cu:10,16; the readers of data.h; the nine-argument constructor,
    main.cu:131; do_test(false/true, dim), main.cu:146,166; the host-clock helpers of
    util.h) builds against include/ alone and links against the library."""
    import shutil
    import subprocess
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    src = ROOT / "tests" / "cases" / "upstream_shaped_caller.cpp"
    lib_dir = Path(pkg._lib.LIB_PATH).parent
    exe = tmp_path / "caller"
    r = subprocess.run([hipcc, "-x", "hip", "--offload-arch=gfx950", "-std=c++17", "-Wno-unused-value",
                        f"-I{ROOT / 'include'}", str(src), "-o", str(exe), f"-L{lib_dir}", "-laccelgcn"],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert exe.exists()
