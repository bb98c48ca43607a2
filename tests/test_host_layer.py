"""The C++ host layer (hp-spmm-sddmm_amd/host): containers, loaders and the command-line driver
with the reference's entry-point shapes (test/test_all.cpp:27-109)."""
import os
import subprocess

import numpy as np
import pytest


def _exe(pkg, name):
    path = os.path.join(os.path.dirname(pkg.__file__), name)
    assert os.path.exists(path), f"{path} is missing: build with hp-spmm-sddmm_amd/build.py"
    return path


def test_host_selftest(pkg, tmp_path):
    """Readers, COO expansion/padding, reorder, CV, CSR->dense, CSV writer, host Matrix: CPU only."""
    out = subprocess.run([_exe(pkg, "spmm_host_selftest"), str(tmp_path)], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout[-2000:] + out.stderr[-2000:]
    assert "host selftest OK" in out.stdout


def test_driver_usage_error(pkg):
    out = subprocess.run([_exe(pkg, "spmm_test_all")], capture_output=True, text=True)
    assert out.returncode == 2 and "usage" in out.stderr


def _write_smtx(path, g):
    with open(path, "w") as f:
        f.write(f"{g.rows}, {g.cols}, {g.nnz}\n")
        f.write(" ".join(map(str, g.rowptr.tolist())) + " \n")
        f.write(" ".join(map(str, g.col.tolist())) + " \n")


def _parse_csv_line(line):
    parts = line.strip().split(",")
    return parts


@pytest.mark.gpu
@pytest.mark.parametrize("k", [32, 64, 128])
def test_driver_on_smtx_with_reorder(pkg, gpu, tmp_path, k):
    """argv = <graph.smtx> <graph.reorder> <K>, checked against rocSPARSE at the reference's 0.1 bar."""
    g = pkg.graphs.make_graph("c4_rmat", 0.002)
    smtx = tmp_path / "g.smtx"
    _write_smtx(smtx, g)
    order = np.argsort(-np.diff(g.rowptr), kind="stable")  # a degree-sorted processing order
    (tmp_path / "g.reorder").write_text(" ".join(map(str, order.tolist())) + "\n")
    csv = tmp_path / "res.csv"
    out = subprocess.run([_exe(pkg, "spmm_test_all"), str(smtx), str(tmp_path / "g.reorder"), str(k),
                          "--check", "--csv", str(csv)], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-3000:]
    assert out.stdout.count("PASSed!!") == 3, out.stdout[-3000:]
    line = csv.read_text().strip().splitlines()[-1]
    assert line.startswith(f"{smtx},{g.rows},{g.cols},{g.nnz},{k},")
    assert "GE-SpMM: ," in line and "HP-SpMM ," in line
    ge = line.split("GE-SpMM: ,")[1].split(",")
    assert float(ge[0]) > 0 and float(ge[1]) > 0  # ms and GFLOPS of the CSR entry point


@pytest.mark.gpu
@pytest.mark.parametrize("k", [32, 128])
def test_driver_results_against_oracle(pkg, oracle, gpu, tmp_path, k):
    """The driver's own outputs (--dump-c) for a .smtx + reorder input against the CPU oracle at the
    1e-4 normalised bar: GESpMM, HPSpMM (values bound) and LBSpMM (the sum of its 200 accumulating
    launches).  The driver itself never links the oracle; rocSPARSE at 0.1 absolute is only its
    in-harness check."""
    g = pkg.graphs.make_graph("c4_rmat", 0.004)
    smtx = tmp_path / "g.smtx"
    _write_smtx(smtx, g)
    order = np.random.default_rng(5).permutation(g.rows)
    (tmp_path / "g.reorder").write_text(" ".join(map(str, order.tolist())) + "\n")
    prefix = tmp_path / "out"
    out = subprocess.run([_exe(pkg, "spmm_test_all"), str(smtx), str(tmp_path / "g.reorder"), str(k), "--check",
                          "--csv", str(tmp_path / "res.csv"), "--dump-c", str(prefix), "--vendor-algs", "3"],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-3000:]
    B = np.fromfile(str(prefix) + ".B.f32", dtype=np.float32).reshape(g.cols, k)
    ones = np.ones(g.nnz, dtype=np.float32)  # .smtx files carry no values
    C64, S64 = oracle.csr_spmm_f64(g.rowptr, g.col, ones, B)
    for name, div in (("gespmm", 1.0), ("hpspmm", 1.0), ("lbspmm", 200.0)):
        C = np.fromfile(f"{prefix}.{name}.f32", dtype=np.float32).reshape(g.rows, k)
        assert np.isfinite(C).all(), name
        err, pos = oracle.max_norm_err(C / np.float32(div), C64, S64)
        assert err <= 1e-4, (name, err, pos)


@pytest.mark.gpu
def test_driver_check_needs_a_comparator(pkg, gpu, tmp_path):
    """--check with every vendor algorithm switched off is an error, not a silent pass."""
    out = subprocess.run([_exe(pkg, "spmm_test_all"), "--synthetic", "c1_citation", "0.1", "32", "--check",
                          "--csv", str(tmp_path / "res.csv"), "--vendor-algs", "none"],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 3, out.stdout[-2000:] + out.stderr[-2000:]
    assert "comparator" in out.stderr


@pytest.mark.gpu
def test_driver_full_size_rmat_k128(pkg, gpu, tmp_path):
    """R-MAT scale 22 at K=128 through the C++ host layer: B and C are 2^31 bytes each, the size at
    which the reference's int byte counts overflow (copy_kernel.cu:12,30).  Matrix::to, csr_to_cuda,
    full() on the device, GESpMM / LBSpMM / HPSpMM, checked in-harness against rocSPARSE."""
    csv = tmp_path / "res.csv"
    out = subprocess.run([_exe(pkg, "spmm_test_all"), "--synthetic", "c4_rmat", "1.0", "128", "--check",
                          "--csv", str(csv), "--vendor-algs", "3"], capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-3000:]
    assert out.stdout.count("PASSed!!") == 3, out.stdout[-3000:]
    line = csv.read_text().strip().splitlines()[-1]
    assert line.startswith("c4_rmat@1.0,4194304,4194304,128313265,128,")


@pytest.mark.gpu
def test_driver_on_synthetic(pkg, gpu, tmp_path):
    csv = tmp_path / "res.csv"
    out = subprocess.run([_exe(pkg, "spmm_test_all"), "--synthetic", "c1_citation", "1.0", "64", "--check",
                          "--csv", str(csv)], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-3000:]
    assert out.stdout.count("PASSed!!") == 3
    assert csv.read_text().startswith("c1_citation@1.0,20000,20000,101878,64,")
