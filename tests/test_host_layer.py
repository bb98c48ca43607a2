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
def test_driver_on_synthetic(pkg, gpu, tmp_path):
    csv = tmp_path / "res.csv"
    out = subprocess.run([_exe(pkg, "spmm_test_all"), "--synthetic", "c1_citation", "1.0", "64", "--check",
                          "--csv", str(csv)], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-3000:]
    assert out.stdout.count("PASSed!!") == 3
    assert csv.read_text().startswith("c1_citation@1.0,20000,20000,101878,64,")
