"""C-ABI checks that need no GPU: the library loads, exports every symbol the
header declares, and rejects bad arguments with status codes before touching a device."""
import ctypes
import re

import pytest


def _declared(header_text):
    body = re.sub(r"/\*.*?\*/", "", header_text, flags=re.S)
    return sorted(set(re.findall(r"\b(hpspmm_[a-z0-9_]+)\s*\(", body)))


def test_header_symbols_are_exported(pkg):
    capi = pkg.capi
    names = _declared(open(capi.HEADER_PATH).read())
    assert names, "no declarations found in include/hpspmm.h"
    L = ctypes.CDLL(capi.LIB_PATH)
    missing = [n for n in names if not hasattr(L, n)]
    assert not missing, f"declared but not exported: {missing}"
    assert sorted(capi.EXPORTS) == names


def test_version_and_error_string(pkg):
    L = pkg.capi.lib()
    assert L.hpspmm_version() >= 100
    assert isinstance(L.hpspmm_last_error(), bytes)


def test_argument_validation_without_device(pkg):
    capi = pkg.capi
    L = capi.lib()
    h = ctypes.c_void_p()
    fake = ctypes.c_void_p(4096)  # never dereferenced: argument checks come first
    cases = [
        ((-1, 4, 0, fake, fake, 32), capi.ERR_INVALID_ARG),
        ((4, 4, -1, fake, fake, 32), capi.ERR_INVALID_ARG),
        ((4, 4, 0, fake, fake, 0), capi.ERR_INVALID_ARG),
        ((4, 4, 0, None, fake, 32), capi.ERR_INVALID_ARG),
        ((4, 4, 3, fake, None, 32), capi.ERR_INVALID_ARG),
        ((1 << 31, 4, 0, fake, fake, 32), capi.ERR_INVALID_ARG),
        ((4, 4, 1 << 31, fake, fake, 32), capi.ERR_INVALID_ARG),
        ((4, 0, 3, fake, fake, 32), capi.ERR_INVALID_ARG),
    ]
    for (rows, cols, nnz, rp, ci, k), want in cases:
        rc = L.hpspmm_plan_create(rows, cols, nnz, rp, ci, k, 0, None, ctypes.byref(h))
        assert rc == want, (rows, cols, nnz, k, rc, L.hpspmm_last_error())
        assert L.hpspmm_last_error() != b""
        assert not h.value
    assert L.hpspmm_plan_create(4, 4, 0, fake, fake, 32, 0, None, None) == capi.ERR_INVALID_ARG
    assert L.hpspmm_csr_spmm(None, fake, fake, fake, fake, fake, None) == capi.ERR_INVALID_ARG
    assert L.hpspmm_plan_destroy(None) == capi.OK
    assert L.hpspmm_fill_f32(None, 10, 0.0, None) == capi.ERR_INVALID_ARG
    assert L.hpspmm_fill_f32(fake, -1, 0.0, None) == capi.ERR_INVALID_ARG
    assert L.hpspmm_csr_spmm_noplan(4, 4, 2, fake, fake, None, fake, 32, fake, None) == capi.ERR_INVALID_ARG
    assert L.hpspmm_coo_spmm_accumulate(4, 4, 2, fake, fake, fake, fake, -3, fake, None) == capi.ERR_INVALID_ARG
    ms = ctypes.c_float()
    assert L.hpspmm_csr_spmm_timed(None, fake, fake, fake, fake, fake, None, 0, 0, ctypes.byref(ms)) == capi.ERR_INVALID_ARG


def test_no_device_is_an_error_not_a_fallback(pkg):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    capi = pkg.capi
    h = ctypes.c_void_p()
    fake = ctypes.c_void_p(4096)
    rc = capi.lib().hpspmm_plan_create(4, 4, 0, fake, fake, 32, 0, None, ctypes.byref(h))
    assert rc == capi.ERR_NO_DEVICE
    with pytest.raises(TypeError):
        capi.Plan(4, 4, torch.zeros(5, dtype=torch.int32), torch.zeros(0, dtype=torch.int32), 32)


def test_product_does_not_import_the_oracle(pkg):
    """The shipped package and the benchmark's measured path never touch oracle/."""
    import os
    pkg_dir = os.path.dirname(pkg.__file__)
    for dirpath, _, files in os.walk(pkg_dir):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".hpp", ".h")):
                text = open(os.path.join(dirpath, f), errors="replace").read()
                assert "oracle" not in text.lower(), f"{f} mentions the oracle"


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU and says so instead of producing a figure for several."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"],
                         capture_output=True, text=True, timeout=120)
    assert out.returncode != 0
    assert "one GPU" in out.stderr and out.stdout.strip() == ""
