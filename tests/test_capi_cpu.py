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


def test_plan_options_are_validated_without_device(pkg):
    """hpspmm_plan_create_ex: a struct size that is none, values outside a field's range and flags
    that contradict each other are refused before any device is touched; the python mirror of the
    struct has the header's fields in the header's order."""
    capi = pkg.capi
    L = capi.lib()
    h = ctypes.c_void_p()
    fake = ctypes.c_void_p(4096)

    def create(**fields):
        o = capi.PlanOptions()
        o.struct_size = ctypes.sizeof(capi.PlanOptions)
        for name, value in fields.items():
            setattr(o, name, value)
        rc = L.hpspmm_plan_create_ex(ctypes.c_int64(4), ctypes.c_int64(4), ctypes.c_int64(0), fake, fake,
                                     ctypes.c_int64(32), ctypes.byref(o), None, ctypes.byref(h))
        return rc, L.hpspmm_last_error()

    for bad in ({"struct_size": 0}, {"struct_size": 6}, {"struct_size": 10},
                {"routed_tile_width": 48}, {"xcd_dealing": 3}, {"xcd_dealing": -1}, {"row_tiles_pad": 3},
                {"row_tiles_chunk_log2": 17}, {"row_tiles_chunk_log2": -2}):
        rc, msg = create(**bad)
        assert rc == capi.ERR_INVALID_ARG, (bad, rc, msg)
        assert msg != b"" and not h.value
    # the mirror of the struct: every field the header declares, in its order
    header = open(capi.HEADER_PATH).read()
    body = header[header.index("typedef struct hpspmm_plan_options {"):header.index("} hpspmm_plan_options;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    declared = re.findall(r"\b(?:uint32_t|int32_t|const int32_t \*)\s*([a-z0-9_]+);", body)
    assert declared == [n for n, _ in capi.PlanOptions._fields_]


def test_info_structs_mirror_the_header(pkg):
    """hpspmm_plan_info and hpspmm_device_info in capi.py: the header's fields in the header's order."""
    capi = pkg.capi
    header = open(capi.HEADER_PATH).read()
    for c_name, mirror in (("hpspmm_plan_info", capi.PlanInfo), ("hpspmm_device_info", capi.DeviceInfo)):
        body = header[header.index("typedef struct %s {" % c_name):header.index("} %s;" % c_name)]
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        declared = []
        for types, names in re.findall(r"\b(int64_t|int32_t|double|char)\s+([a-z0-9_,\s\[\]]+);", body):
            declared += [n.strip().split("[")[0] for n in names.split(",")]
        assert declared == [n for n, _ in mirror._fields_], c_name


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
