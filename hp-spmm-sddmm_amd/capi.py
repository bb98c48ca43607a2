"""ctypes binding of libhpspmm.so (the C ABI declared in include/hpspmm.h).

PyTorch is used only to hold device memory and to name the stream; every
compute call goes through the C ABI into the HIP kernels.  There is no CPU or
PyTorch fallback: if the library is missing or no GPU is present the calls
raise.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libhpspmm.so")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "hpspmm.h")

OK = 0
ERR_INVALID_ARG = 1
ERR_BAD_CSR = 2
ERR_HIP = 3
ERR_NO_DEVICE = 4
ERR_ALLOC = 5

PLAN_DEFAULT = 0
PLAN_NO_VALIDATE = 1
PLAN_FORCE_ROWS = 2
PLAN_FORCE_SEGMENTS = 4
PLAN_NO_XCD_REMAP = 8
PLAN_HUB_CACHE = 16
PLAN_NO_HUB_CACHE = 32
PLAN_FORCE_ROUTED = 64
PLAN_NO_ROUTED = 128
PLAN_CLUSTER = 4096
PLAN_NO_CLUSTER = 8192
PLAN_NO_ROW_TILES = 16384
PLAN_ROUTED_SORT_VALUES = 32768
PLAN_ALLOW_MOVED_CSR = 1 << 21
PLAN_FORCE_SWEEP = 1 << 22
PLAN_NO_SWEEP = 1 << 23


def plan_hub_log2(log2_rows):
    return (int(log2_rows) & 0x1F) << 16


def plan_routed_row_log2(log2_nnz):
    return (int(log2_nnz) & 0x1F) << 24


def plan_routed_phases(n):
    return (int(n) & 0x7) << 29


def plan_segment_shift(log2_len):
    return (int(log2_len) & 0xF) << 8


class FlagsWithOptions(int):
    """A plan-flag word that carries hpspmm_plan_options fields along (Plan then goes through
    hpspmm_plan_create_ex): flags_with_options(PLAN_FORCE_ROUTED, routed_tile_width=32).  Or-ing further
    flag bits onto it keeps the options."""

    def __new__(cls, flags, options):
        self = super().__new__(cls, flags)
        self.options = dict(options)
        return self

    def __or__(self, other):
        return FlagsWithOptions(int(self) | int(other), {**getattr(other, "options", {}), **self.options})

    __ror__ = __or__


def flags_with_options(flags=0, **options):
    return FlagsWithOptions(flags, options)


STRATEGY_ROWS = 1
STRATEGY_SEGMENTS = 2
STRATEGY_GENERIC_K = 3
STRATEGY_ROUTED = 4
STRATEGY_ORDERED = 5
STRATEGY_SWEEP = 6

# every symbol include/hpspmm.h declares
EXPORTS = (
    "hpspmm_version", "hpspmm_last_error", "hpspmm_plan_create", "hpspmm_plan_get_info",
    "hpspmm_plan_destroy", "hpspmm_csr_spmm", "hpspmm_csr_spmm_noplan", "hpspmm_coo_spmm_accumulate",
    "hpspmm_fill_f32", "hpspmm_csr_spmm_timed", "hpspmm_plan_bind_values", "hpspmm_plan_create_ordered",
    "hpspmm_csr_spmm_static", "hpspmm_csr_spmm_timed_launches", "hpspmm_plan_create_ex",
    "hpspmm_static_workspace_init", "hpspmm_csr_spmm_timed_min", "hpspmm_get_device_info",
)

_i64 = ctypes.c_int64
_p = ctypes.c_void_p


class PlanInfo(ctypes.Structure):
    _fields_ = [
        ("rows", _i64), ("cols", _i64), ("nnz", _i64), ("k", _i64),
        ("strategy", ctypes.c_int32), ("segment_length", ctypes.c_int32),
        ("num_segments", _i64), ("max_row_nnz", _i64), ("empty_rows", _i64),
        ("workspace_bytes", _i64), ("launches_per_spmm", ctypes.c_int32), ("column_tiles", ctypes.c_int32),
        ("hub_rows", _i64), ("lds_served_nnz", _i64), ("row_tiles", _i64),
        ("stored_order_miss_share", ctypes.c_double),
    ]

    def as_dict(self):
        return {name: getattr(self, name) for name, _ in self._fields_}


class DeviceInfo(ctypes.Structure):
    _fields_ = [
        ("device", ctypes.c_int32), ("compute_units", ctypes.c_int32), ("clock_khz", ctypes.c_int32),
        ("memory_clock_khz", ctypes.c_int32), ("l2_bytes", _i64), ("lds_bytes_per_cu", _i64), ("global_bytes", _i64),
        ("xcd_dealing", ctypes.c_int32), ("arch", ctypes.c_char * 60),
    ]


class PlanOptions(ctypes.Structure):
    """hpspmm_plan_options (include/hpspmm.h): zero in a field = the library's default."""
    _fields_ = [
        ("struct_size", ctypes.c_uint32), ("flags", ctypes.c_uint32), ("d_row_order", ctypes.c_void_p),
        ("segment_shift", ctypes.c_int32), ("hub_log2", ctypes.c_int32), ("routed_row_log2", ctypes.c_int32),
        ("routed_phases", ctypes.c_int32), ("routed_tile_width", ctypes.c_int32),
        ("routed_split_launch", ctypes.c_int32), ("routed_lds_rows", ctypes.c_int32),
        ("xcd_dealing", ctypes.c_int32),
        ("no_column_tiles", ctypes.c_int32), ("row_tiles_min_k", ctypes.c_int32), ("row_tiles_pad", ctypes.c_int32),
        ("row_tiles_wide", ctypes.c_int32), ("row_tiles_round_robin", ctypes.c_int32),
        ("sweep_window_log2", ctypes.c_int32), ("sweep_lead", ctypes.c_int32), ("sweep_spin", ctypes.c_int32),
        ("sweep_limit", ctypes.c_int32), ("sweep_no_priorities", ctypes.c_int32), ("cluster_sweeps", ctypes.c_int32),
        ("report", ctypes.c_int32), ("row_tiles_chunk_log2", ctypes.c_int32),
    ]

    OPTION_NAMES = tuple(n for n, _ in _fields_[3:])


class HpSpmmError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"hpspmm status {code}: {message}")
        self.code = code


_lib = None


def lib():
    """Load libhpspmm.so (raises if it has not been built)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing; build it with hp-spmm-sddmm_amd/build.py "
                               "(there is no fallback path)")
        L = ctypes.CDLL(LIB_PATH)
        L.hpspmm_version.restype = ctypes.c_int
        L.hpspmm_last_error.restype = ctypes.c_char_p
        L.hpspmm_plan_create.argtypes = [_i64, _i64, _i64, _p, _p, _i64, ctypes.c_uint32, _p,
                                         ctypes.POINTER(_p)]
        L.hpspmm_plan_create_ordered.argtypes = [_i64, _i64, _i64, _p, _p, _i64, ctypes.c_uint32, _p, _p,
                                                 ctypes.POINTER(_p)]
        L.hpspmm_plan_create_ex.argtypes = [_i64, _i64, _i64, _p, _p, _i64, ctypes.POINTER(PlanOptions), _p,
                                            ctypes.POINTER(_p)]
        L.hpspmm_static_workspace_init.argtypes = []
        L.hpspmm_get_device_info.argtypes = [ctypes.POINTER(DeviceInfo)]
        L.hpspmm_csr_spmm_timed_min.argtypes = [_p, _p, _p, _p, _p, _p, _p, ctypes.c_int, ctypes.c_int, ctypes.c_float,
                                                ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_int64)]
        L.hpspmm_plan_get_info.argtypes = [_p, ctypes.POINTER(PlanInfo)]
        L.hpspmm_plan_destroy.argtypes = [_p]
        L.hpspmm_plan_bind_values.argtypes = [_p, _p, _p]
        L.hpspmm_csr_spmm.argtypes = [_p, _p, _p, _p, _p, _p, _p]
        L.hpspmm_csr_spmm_noplan.argtypes = [_i64, _i64, _i64, _p, _p, _p, _p, _i64, _p, _p]
        L.hpspmm_csr_spmm_static.argtypes = [_i64, _i64, _i64, _p, _p, _p, _p, _i64, _p, _p]
        L.hpspmm_coo_spmm_accumulate.argtypes = [_i64, _i64, _i64, _p, _p, _p, _p, _i64, _p, _p]
        L.hpspmm_fill_f32.argtypes = [_p, _i64, ctypes.c_float, _p]
        L.hpspmm_csr_spmm_timed.argtypes = [_p, _p, _p, _p, _p, _p, _p, ctypes.c_int, ctypes.c_int,
                                            ctypes.POINTER(ctypes.c_float)]
        L.hpspmm_csr_spmm_timed_launches.argtypes = [_p, _p, _p, _p, _p, _p, _p, ctypes.c_int, ctypes.c_int,
                                                     ctypes.c_int, ctypes.POINTER(ctypes.c_float),
                                                     ctypes.POINTER(ctypes.c_char_p), ctypes.POINTER(ctypes.c_int)]
        _lib = L
    return _lib


def check(code):
    if code != OK:
        raise HpSpmmError(code, lib().hpspmm_last_error().decode())


def _ptr(t):
    """Device pointer of a torch tensor (None -> NULL)."""
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream(stream):
    if stream is None:
        import torch
        stream = torch.cuda.current_stream()
    return ctypes.c_void_p(stream.cuda_stream)


def _dev(t, dtype, name):
    import torch
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError(f"{name} must be a torch tensor in GPU memory")
    if t.dtype != dtype or not t.is_contiguous():
        raise TypeError(f"{name} must be contiguous {dtype}")
    return t


class Plan:
    """Owns an hpspmm_plan (see hpspmm_plan_create in include/hpspmm.h)."""

    def __init__(self, rows, cols, rowptr, col, k, flags=PLAN_DEFAULT, stream=None, row_order=None, options=None):
        """options: dict of hpspmm_plan_options fields (then the plan is made by hpspmm_plan_create_ex)."""
        import torch
        _dev(rowptr, torch.int32, "rowptr")
        _dev(col, torch.int32, "col")
        if rowptr.numel() != rows + 1:
            raise ValueError("rowptr must have rows + 1 entries")
        self._h = ctypes.c_void_p()
        self.rows, self.cols, self.nnz, self.k = int(rows), int(cols), int(col.numel()), int(k)
        if getattr(flags, "options", None):
            options = {**flags.options, **(options or {})}
        flags = int(flags)
        if options is not None:
            o = PlanOptions()
            o.struct_size = ctypes.sizeof(PlanOptions)
            o.flags = flags
            if row_order is not None:
                _dev(row_order, torch.int32, "row_order")
                if row_order.numel() != rows:
                    raise ValueError("row_order must have rows entries")
                o.d_row_order = row_order.data_ptr()
            for name, value in options.items():
                if name not in PlanOptions.OPTION_NAMES:
                    raise KeyError(f"hpspmm_plan_options has no field {name!r}")
                setattr(o, name, int(value))
            check(lib().hpspmm_plan_create_ex(rows, cols, self.nnz, _ptr(rowptr), _ptr(col), k, ctypes.byref(o),
                                              _stream(stream), ctypes.byref(self._h)))
        elif row_order is None:
            check(lib().hpspmm_plan_create(rows, cols, self.nnz, _ptr(rowptr), _ptr(col), k, flags,
                                           _stream(stream), ctypes.byref(self._h)))
        else:
            _dev(row_order, torch.int32, "row_order")
            if row_order.numel() != rows:
                raise ValueError("row_order must have rows entries")
            check(lib().hpspmm_plan_create_ordered(rows, cols, self.nnz, _ptr(rowptr), _ptr(col), k, flags,
                                                   _ptr(row_order), _stream(stream), ctypes.byref(self._h)))

    @property
    def info(self):
        out = PlanInfo()
        check(lib().hpspmm_plan_get_info(self._h, ctypes.byref(out)))
        return out.as_dict()

    def bind_values(self, val, stream=None):
        """hpspmm_plan_bind_values: `val` (or None to unbind) stays unchanged until the next bind."""
        import torch
        if val is not None:
            _dev(val, torch.float32, "val")
            if val.numel() != self.nnz:
                raise ValueError("val must have nnz entries")
        check(lib().hpspmm_plan_bind_values(self._h, _ptr(val) if val is not None else None, _stream(stream)))

    def destroy(self):
        if getattr(self, "_h", None):
            lib().hpspmm_plan_destroy(self._h)
            self._h = None

    def __del__(self):
        # at interpreter exit the module's globals may already be gone; the process frees the plan
        try:
            self.destroy()
        except Exception:
            pass


def _check_operands(rows, cols, nnz, k, rowptr, col, val, B, C):
    import torch
    if rowptr is not None:
        _dev(rowptr, torch.int32, "rowptr")
        if rowptr.numel() != rows + 1:
            raise ValueError("rowptr must have rows + 1 entries")
    _dev(col, torch.int32, "col")
    _dev(val, torch.float32, "val")
    _dev(B, torch.float32, "B")
    _dev(C, torch.float32, "C")
    if col.numel() != nnz or val.numel() != nnz:
        raise ValueError("col / val length differs from nnz")
    if tuple(B.shape) != (cols, k) or tuple(C.shape) != (rows, k):
        raise ValueError(f"B must be {(cols, k)} and C {(rows, k)}; got {tuple(B.shape)}, {tuple(C.shape)}")


def csr_spmm(plan, rowptr, col, val, B, C, stream=None):
    """C = A @ B through hpspmm_csr_spmm."""
    _check_operands(plan.rows, plan.cols, plan.nnz, plan.k, rowptr, col, val, B, C)
    check(lib().hpspmm_csr_spmm(plan._h, _ptr(rowptr), _ptr(col), _ptr(val), _ptr(B), _ptr(C),
                                _stream(stream)))
    return C


def csr_spmm_noplan(rows, cols, rowptr, col, val, B, C, stream=None):
    """C = A @ B through hpspmm_csr_spmm_noplan."""
    k = int(B.shape[1])
    _check_operands(rows, cols, int(col.numel()), k, rowptr, col, val, B, C)
    check(lib().hpspmm_csr_spmm_noplan(rows, cols, int(col.numel()), _ptr(rowptr), _ptr(col), _ptr(val),
                                       _ptr(B), k, _ptr(C), _stream(stream)))
    return C


def csr_spmm_static(rows, cols, rowptr, col, val, B, C, stream=None):
    """C = A @ B through hpspmm_csr_spmm_static (no plan, no allocation; k in {32,64,128}, nnz <= 2^22)."""
    k = int(B.shape[1])
    _check_operands(rows, cols, int(col.numel()), k, rowptr, col, val, B, C)
    check(lib().hpspmm_csr_spmm_static(rows, cols, int(col.numel()), _ptr(rowptr), _ptr(col), _ptr(val),
                                       _ptr(B), k, _ptr(C), _stream(stream)))
    return C


def coo_spmm_accumulate(rows, cols, row, col, val, B, C, stream=None):
    """C += A @ B through hpspmm_coo_spmm_accumulate."""
    import torch
    k = int(B.shape[1])
    _dev(row, torch.int32, "row")
    _check_operands(rows, cols, int(col.numel()), k, None, col, val, B, C)
    if row.numel() != col.numel():
        raise ValueError("row / col length differs")
    check(lib().hpspmm_coo_spmm_accumulate(rows, cols, int(col.numel()), _ptr(row), _ptr(col), _ptr(val),
                                           _ptr(B), k, _ptr(C), _stream(stream)))
    return C


def fill_f32(x, value, stream=None):
    import torch
    _dev(x, torch.float32, "x")
    check(lib().hpspmm_fill_f32(_ptr(x), x.numel(), float(value), _stream(stream)))
    return x


def csr_spmm_timed(plan, rowptr, col, val, B, C, warmup=20, iters=200, stream=None):
    """Mean milliseconds per SpMM over `iters` back-to-back launches (HIP events on the launch stream)."""
    _check_operands(plan.rows, plan.cols, plan.nnz, plan.k, rowptr, col, val, B, C)
    ms = ctypes.c_float(0.0)
    check(lib().hpspmm_csr_spmm_timed(plan._h, _ptr(rowptr), _ptr(col), _ptr(val), _ptr(B), _ptr(C),
                                      _stream(stream), warmup, iters, ctypes.byref(ms)))
    return float(ms.value)


def csr_spmm_timed_min(plan, rowptr, col, val, B, C, warmup=20, iters=200, min_total_ms=10.0, stream=None):
    """(mean ms per SpMM, launches timed): hpspmm_csr_spmm_timed_min - a region of `iters` launches, or of as
    many as fill min_total_ms when those take less."""
    _check_operands(plan.rows, plan.cols, plan.nnz, plan.k, rowptr, col, val, B, C)
    ms = ctypes.c_float(0.0)
    done = ctypes.c_int64(0)
    check(lib().hpspmm_csr_spmm_timed_min(plan._h, _ptr(rowptr), _ptr(col), _ptr(val), _ptr(B), _ptr(C),
                                          _stream(stream), warmup, iters, float(min_total_ms), ctypes.byref(ms),
                                          ctypes.byref(done)))
    return float(ms.value), int(done.value)


def device_info():
    """hpspmm_get_device_info as a dict."""
    out = DeviceInfo()
    check(lib().hpspmm_get_device_info(ctypes.byref(out)))
    d = {name: getattr(out, name) for name, _ in DeviceInfo._fields_}
    d["arch"] = d["arch"].decode()
    return d


def static_workspace_init():
    """hpspmm_static_workspace_init: look up the static workspace of csr_spmm_static on the current device."""
    check(lib().hpspmm_static_workspace_init())


def csr_spmm_timed_launches(plan, rowptr, col, val, B, C, warmup=5, iters=50, stream=None):
    """[(kernel name, mean ms)] for every launch of one SpMM, in launch order (HIP events between the launches)."""
    _check_operands(plan.rows, plan.cols, plan.nnz, plan.k, rowptr, col, val, B, C)
    cap = 40
    ms = (ctypes.c_float * cap)()
    names = (ctypes.c_char_p * cap)()
    n = ctypes.c_int(0)
    check(lib().hpspmm_csr_spmm_timed_launches(plan._h, _ptr(rowptr), _ptr(col), _ptr(val), _ptr(B), _ptr(C),
                                               _stream(stream), warmup, iters, cap, ms, names, ctypes.byref(n)))
    return [(names[i].decode(), float(ms[i])) for i in range(n.value)]
