"""MI355X-native HomComp: ctypes binding of libhomcomp_amd.so (the C ABI of include/homcomp.h).

The directory name is not a valid Python identifier; load it with ``__graft_entry__.load_package()``
(it registers the module as ``tirocinio_triennale_amd``).

There is no CPU fallback: if the HIP library is missing or no GPU is present every call raises.
torch is used for device memory and streams only; all codec work happens in the HIP kernels.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libhomcomp_amd.so")

# every symbol include/homcomp.h declares
EXPORTS = (
    "homcomp_status_string", "homcomp_last_hip_error", "homcomp_header_bytes",
    "homcomp_max_stream_bytes", "homcomp_ref_cmpsize", "homcomp_workspace_create",
    "homcomp_workspace_destroy", "homcomp_workspace_set_option", "homcomp_tile_offsets_count",
    "homcomp_workspace_tile_offsets", "homcomp_workspace_last_launch", "homcomp_compress_f32", "homcomp_decompress_f32",
    "homcomp_compress_plain_f32", "homcomp_decompress_plain_f32",
    "homcomp_hom_sum_f32", "homcomp_hom_sum_i32", "homcomp_hom_add", "homcomp_hom_sum_f32_static",
    "homcomp_quant_predict_f32", "homcomp_range_f32", "homcomp_rel_to_abs", "homcomp_last_size",
)


OPT_GRID_PERCENT = 1
OPT_SPIN_LIMIT = 2
OPT_LDS_BUDGET = 3      # -1 automatic, 0 small, 1 medium, 2 large
OPT_PLANE_PATHS = 4     # 1 automatic, 0 general path only, 2 few-plane kernels, 3 wide-block kernel for stream (+) stream
KERNEL_KINDS = {-1: None, 0: "general", 1: "few_planes", 2: "wide_planes"}
LDS_BUDGETS = {-1: None, 0: "small", 1: "medium", 2: "large"}
ERR_SCAN_TIMEOUT = -6


class HomCompError(RuntimeError):
    def __init__(self, status: int, what: str):
        self.status = status
        super().__init__(f"{what}: {status_string(status)} (status {status}, "
                         f"hip error {lib().homcomp_last_hip_error()})")


_lib = None


def lib() -> C.CDLL:
    """Load the HIP library; raises if it has not been built (no fallback)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                f"{LIB_PATH} is missing: build it with __graft_entry__.build() "
                f"(python tirocinio-triennale_amd/build.py)")
        # torch ships its own HIP runtime and publishes it process-wide.  It has to be loaded
        # before this library so that both bind to the same runtime instance: device pointers
        # and hipStream_t handles are only meaningful inside the runtime that created them.
        import torch  # noqa: F401
        L = C.CDLL(LIB_PATH)
        vp, sz, u64p = C.c_void_p, C.c_size_t, C.c_void_p
        L.homcomp_status_string.argtypes = [C.c_int]
        L.homcomp_status_string.restype = C.c_char_p
        L.homcomp_last_hip_error.restype = C.c_int
        for name in ("homcomp_header_bytes", "homcomp_max_stream_bytes"):
            getattr(L, name).argtypes = [sz]
            getattr(L, name).restype = sz
        L.homcomp_ref_cmpsize.argtypes = [sz, sz]
        L.homcomp_ref_cmpsize.restype = sz
        L.homcomp_workspace_create.argtypes = [C.POINTER(vp), sz]
        L.homcomp_workspace_destroy.argtypes = [vp]
        L.homcomp_workspace_set_option.argtypes = [vp, C.c_int, C.c_long]
        L.homcomp_tile_offsets_count.argtypes = [sz]
        L.homcomp_tile_offsets_count.restype = sz
        L.homcomp_workspace_tile_offsets.argtypes = [vp, vp, vp, vp]
        L.homcomp_workspace_last_launch.argtypes = [vp, C.POINTER(C.c_int), C.POINTER(C.c_int)]
        L.homcomp_compress_f32.argtypes = [vp, vp, sz, C.c_float, vp, u64p, vp]
        L.homcomp_decompress_f32.argtypes = [vp, vp, sz, sz, C.c_float, vp, vp]
        L.homcomp_compress_plain_f32.argtypes = [vp, vp, sz, C.c_float, vp, u64p, vp]
        L.homcomp_decompress_plain_f32.argtypes = [vp, vp, sz, C.c_float, vp, vp]
        L.homcomp_hom_sum_f32.argtypes = [vp, vp, sz, vp, sz, C.c_float, vp, u64p, vp]
        L.homcomp_hom_sum_i32.argtypes = [vp, vp, sz, vp, sz, vp, u64p, vp]
        L.homcomp_hom_add.argtypes = [vp, vp, sz, vp, sz, sz, vp, u64p, vp]
        L.homcomp_hom_sum_f32_static.argtypes = [vp, sz, vp, sz, C.c_float, vp, u64p, vp]
        L.homcomp_quant_predict_f32.argtypes = [vp, sz, C.c_float, vp, vp]
        L.homcomp_range_f32.argtypes = [vp, vp, sz, vp, vp]
        L.homcomp_rel_to_abs.argtypes = [C.c_float, C.c_float, C.c_float]
        L.homcomp_rel_to_abs.restype = C.c_float
        L.homcomp_last_size.argtypes = [vp, C.POINTER(sz), vp]
        _lib = L
    return _lib


def status_string(status: int) -> str:
    return lib().homcomp_status_string(status).decode()


def header_bytes(n: int) -> int:
    return int(lib().homcomp_header_bytes(n))


def max_stream_bytes(n: int) -> int:
    return int(lib().homcomp_max_stream_bytes(n))


def tile_offsets_count(n: int) -> int:
    return int(lib().homcomp_tile_offsets_count(n))


STREAM_SLACK = 160   # HOMCOMP_STREAM_SLACK: bytes an input stream buffer must be readable beyond its stated size


def ref_cmpsize(stream_len: int, n: int) -> int:
    return int(lib().homcomp_ref_cmpsize(stream_len, n))


def rel_to_abs(rel: float, vmin: float, vmax: float) -> float:
    return float(lib().homcomp_rel_to_abs(rel, vmin, vmax))


def _check(status: int, what: str) -> None:
    if status != 0:
        raise HomCompError(status, what)


def _stream_ptr(stream) -> int:
    import torch
    s = torch.cuda.current_stream() if stream is None else stream
    return int(s.cuda_stream)


class Workspace:
    """Scan state for one in-flight call (homcomp_workspace_create / _destroy).

    Methods take torch CUDA tensors, enqueue on ``stream`` (default: torch's current stream)
    and return immediately; ``last_size`` is the only blocking call.
    """

    def __init__(self, max_n: int):
        self._h = C.c_void_p()
        self.max_n = int(max_n)
        _check(lib().homcomp_workspace_create(C.byref(self._h), self.max_n), "workspace_create")

    def close(self) -> None:
        if self._h:
            _check(lib().homcomp_workspace_destroy(self._h), "workspace_destroy")
            self._h = C.c_void_p()

    def set_option(self, option: int, value: int) -> None:
        _check(lib().homcomp_workspace_set_option(self._h, int(option), int(value)), "workspace_set_option")

    def last_launch(self) -> dict:
        """Kernel kind and LDS budget of the last stream-producing call on this workspace."""
        kind, budget = C.c_int(), C.c_int()
        _check(lib().homcomp_workspace_last_launch(self._h, C.byref(kind), C.byref(budget)), "workspace_last_launch")
        return {"kernel": KERNEL_KINDS[kind.value], "lds_budget": LDS_BUDGETS[budget.value]}

    def tile_offsets(self, in_a=None, in_b=None, out=None) -> None:
        """Tile offsets for the next call on this workspace (homcomp_workspace_tile_offsets): int64 device
        tensors of tile_offsets_count(n) entries; the incoming streams' as left by the calls that
        produced them, and/or where the next call leaves those of the stream it produces."""
        ptr = lambda t: None if t is None else t.data_ptr()
        _check(lib().homcomp_workspace_tile_offsets(self._h, ptr(in_a), ptr(in_b), ptr(out)), "workspace_tile_offsets")

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    # -- raw entry points (tensor arguments, explicit sizes) ---------------------------------
    def compress(self, data, eb: float, cmp, stream_len=None, n: int | None = None, stream=None):
        n = data.numel() if n is None else n
        _check(lib().homcomp_compress_f32(self._h, data.data_ptr(), n, eb, cmp.data_ptr(),
                                          stream_len.data_ptr() if stream_len is not None else None,
                                          _stream_ptr(stream)), "compress_f32")

    def compress_plain(self, data, eb: float, cmp, stream_len=None, n: int | None = None, stream=None):
        n = data.numel() if n is None else n
        _check(lib().homcomp_compress_plain_f32(self._h, data.data_ptr(), n, eb, cmp.data_ptr(),
                                                stream_len.data_ptr() if stream_len is not None else None,
                                                _stream_ptr(stream)), "compress_plain_f32")

    def decompress_plain(self, cmp, n: int, eb: float, out, stream=None):
        _check(lib().homcomp_decompress_plain_f32(self._h, cmp.data_ptr(), n, eb, out.data_ptr(),
                                                  _stream_ptr(stream)), "decompress_plain_f32")

    def decompress(self, cmp, cmp_size: int, n: int, eb: float, out, stream=None):
        _check(lib().homcomp_decompress_f32(self._h, cmp.data_ptr(), cmp_size, n, eb,
                                            out.data_ptr(), _stream_ptr(stream)), "decompress_f32")

    def hom_sum_f32(self, cmp_in, cmp_in_size: int, local, eb: float, cmp_out, stream_len=None,
                    n: int | None = None, stream=None):
        n = local.numel() if n is None else n
        _check(lib().homcomp_hom_sum_f32(self._h, cmp_in.data_ptr(), cmp_in_size, local.data_ptr(),
                                         n, eb, cmp_out.data_ptr(),
                                         stream_len.data_ptr() if stream_len is not None else None,
                                         _stream_ptr(stream)), "hom_sum_f32")

    def hom_sum_i32(self, cmp_in, cmp_in_size: int, local_delta, cmp_out, stream_len=None,
                    n: int | None = None, stream=None):
        n = local_delta.numel() if n is None else n
        _check(lib().homcomp_hom_sum_i32(self._h, cmp_in.data_ptr(), cmp_in_size,
                                         local_delta.data_ptr(), n, cmp_out.data_ptr(),
                                         stream_len.data_ptr() if stream_len is not None else None,
                                         _stream_ptr(stream)), "hom_sum_i32")

    def hom_add(self, cmp_a, size_a: int, cmp_b, size_b: int, n: int, cmp_out, stream_len=None,
                stream=None):
        _check(lib().homcomp_hom_add(self._h, cmp_a.data_ptr(), size_a, cmp_b.data_ptr(), size_b,
                                     n, cmp_out.data_ptr(),
                                     stream_len.data_ptr() if stream_len is not None else None,
                                     _stream_ptr(stream)), "hom_add")

    def value_range(self, data, minmax, n: int | None = None, stream=None):
        n = data.numel() if n is None else n
        _check(lib().homcomp_range_f32(self._h, data.data_ptr(), n, minmax.data_ptr(),
                                       _stream_ptr(stream)), "range_f32")

    def last_size(self, stream=None) -> int:
        out = C.c_size_t()
        _check(lib().homcomp_last_size(self._h, C.byref(out), _stream_ptr(stream)), "last_size")
        return int(out.value)


STATIC_MAX_ELEMENTS = 1 << 24


def hom_sum_f32_static(cmp_in, cmp_in_size: int, local, eb: float, cmp_out, result, n: int | None = None,
                       stream=None) -> None:
    """homcomp_hom_sum_f32_static: no workspace, nothing allocated; ``result`` is a device int64[2]
    (stream length, scan time-out flag)."""
    n = local.numel() if n is None else n
    _check(lib().homcomp_hom_sum_f32_static(cmp_in.data_ptr(), cmp_in_size, local.data_ptr(), n, eb,
                                            cmp_out.data_ptr(), result.data_ptr(), _stream_ptr(stream)),
           "hom_sum_f32_static")


def quant_predict(data, eb: float, delta, n: int | None = None, stream=None) -> None:
    n = data.numel() if n is None else n
    _check(lib().homcomp_quant_predict_f32(data.data_ptr(), n, eb, delta.data_ptr(),
                                           _stream_ptr(stream)), "quant_predict_f32")
