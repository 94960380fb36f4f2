"""ctypes binding of ``libappy_hip.so`` (C ABI: include/appy_hip.h).

The library is the only way generated kernels reach the GPU; there is no
fallback.  A missing library is a hard error that says how to build it.
"""
from __future__ import annotations

import ctypes as C
import os
import threading

_LIB_NAME = "libappy_hip.so"
_PKG_ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

ABI_VERSION = 5


class Props(C.Structure):
    _fields_ = [
        ("name", C.c_char * 128),
        ("arch", C.c_char * 64),
        ("compute_units", C.c_int32),
        ("wavefront_size", C.c_int32),
        ("max_threads_per_block", C.c_int32),
        ("lds_bytes_per_block", C.c_int32),
        ("l2_bytes", C.c_int32),
        ("clock_khz", C.c_int32),
        ("mem_clock_khz", C.c_int32),
        ("mem_bus_bits", C.c_int32),
        ("hbm_bytes", C.c_uint64),
    ]


class Topology(C.Structure):
    _fields_ = [
        ("xcds", C.c_int32),
        ("compute_units", C.c_int32),
        ("l2_bytes_per_xcd", C.c_int32),
        ("lds_bytes_per_cu", C.c_int32),
    ]


class FuncInfo(C.Structure):
    _fields_ = [
        ("num_vgprs", C.c_int32),
        ("static_lds_bytes", C.c_int32),
        ("scratch_bytes", C.c_int32),
        ("max_threads_per_block", C.c_int32),
    ]


class RowPlanShape(C.Structure):
    _fields_ = [
        ("entries", C.c_uint64),
        ("row_blocks", C.c_uint32),
        ("groups", C.c_uint32),
        ("group_width", C.c_uint32),
        ("col_bits", C.c_uint32),
        ("tile", C.c_uint32),
        ("line_bits", C.c_uint32),
        ("full", C.c_uint32),
    ]


class HipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"[appy_hip error {code}] {message}")
        self.code = code


_u32 = C.c_uint32
_vp = C.c_void_p

# name -> (restype, argtypes); every symbol declared in include/appy_hip.h
SIGNATURES = {
    "appy_hip_abi_version": (C.c_int, []),
    "appy_hip_last_error": (C.c_char_p, []),
    "appy_hip_device_count": (C.c_int, [C.POINTER(C.c_int)]),
    "appy_hip_init": (C.c_int, [C.c_int]),
    "appy_hip_device_props": (C.c_int, [C.c_int, C.POINTER(Props)]),
    "appy_hip_device_topology": (C.c_int, [C.c_int, C.POINTER(Topology)]),
    "appy_hip_compile": (
        C.c_int,
        [C.c_char_p, C.c_char_p, C.c_char_p, C.POINTER(C.c_char_p), C.c_int, C.POINTER(_vp), C.POINTER(C.c_size_t)],
    ),
    "appy_hip_compile_log": (C.c_char_p, []),
    "appy_hip_code_free": (None, [_vp]),
    "appy_hip_module_load": (C.c_int, [_vp, C.c_size_t, C.POINTER(_vp)]),
    "appy_hip_module_get_function": (C.c_int, [_vp, C.c_char_p, C.POINTER(_vp)]),
    "appy_hip_module_unload": (C.c_int, [_vp]),
    "appy_hip_func_get_info": (C.c_int, [_vp, C.POINTER(FuncInfo)]),
    "appy_hip_occupancy": (C.c_int, [_vp, C.c_int, C.c_size_t, C.POINTER(C.c_int)]),
    "appy_hip_malloc": (C.c_int, [C.c_size_t, C.POINTER(_vp)]),
    "appy_hip_free": (C.c_int, [_vp]),
    "appy_hip_pool_trim": (C.c_int, []),
    "appy_hip_pool_stats": (C.c_int, [C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "appy_hip_memcpy_h2d": (C.c_int, [_vp, _vp, C.c_size_t, _vp]),
    "appy_hip_memcpy_d2h": (C.c_int, [_vp, _vp, C.c_size_t, _vp]),
    "appy_hip_memcpy_h2d_async": (C.c_int, [_vp, _vp, C.c_size_t, _vp]),
    "appy_hip_host_alloc": (C.c_int, [C.c_size_t, C.POINTER(_vp)]),
    "appy_hip_host_free": (C.c_int, [_vp]),
    "appy_hip_host_is_pinned": (C.c_int, [_vp, C.c_size_t]),
    "appy_hip_memcpy_d2d_async": (C.c_int, [_vp, _vp, C.c_size_t, _vp]),
    "appy_hip_memset_async": (C.c_int, [_vp, C.c_int, C.c_size_t, _vp]),
    "appy_hip_launch": (C.c_int, [_vp, _u32, _u32, _u32, _u32, _u32, _u32, _u32, _vp, _vp, C.c_size_t]),
    "appy_hip_sync": (C.c_int, [_vp]),
    "appy_hip_device_sync": (C.c_int, []),
    "appy_hip_launch_static_scratch": (
        C.c_int, [_vp, _u32, _u32, _u32, _u32, _u32, _u32, _u32, _vp, _vp, C.c_size_t, C.c_size_t, C.c_size_t]),
    "appy_hip_rtc_version": (C.c_int, [C.POINTER(C.c_int)]),
    "appy_hip_rowplan_sizes": (C.c_int, [C.POINTER(RowPlanShape), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "appy_hip_rowplan_build": (C.c_int, [C.POINTER(RowPlanShape), _vp, _vp, _vp, _vp, _vp, C.c_size_t, _vp, _vp, _vp, _vp]),
    "appy_hip_stream_create": (C.c_int, [C.POINTER(_vp)]),
    "appy_hip_stream_destroy": (C.c_int, [_vp]),
    "appy_hip_graph_begin": (C.c_int, [_vp]),
    "appy_hip_graph_end": (C.c_int, [_vp, C.POINTER(_vp)]),
    "appy_hip_graph_launch": (C.c_int, [_vp, _vp]),
    "appy_hip_graph_destroy": (C.c_int, [_vp]),
    "appy_hip_event_create": (C.c_int, [C.POINTER(_vp)]),
    "appy_hip_event_record": (C.c_int, [_vp, _vp]),
    "appy_hip_event_sync": (C.c_int, [_vp]),
    "appy_hip_event_elapsed_ms": (C.c_int, [_vp, _vp, C.POINTER(C.c_float)]),
    "appy_hip_event_destroy": (C.c_int, [_vp]),
    "appy_hip_launch_timed": (
        C.c_int,
        [_vp, _u32, _u32, _u32, _u32, _u32, _u32, _u32, _vp, _vp, C.c_size_t, C.c_int, C.c_int, C.POINTER(C.c_float)],
    ),
}

_lib = None
_lib_lock = threading.Lock()


def library_path() -> str:
    return os.environ.get("APPY_HIP_LIBRARY") or os.path.join(_PKG_ROOT, _LIB_NAME)


def lib():
    """The loaded library (loaded on first use)."""
    global _lib
    if _lib is not None:
        return _lib
    with _lib_lock:
        if _lib is not None:
            return _lib
        path = library_path()
        if not os.path.exists(path):
            raise RuntimeError(
                f"{_LIB_NAME} not found at {path}: the HIP runtime layer is not built. "
                "Run `python -c 'import __graft_entry__ as g; g.build()'` at the repository root "
                "(or `make -C appy_amd/csrc`)."
            )
        handle = C.CDLL(path, mode=C.RTLD_GLOBAL)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        got = handle.appy_hip_abi_version()
        if got != ABI_VERSION:
            raise RuntimeError(f"{path} has ABI version {got}, this package needs {ABI_VERSION}")
        _lib = handle
    return _lib


def last_error() -> str:
    return (lib().appy_hip_last_error() or b"").decode("utf-8", "replace")


def check(rc: int) -> None:
    if rc != 0:
        raise HipError(rc, last_error())


# ---- thin, typed helpers ----------------------------------------------------
def device_count() -> int:
    n = C.c_int(0)
    check(lib().appy_hip_device_count(C.byref(n)))
    return n.value


def init(device: int = 0) -> None:
    check(lib().appy_hip_init(int(device)))


def device_props(device: int = 0) -> dict:
    p = Props()
    check(lib().appy_hip_device_props(int(device), C.byref(p)))
    out = {}
    for f, _ in Props._fields_:
        v = getattr(p, f)
        out[f] = v.decode() if isinstance(v, bytes) else v
    return out


def device_topology(device: int = 0) -> dict:
    t = Topology()
    check(lib().appy_hip_device_topology(int(device), C.byref(t)))
    return {f: getattr(t, f) for f, _ in Topology._fields_}


# Options every kernel is compiled with.  Contraction is off so that
# elementwise results equal the interpreter's bit for bit (no fused
# multiply-add where the source has a multiply and an add); the packed-fp32
# feature is disabled because some packed forms have shown wrong results.
BASE_COMPILE_OPTIONS = (
    "-O3",
    "-std=c++17",
    "-ffp-contract=off",
    "-munsafe-fp-atomics",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # no 8-bit dot-product instructions: the compiler's fold of byte multiply-add chains into
    # v_dot4_u32_u8 rewrote `u * u + max(u, u * u)` (uint8) as `dot4((u, u, 0, 0), (u, u, 0, 0)) + u`,
    # a different value, and crashed in instruction selection on the 16-byte form of the same loop
    "-Xclang", "-target-feature", "-Xclang", "-dot7-insts",
    "-Xclang", "-target-feature", "-Xclang", "-dot1-insts",
)


def extra_compile_options() -> tuple:
    """Options appended to every hiprtc compilation: ``APPY_HIP_EXTRA_COMPILE_OPTIONS``
    (space separated)."""
    return tuple(os.environ.get("APPY_HIP_EXTRA_COMPILE_OPTIONS", "").split())


def compile_to_code_object(source: str, name: str, arch: str = "gfx950", extra_opts=()) -> bytes:
    """HIP C++ text -> code object bytes (works without a GPU)."""
    opts = [o.encode() for o in (*BASE_COMPILE_OPTIONS, *extra_opts, *extra_compile_options())]
    arr = (C.c_char_p * len(opts))(*opts)
    code = _vp()
    size = C.c_size_t(0)
    rc = lib().appy_hip_compile(source.encode(), name.encode(), arch.encode(), arr, len(opts), C.byref(code), C.byref(size))
    if rc != 0:
        raise HipError(rc, "hiprtc compilation failed:\n" + last_error())
    try:
        return C.string_at(code.value, size.value)
    finally:
        lib().appy_hip_code_free(code)


def rtc_version() -> int:
    out = C.c_int()
    check(lib().appy_hip_rtc_version(C.byref(out)))
    return out.value


def compile_log() -> str:
    return (lib().appy_hip_compile_log() or b"").decode("utf-8", "replace")


class Module:
    """A code object loaded on the current device."""

    def __init__(self, code: bytes):
        self._code = code  # keep alive
        h = _vp()
        check(lib().appy_hip_module_load(code, len(code), C.byref(h)))
        self.handle = h

    def function(self, name: str):
        f = _vp()
        check(lib().appy_hip_module_get_function(self.handle, name.encode(), C.byref(f)))
        return f


def func_info(func) -> dict:
    fi = FuncInfo()
    check(lib().appy_hip_func_get_info(func, C.byref(fi)))
    return {f: getattr(fi, f) for f, _ in FuncInfo._fields_}


def occupancy(func, block_threads: int, dynamic_lds: int = 0) -> int:
    n = C.c_int(0)
    check(lib().appy_hip_occupancy(func, int(block_threads), int(dynamic_lds), C.byref(n)))
    return n.value


def malloc(nbytes: int) -> int:
    p = _vp()
    check(lib().appy_hip_malloc(int(nbytes), C.byref(p)))
    return p.value or 0


def free(dptr: int) -> None:
    check(lib().appy_hip_free(_vp(dptr)))


def memcpy_h2d(dst: int, src_host_ptr: int, nbytes: int, stream: int = 0) -> None:
    check(lib().appy_hip_memcpy_h2d(_vp(dst), _vp(src_host_ptr), int(nbytes), _vp(stream)))


def memcpy_h2d_async(dst: int, src_pinned_ptr: int, nbytes: int, stream: int = 0) -> None:
    """Upload from page-locked memory that returns once it is queued on ``stream``."""
    check(lib().appy_hip_memcpy_h2d_async(_vp(dst), _vp(src_pinned_ptr), int(nbytes), _vp(stream)))


def memcpy_d2h(dst_host_ptr: int, src: int, nbytes: int, stream: int = 0) -> None:
    check(lib().appy_hip_memcpy_d2h(_vp(dst_host_ptr), _vp(src), int(nbytes), _vp(stream)))


def host_alloc(nbytes: int) -> int:
    """Page-locked host memory (address as int)."""
    out = _vp()
    check(lib().appy_hip_host_alloc(int(nbytes), C.byref(out)))
    return out.value


def host_free(ptr: int) -> None:
    check(lib().appy_hip_host_free(_vp(ptr)))


def host_is_pinned(ptr: int, nbytes: int) -> bool:
    return bool(lib().appy_hip_host_is_pinned(_vp(ptr), int(nbytes)))


def memset_async(dst: int, value: int, nbytes: int, stream: int = 0) -> None:
    check(lib().appy_hip_memset_async(_vp(dst), int(value), int(nbytes), _vp(stream)))


def launch(func, grid, block, args_struct, stream: int = 0, dynamic_lds: int = 0) -> None:
    gx, gy, gz = grid
    bx, by, bz = block
    check(
        lib().appy_hip_launch(
            func, gx, gy, gz, bx, by, bz, int(dynamic_lds), _vp(stream),
            C.byref(args_struct), C.sizeof(args_struct),
        )
    )


STATIC_SCRATCH_BYTES = 8 << 20


def launch_static_scratch(func, grid, block, args_struct, scratch_field: str, scratch_bytes: int, stream: int = 0,
                          dynamic_lds: int = 0) -> None:
    """Launch with the pointer field ``scratch_field`` of the argument block replaced by the
    library's static scratch buffer of the current device; allocates nothing."""
    gx, gy, gz = grid
    bx, by, bz = block
    offset = getattr(type(args_struct), scratch_field).offset
    check(
        lib().appy_hip_launch_static_scratch(
            func, gx, gy, gz, bx, by, bz, int(dynamic_lds), _vp(stream),
            C.byref(args_struct), C.sizeof(args_struct), offset, int(scratch_bytes),
        )
    )


def launch_timed(func, grid, block, args_struct, stream: int = 0, dynamic_lds: int = 0, warmup: int = 2, reps: int = 20) -> float:
    """Mean milliseconds per launch over ``reps`` back-to-back launches,
    measured with HIP events on ``stream``."""
    gx, gy, gz = grid
    bx, by, bz = block
    ms = C.c_float(0.0)
    check(
        lib().appy_hip_launch_timed(
            func, gx, gy, gz, bx, by, bz, int(dynamic_lds), _vp(stream),
            C.byref(args_struct), C.sizeof(args_struct), int(warmup), int(reps), C.byref(ms),
        )
    )
    return ms.value


def sync(stream: int = 0) -> None:
    check(lib().appy_hip_sync(_vp(stream)))


def device_sync() -> None:
    """Wait for every stream of the current device."""
    check(lib().appy_hip_device_sync())


def stream_create() -> int:
    out = _vp()
    check(lib().appy_hip_stream_create(C.byref(out)))
    return out.value


def stream_destroy(stream: int) -> None:
    check(lib().appy_hip_stream_destroy(_vp(stream)))


def graph_begin(stream: int) -> None:
    check(lib().appy_hip_graph_begin(_vp(stream)))


def graph_end(stream: int) -> int:
    out = _vp()
    check(lib().appy_hip_graph_end(_vp(stream), C.byref(out)))
    return out.value


def graph_launch(graph_exec: int, stream: int) -> None:
    check(lib().appy_hip_graph_launch(_vp(graph_exec), _vp(stream)))


def graph_destroy(graph_exec: int) -> None:
    check(lib().appy_hip_graph_destroy(_vp(graph_exec)))


class Event:
    def __init__(self):
        h = _vp()
        check(lib().appy_hip_event_create(C.byref(h)))
        self.handle = h

    def record(self, stream: int = 0):
        check(lib().appy_hip_event_record(self.handle, _vp(stream)))

    def synchronize(self):
        check(lib().appy_hip_event_sync(self.handle))

    def elapsed_ms(self, stop: "Event") -> float:
        ms = C.c_float(0.0)
        check(lib().appy_hip_event_elapsed_ms(self.handle, stop.handle, C.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            if self.handle:
                lib().appy_hip_event_destroy(self.handle)
                self.handle = None
        except Exception:
            pass
