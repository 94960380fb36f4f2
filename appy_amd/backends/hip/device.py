"""What the launcher knows of a device and how kernels get onto it: the facts the launch heuristics use
(compute units, XCDs, cache sizes), the limit on device memory a loop may hold, hiprtc with its on-disk
cache, compiled kernels and their per-device function handles, HIP's per-thread current device, PyTorch's
current stream."""
from __future__ import annotations

import ctypes as C
import dataclasses
import hashlib
import os
import threading

from . import runtime as rt
from .kernelgen import KernelSource

ARCH = "gfx950"
_HEADER_PATH = os.path.join(os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))), "csrc", "appy_device.h")
_device_header = None


@dataclasses.dataclass(frozen=True)
class Hardware:
    """What the launch heuristics know of a device.  The defaults are MI355X's: 256 CUs in 8 XCDs, an L2 of
    4 MiB per XCD, 256 MiB of memory-side cache in front of the HBM3E (the one figure the runtime does not
    report: `APPY_HIP_MALL_BYTES` overrides it)."""

    cus: int = 256
    xcds: int = 8
    l2_bytes: int = 4 << 20
    mall_bytes: int = 256 << 20

    @property
    def stripe_bytes(self) -> int:
        """Most of a gathered operand that one XCD is given to keep in its L2 next to the streams: half the L2."""
        return self.l2_bytes // 2

    @property
    def stripe_min_bytes(self) -> int:
        """A gathered operand up to this size is left to every L2 as a whole."""
        return 3 * self.l2_bytes // 4

    @property
    def pinned_stripes(self) -> bool:
        """Stripes of a gathered operand are pinned to XCDs by workgroup number modulo 8 in the generated kernels."""
        return self.xcds == 8


MI355X = Hardware()
_hardware = {}


def hardware(device=None) -> Hardware:
    """The facts of ``device`` as the runtime reports them; MI355X's when no device is named (kernels generated
    and launch shapes chosen without a GPU)."""
    if device is None:
        return MI355X
    hw = _hardware.get(device)
    if hw is None:
        t = rt.device_topology(device)
        hw = Hardware(cus=int(t["compute_units"]) or MI355X.cus, xcds=int(t["xcds"]) or 1,
                      l2_bytes=int(t["l2_bytes_per_xcd"]) or MI355X.l2_bytes,
                      mall_bytes=int(os.environ.get("APPY_HIP_MALL_BYTES") or MI355X.mall_bytes))
        _hardware[device] = hw
    return hw


def scratch_limit(device: int) -> int:
    """Most bytes of device memory one loop may hold for its own purposes (scratch buffers of launches made of
    several kernels, row plans): `APPY_HIP_SCRATCH_MAX_BYTES`, or a quarter of the device's memory."""
    env = os.environ.get("APPY_HIP_SCRATCH_MAX_BYTES")
    if env:
        return int(env)
    if device not in _hbm_bytes:
        _hbm_bytes[device] = int(rt.device_props(device)["hbm_bytes"])
    return _hbm_bytes[device] // 4


_hbm_bytes = {}


def device_header() -> str:
    global _device_header
    if _device_header is None:
        with open(_HEADER_PATH) as f:
            _device_header = f.read()
    return _device_header


# ---------------------------------------------------------------------------
# compiled kernels
# ---------------------------------------------------------------------------
def _disk_cache_dir():
    if os.environ.get("APPY_HIP_NO_DISK_CACHE") == "1":
        return None
    d = os.environ.get("APPY_HIP_CACHE_DIR") or os.path.join(os.path.expanduser("~"), ".cache", "appy_hip")
    try:
        os.makedirs(d, exist_ok=True)
    except OSError:
        return None
    return d


def compile_source(text: str, name: str) -> bytes:
    """HIP C++ -> gfx950 code object, through hiprtc, with an on-disk cache
    keyed on the source text, the compiler options and the compiler version."""
    d = _disk_cache_dir()
    path = None
    if d:
        h = hashlib.sha256()
        h.update(text.encode())
        h.update(repr(rt.BASE_COMPILE_OPTIONS + rt.extra_compile_options()).encode())
        h.update(ARCH.encode())
        h.update(str(rt.rtc_version()).encode())
        path = os.path.join(d, h.hexdigest() + ".co")
        if os.path.exists(path):
            with open(path, "rb") as f:
                code = f.read()
            if code[:4] == b"\x7fELF":
                return code
    code = rt.compile_to_code_object(text, name + ".hip", ARCH)
    if path:
        tmp = path + f".{os.getpid()}.tmp"
        try:
            with open(tmp, "wb") as f:
                f.write(code)
            os.replace(tmp, path)
        except OSError:
            pass
    return code


class Kernel:
    """One compiled variant of a loop."""

    def __init__(self, src: KernelSource):
        self.src = src
        self._code = None
        self._compile_lock = threading.Lock()
        self._funcs = {}   # device -> function handle
        fields = [(f"f{i}", p.ctype) for i, p in enumerate(src.params)]
        self.ArgStruct = type("Args" + src.name, (C.Structure,), {"_fields_": fields})
        self._field_names = [f for f, _ in fields]

    @property
    def code(self) -> bytes:
        """The code object, compiled when first asked for: a loop is generated in its default
        shape when it is first seen, but the launch may pick another shape, and hiprtc takes a
        few hundred milliseconds per variant."""
        if self._code is None:
            with self._compile_lock:
                if self._code is None:
                    self._code = compile_source(self.src.text, self.src.name)
        return self._code

    def function(self, device: int):
        f = self._funcs.get(device)
        if f is None:
            mod = rt.Module(self.code)
            f = (mod, mod.function(self.src.name))
            self._funcs[device] = f
        return f[1]


# ---------------------------------------------------------------------------
# the launcher
# ---------------------------------------------------------------------------
_tls = threading.local()


def _ensure_device(dev: int):
    """HIP's current device is a per-thread setting."""
    if getattr(_tls, "device", None) != dev:
        rt.init(dev)
        _tls.device = dev


_raw_stream_getter = None


def _current_raw_stream(device: int) -> int:
    """PyTorch's current stream on ``device`` as a raw handle."""
    global _raw_stream_getter
    if _raw_stream_getter is None:
        import torch

        _raw_stream_getter = getattr(torch._C, "_cuda_getCurrentRawStream", None) or (
            lambda dev: torch.cuda.current_stream(dev).cuda_stream)
    return _raw_stream_getter(device)
