"""The C-ABI library: loads, exports exactly what include/appy_hip.h declares,
and its GPU-independent entry points (run-time compilation, error reporting)
behave as documented.  No kernel is launched here."""
import ctypes
import os
import re
import subprocess

import pytest

from appy_amd.backends.hip import runtime as rt

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "appy_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(appy_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    decl = declared_symbols()
    assert len(decl) >= 25
    assert sorted(rt.SIGNATURES) == decl


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(rt.library_path())
    for name in declared_symbols():
        assert hasattr(lib, name), name
    out = subprocess.run(["nm", "-D", "--defined-only", rt.library_path()], capture_output=True, text=True, check=True).stdout
    exported = set(re.findall(r"\bT (appy_hip_[a-z0-9_]+)", out))
    assert exported == set(declared_symbols())          # nothing undeclared leaks out either


def test_abi_version():
    assert rt.lib().appy_hip_abi_version() == rt.ABI_VERSION
    text = open(HEADER).read()
    assert f"#define APPY_HIP_ABI_VERSION {rt.ABI_VERSION}" in text


def test_a_library_built_from_other_sources_is_rebuilt(monkeypatch):
    """The build leaves a digest of the library's sources and flags next to the binary; the tests,
    the smoke run and the benchmark rebuild when it does not match the tree."""
    import __graft_entry__ as entry

    assert entry.library_is_current()
    monkeypatch.setattr(entry, "_sources_digest", lambda: "0" * 64)
    assert not entry.library_is_current()
    calls = []
    monkeypatch.setattr(entry, "build", lambda: calls.append(1))
    entry.ensure_built()
    assert calls == [1]


def test_compile_produces_a_gfx950_code_object():
    src = 'extern "C" __global__ void k(float* a, long long n) { long long i = blockIdx.x * 64ll + threadIdx.x; if (i < n) a[i] += 1.0f; }'
    code = rt.compile_to_code_object(src, "k.hip")
    assert code[:4] == b"\x7fELF" and len(code) > 1000
    assert b"gfx950" in code


def test_compile_error_carries_the_compiler_log():
    with pytest.raises(rt.HipError) as e:
        rt.compile_to_code_object('extern "C" __global__ void k() { this is not C++; }', "bad.hip")
    assert e.value.code >= 10000                          # hiprtc result space
    assert "error" in str(e.value) and "bad.hip" in str(e.value)


def test_invalid_arguments_are_reported_not_crashed():
    lib = rt.lib()
    assert lib.appy_hip_device_count(None) != 0
    assert "count_out" in rt.last_error()
    assert lib.appy_hip_launch(None, 1, 1, 1, 64, 1, 1, 0, None, None, 0) != 0
    assert "func" in rt.last_error()
    ms = ctypes.c_float()
    assert lib.appy_hip_launch_timed(None, 1, 1, 1, 64, 1, 1, 0, None, None, 0, 0, 1, ctypes.byref(ms)) != 0
    assert lib.appy_hip_free(None) == 0                   # freeing NULL is a no-op
    assert lib.appy_hip_module_unload(None) == 0


def test_device_count_without_gpu_is_zero_not_an_error():
    assert rt.device_count() >= 0


CLIENT_SRC = os.path.join(ROOT, "tests", "cabi", "client.c")


def _build_client(tmp_path):
    exe = tmp_path / "cabi_client"
    lib_dir = os.path.dirname(rt.library_path())
    subprocess.run(
        ["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I" + os.path.join(ROOT, "include"), CLIENT_SRC,
         "-o", str(exe), "-L" + lib_dir, "-lappy_hip", "-Wl,-rpath," + lib_dir],
        check=True, capture_output=True, text=True)
    return str(exe)


def test_header_is_plain_c_and_a_c_client_can_compile_kernels(tmp_path):
    exe = _build_client(tmp_path)
    out = subprocess.run([exe, "compile"], check=True, capture_output=True, text=True).stdout
    assert out.startswith("compiled ") and int(out.split()[1]) > 1000


@pytest.mark.gpu
def test_c_client_runs_a_kernel_end_to_end(tmp_path, gpu):
    exe = _build_client(tmp_path)
    out = subprocess.run([exe, "run"], check=True, capture_output=True, text=True, timeout=120).stdout
    assert "ran 100003 elements, 0 mismatches" in out
