"""Host-only checks of the library's launch arithmetic (tests/host/host_checks.cpp): the rules that split K over the
grid, with the chip's compute units as a parameter, and the mapping of a failing HIP call to the status codes of the C ABI.
Compiled here with the host compiler against the library's own headers; nothing runs on a GPU."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


def test_split_rules_and_error_statuses(tmp_path):
    exe = str(tmp_path / "host_checks")
    build = subprocess.run(
        ["g++", "-std=c++17", "-O1", "-Wall", "-D__HIP_PLATFORM_AMD__", f"-I{ROCM}/include", f"-I{ROOT}/include",
         f"-I{ROOT}/nuvec_amd/csrc", f"{ROOT}/tests/host/host_checks.cpp", "-o", exe, f"-L{ROCM}/lib", "-lamdhip64",
         f"-Wl,-rpath,{ROCM}/lib"], capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-4000:]
    run = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stdout[-4000:] + run.stderr[-2000:]
    assert "0 failures" in run.stdout and "plans checked" in run.stdout, run.stdout[-2000:]


def test_statuses_raise_their_exceptions():
    """The Python side of the same mapping: out of memory is MemoryError, a backend failure RuntimeError with the
    library's message (the reference: Error::OutOfMemory / Error::Backend, crates/nuvec-core/src/error.rs:30-32)."""
    import pytest

    from nuvec_amd import _lib
    for status, exc in ((_lib.OUT_OF_MEMORY, MemoryError), (_lib.BACKEND, RuntimeError), (_lib.NO_DEVICE, RuntimeError)):
        with pytest.raises(exc):
            _lib.check(status)
    _lib.check(_lib.OK)
