"""The host side of the C ABI (argument checks, launch plumbing) under AddressSanitizer + UBSan.

The library is rebuilt with the host pass instrumented (device code as usual) and tests/test_abi.py runs against
that build in a child process with the sanitizer runtime preloaded. Any report fails the run: ASan aborts the
process, UBSan is told to halt."""

import os
import subprocess
import sys

import pytest

from verl_amd import build as hip_build

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_abi_host_checks_under_asan_and_ubsan(tmp_path):
    try:
        runtime = hip_build.asan_runtime()
    except RuntimeError as exc:
        pytest.skip(str(exc))
    lib = hip_build.build(verbose=False, sanitize_host=True, out_path=str(tmp_path / "libvrl_hip_hostsan.so"))
    nm = subprocess.run(["nm", "-D", "--undefined-only", lib], stdout=subprocess.PIPE, text=True)
    assert "__asan_init" in nm.stdout and "__ubsan_handle" in nm.stdout, "the host pass was not instrumented"
    env = dict(os.environ)
    env["LD_PRELOAD"] = runtime + (":" + env["LD_PRELOAD"] if env.get("LD_PRELOAD") else "")
    env["ASAN_OPTIONS"] = "detect_leaks=0:abort_on_error=1"      # the interpreter's own allocations are not ours to judge
    env["UBSAN_OPTIONS"] = "halt_on_error=1:print_stacktrace=1"
    env["VERL_AMD_LIB"] = lib
    out = subprocess.run([sys.executable, "-m", "pytest", os.path.join(REPO, "tests", "test_abi.py"), "-x", "-q",
                          "-p", "no:cacheprovider"], cwd=REPO, env=env, stdout=subprocess.PIPE,
                         stderr=subprocess.STDOUT, text=True, timeout=600)
    assert out.returncode == 0, out.stdout[-4000:]
    assert "passed" in out.stdout and "ERROR: AddressSanitizer" not in out.stdout and "runtime error" not in out.stdout
