"""A plain C program against the public headers (tests/c_api/lifecycle.c): handles, descriptors and
info bundles through their whole lifecycle, stale analysis records under freed and reallocated
device arrays, all four element types, results checked on the CPU inside the program.  Built by
`make -C tests/c_api` (the package's build step runs it).  When `make -C tests/c_api asan` was run
as well, the same program is run against the library built with ASan + UBSan on its host code."""
import glob
import hashlib
import os
import subprocess

import pytest

from helpers import announce

pytestmark = pytest.mark.gpu
BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c_api", "bin")


def run(exe, env=None):
    announce("C program", exe)
    r = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300, env=env)
    assert r.returncode == 0, r.stdout[-3000:]
    assert "lifecycle: all passed" in r.stdout, r.stdout[-3000:]
    assert "runtime error" not in r.stdout and "AddressSanitizer" not in r.stdout, r.stdout[-3000:]


def test_c_lifecycle_program(gpu):
    exe = os.path.join(BIN, "lifecycle")
    if not os.path.exists(exe):
        pytest.skip("tests/c_api/bin/lifecycle was not built (make -C tests/c_api)")
    run(exe)


def test_c_lifecycle_program_with_host_sanitizers(gpu):
    exe = os.path.join(BIN, "asan", "lifecycle")
    if not os.path.exists(exe):
        pytest.skip("the sanitized build is optional (make -C tests/c_api asan)")
    # the build keeps the digest of the sources it was made from (the Makefile's SAN_SOURCES, in byte order)
    root = os.path.abspath(os.path.join(os.path.dirname(BIN), "..", ".."))
    csrc = os.path.join(root, "alsparse_amd", "csrc")
    files = []
    for pattern in ("host/*.c", "host/*.h", "hip/*.hip", "hip/*.hpp"):
        files += glob.glob(os.path.join(csrc, pattern))
    files += glob.glob(os.path.join(root, "include", "*.h")) + [os.path.join(os.path.dirname(BIN), "lifecycle.c")]
    digest = hashlib.sha256()
    for f in sorted(files):
        with open(f, "rb") as fh:
            digest.update(fh.read())
    stamp = os.path.join(BIN, "asan", "sources.sha256")
    if not os.path.exists(stamp) or open(stamp).read().strip() != digest.hexdigest():
        pytest.skip("the sanitized build was made from other sources than the present ones (make -C tests/c_api asan)")
    env = dict(os.environ)
    # the GPU runtime maps memory where the sanitizer would put its shadow gap; leaks of the GPU
    # runtime's own start-up allocations are not this library's
    env["ASAN_OPTIONS"] = "detect_leaks=0:protect_shadow_gap=0:halt_on_error=1"
    env["UBSAN_OPTIONS"] = "print_stacktrace=1:halt_on_error=1"
    run(exe, env)
