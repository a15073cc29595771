"""Build recipe: compiles the HIP kernels for gfx950 and the C host library into
``alsparse_amd/lib/libalpha_spblas.so`` and the workload generators into
``alsparse_amd/lib/libasamd_workloads.so``.  hipcc cross-compiles without a GPU."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_DIR = os.path.join(ROOT, "alsparse_amd", "lib")
# ALSPARSE_AMD_LIB names another build of the same library (kernel experiments); there is no other fallback
LIB_PATH = os.environ.get("ALSPARSE_AMD_LIB") or os.path.join(LIB_DIR, "libalpha_spblas.so")
WORKLOADS_PATH = os.path.join(LIB_DIR, "libasamd_workloads.so")
PROBES_PATH = os.path.join(LIB_DIR, "libasamd_probes.so")


def _run(cmd, cwd=None):
    proc = subprocess.run(cmd, cwd=cwd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("build step failed: %s\n%s" % (" ".join(cmd), proc.stdout))
    return proc.stdout


def build_library(force=True, jobs=8):
    """Compile every HIP extension (always recompiles when ``force``)."""
    csrc = os.path.join(ROOT, "alsparse_amd", "csrc")
    if force:
        _run(["make", "-C", csrc, "clean"])
    _run(["make", "-C", csrc, "-j%d" % jobs])
    return LIB_PATH


def build_workloads():
    os.makedirs(LIB_DIR, exist_ok=True)
    src = os.path.join(ROOT, "alsparse_amd", "workloads", "workloads.c")
    _run(["gcc", "-std=c11", "-O2", "-fopenmp", "-fPIC", "-shared", "-Wall", "-o", WORKLOADS_PATH, src, "-lm"])
    return WORKLOADS_PATH


def build_probes():
    """The benchmark's plain memory kernels (stream / gather ceilings, the counter-calibration copy): a
    library of their own, so that nothing of them ships inside libalpha_spblas.so."""
    os.makedirs(LIB_DIR, exist_ok=True)
    src = os.path.join(ROOT, "alsparse_amd", "probes", "ceilings.hip")
    _run(["/opt/rocm/bin/hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
          "-I" + os.path.join(ROOT, "alsparse_amd", "probes"), "-o", PROBES_PATH, src])
    return PROBES_PATH


def build_oracle():
    """Compile the CPU oracle (test infrastructure) and, when the reference tree
    is present, the reference's own CPU kernels and its own test programs of this path
    (unchanged sources, linked against this library) into oracle/_ref/."""
    _run(["make", "-C", os.path.join(ROOT, "oracle")])
    if os.path.isdir("/root/reference/test") and os.path.exists(LIB_PATH):
        _run(["make", "-C", os.path.join(ROOT, "oracle"), "ref_drivers"])


def build_c_api_program(sanitized=True, jobs=8):
    """Compile the C lifecycle program of the test suite against the freshly built library, and (sanitized)
    the same program with a copy of the library whose host code carries ASan + UBSan: the test that runs it
    refuses a copy made from other sources than the present ones, so it is made whenever the library is."""
    _run(["make", "-C", os.path.join(ROOT, "tests", "c_api")])
    if sanitized:
        _run(["make", "-C", os.path.join(ROOT, "tests", "c_api"), "-j%d" % jobs, "asan"])
