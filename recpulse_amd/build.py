"""Build librp_hip.so (the gfx950 device layer) in-tree with hipcc.

Every translation unit under csrc/ is cross-compiled for gfx950 and linked into
recpulse_amd/lib/librp_hip.so.  No GPU is needed to build.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
BUILD_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(LIB_DIR, "librp_hip.so")
SOURCES = ["rp_runtime.hip", "rp_elementwise.hip", "rp_gemm.hip", "rp_gemm_generic.hip", "rp_gemm_mfma16.hip", "rp_gemm_mfma16_256.hip",
           "rp_gemm_mfma16_128.hip", "rp_gemm_mfma16_64.hip", "rp_gemm_mfma16_64x256.hip", "rp_gemm_mfma16_64x128.hip", "rp_gemm_mfma16_skinny.hip", "rp_gemm_mfma16_stream128.hip", "rp_gemm_mfmaw.hip", "rp_gemm_tiny.hip", "rp_gemm_direct32.hip", "rp_gemm_pipe32.hip", "rp_gemm_pipe16.hip", "rp_gemm_pipe16k.hip", "rp_gemm_pipe32k.hip",
           "rp_attention.hip", "rp_attention_f32.hip", "rp_conv.hip", "rp_rnn.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed-fp32 code generation is switched off for all device code
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _flags_stamp(extra):
    """The compile line an object was built with, kept beside the objects: a change of flags rebuilds everything."""
    import hashlib
    return hashlib.sha256(" ".join([HIPCC] + FLAGS + list(extra)).encode()).hexdigest()


def _fresh(obj, src):
    """True when obj is newer than its source and every header under csrc/ and include/ (and the flags have not changed:
    build() clears the objects when they have).  Sources that include other .hip files are not tracked: none does."""
    if not os.path.exists(obj):
        return False
    t = os.path.getmtime(obj)
    deps = [os.path.join(CSRC, src)] + [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    deps.append(os.path.join(HERE, "..", "include", "rp_hip.h"))
    return all(os.path.getmtime(d) < t for d in deps)


def _compile(src, extra, force=True):
    obj = os.path.join(BUILD_DIR, src.replace(".hip", ".o"))
    if not force and _fresh(obj, src):
        return obj
    cmd = [HIPCC] + FLAGS + extra + ["-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(extra_flags=(), verbose=True, force=True):
    """Compile and link.  force=False recompiles only the translation units older than their sources (development loop)."""
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(BUILD_DIR, exist_ok=True)
    extra = list(extra_flags)
    stamp_path = os.path.join(BUILD_DIR, "flags.sha256")
    stamp = _flags_stamp(extra)
    if not force and (not os.path.exists(stamp_path) or open(stamp_path).read().strip() != stamp):
        force = True                                  # objects of another compile line
    with open(stamp_path, "w") as f:
        f.write(stamp + "\n")
    with ThreadPoolExecutor(max_workers=8) as ex:
        objs = list(ex.map(lambda s: _compile(s, extra, force), SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stderr)
    if verbose:
        print(f"built {LIB_PATH}")
    return LIB_PATH


HOST_DIR = os.path.join(HERE, "host")
DROPIN_DIR = os.path.join(HERE, "dropin")


def build_host(verbose=True, test_hooks=True):
    """Build the CPython extension `recpulse_cuda` (host tensor / autograd layer + pybind11 binding) into
    recpulse_amd/dropin/, linked against lib/librp_hip.so.  Plain g++: the host layer includes no HIP header.
    test_hooks compiles the fault-injection entry the error-path tests use (`_fail_gemm_after`); a build for
    deployment passes False and the symbol does not exist."""
    import sysconfig
    import pybind11
    os.makedirs(DROPIN_DIR, exist_ok=True)
    ext = sysconfig.get_config_var("EXT_SUFFIX")
    out = os.path.join(DROPIN_DIR, "recpulse_cuda" + ext)
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-Wall"] + (["-DRP_TEST_HOOKS"] if test_hooks else []) + [
           "-ffp-contract=off", "-I" + pybind11.get_include(), "-I" + sysconfig.get_paths()["include"],
           os.path.join(HOST_DIR, "rp_host.cpp"), os.path.join(HOST_DIR, "py_module.cpp"),
           "-o", out, "-L" + LIB_DIR, "-lrp_hip", "-Wl,-rpath,$ORIGIN/../lib"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("host extension build failed:\n" + res.stderr)
    if res.stderr.strip():
        sys.stderr.write(res.stderr)
    if verbose:
        print(f"built {out}")
    return out


if __name__ == "__main__":
    args = sys.argv[1:]
    incremental = "--incremental" in args
    build([a for a in args if a != "--incremental"], force=not incremental)
    build_host()
