"""Builds libincin_rocm.so (HIP kernels + C ABI) for gfx950 with hipcc.

The library is built in-tree (incin_amd/lib/) so that it travels with the
source tree; nothing is installed.  `python -m incin_amd.build` rebuilds it.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libincin_rocm.so")
SOURCES = ["incin_rocm.hip", "sdpa_generic.hip", "sdpa_decode.hip", "sdpa_decode_mfma.hip", "sdpa_decode_f32.hip", "sdpa_prefill_mfma.hip", "sdpa_prefill_wide.hip", "sdpa_prefill_f32.hip", "sdpa_bwd_f32.hip", "mask_blocks.hip", "matrix_rate.hip", "copy.hip", "kv_append.hip", "sdpa_bwd_mfma.hip", "sdpa_bwd_generic.hip"]
# per-file flags.  The split-KV matrix-core kernel keeps its accumulators in ordinary vector registers: it rescales them
# only when a reference maximum moves, and with accumulation registers the compiler copies all of them out and back
# around that rare branch on every key block.
EXTRA_FLAGS = {"sdpa_decode_mfma.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"], "sdpa_decode_f32.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}
HOST_DIR = os.path.join(HERE, "host")
HOST_LIB = os.path.join(LIBDIR, "libincin_rocm_host.so")
HOST_SOURCES = ["rocm_backend.cpp", "rocm_capability.cpp", "rocm_exec.cpp", "rocm_backend_c.cpp"]
# test-side harness: the conformance suite, linked against the host library but not part of it
TEST_DIR = os.path.join(os.path.dirname(HERE), "tests", "native")
TEST_LIB = os.path.join(TEST_DIR, "libincin_rocm_conformance.so")
CXX = os.environ.get("CXX", "g++")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -packed-fp32-ops off: the compiler must not form packed-fp32 VALU instructions from float code.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _compile(src):
    """One source to one object.  The compiler's intermediate files are kept for the duration (in a directory of their own,
    removed afterwards) because one of them is the GPU assembly the object was made from: hazards.scan_asm reads it for
    inline copies that sit too close behind a vector write of one of their scalar operands - something the compiler cannot
    check, since it does not see the memory instruction inside the inline assembly."""
    from . import hazards
    name = os.path.splitext(src)[0]
    obj = os.path.join(LIBDIR, name + ".o")
    tmp = os.path.join(LIBDIR, "tmp_" + name)
    shutil.rmtree(tmp, ignore_errors=True)
    os.makedirs(tmp)
    try:
        tmp_obj = os.path.join(tmp, name + ".o")
        cmd = [HIPCC] + FLAGS + EXTRA_FLAGS.get(src, []) + ["-save-temps=obj", "-c", os.path.join(CSRC, src), "-o", tmp_obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, r.stdout, r.stderr))
        asm = [f for f in os.listdir(tmp) if f.endswith(".s") and "amdgcn" in f]
        if not asm:
            raise RuntimeError("no GPU assembly found for %s in %s" % (src, tmp))
        for f in asm:
            bad = hazards.check_file(os.path.join(tmp, f))
            if bad:
                raise RuntimeError("%s: inline copies fewer than %d wait states behind a vector write of a scalar operand:\n%s" % (
                    src, hazards.NEEDED, "\n".join("  %s line %d: %s  <-  %s  (%d wait states)" % b for b in bad)))
        os.replace(tmp_obj, obj)
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    return obj


def build_library(verbose=False):
    os.makedirs(LIBDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=4) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (r.stdout, r.stderr))
    if verbose:
        print("built", LIB)
    return LIB


def build_host_library(verbose=False):
    """C++ host mirror of the backend interface; plain host code that links against the C ABI library."""
    os.makedirs(LIBDIR, exist_ok=True)
    cmd = [CXX, "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-o", HOST_LIB]
    cmd += [os.path.join(HOST_DIR, f) for f in HOST_SOURCES]
    cmd += ["-L" + LIBDIR, "-lincin_rocm", "-Wl,-rpath,$ORIGIN"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("host library build failed:\n%s\n%s" % (r.stdout, r.stderr))
    if verbose:
        print("built", HOST_LIB)
    return HOST_LIB


def build_test_library(verbose=False):
    """The conformance harness of the tests (tests/native/), a library of its own beside the product libraries."""
    cmd = [CXX, "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-o", TEST_LIB, os.path.join(TEST_DIR, "rocm_conformance.cpp"),
           "-L" + LIBDIR, "-lincin_rocm_host", "-lincin_rocm", "-Wl,-rpath," + LIBDIR]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("conformance harness build failed:\n%s\n%s" % (r.stdout, r.stderr))
    if verbose:
        print("built", TEST_LIB)
    return TEST_LIB


if __name__ == "__main__":
    build_library(verbose=True)
    build_host_library(verbose=True)
    build_test_library(verbose=True)
    sys.exit(0)
