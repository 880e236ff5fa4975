"""Builds libstingray_sampler.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

Usage: python -m opentail.stingray_amd.build [--force] [--hooks | --profile]
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "_obj")
LIB_DIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIB_DIR, "libstingray_sampler.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -ffp-contract=off: the managed sampler never fuses a*b+c, so neither may the kernels (the few fused
# operations are written as explicit fma intrinsics).  Packed-fp32 code generation is switched off.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-ffp-contract=off", "-fno-fast-math",
    "-fvisibility=hidden", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
SOURCES = ["sr_api.cpp", "sr_full_host.cpp", "sr_topk.hip", "sr_argmax.hip", "sr_full.hip"]


def _deps():
    return [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")] + [
        os.path.join(HERE, "..", "..", "include", "stingray_sampler.h")]


def _variant(profile: bool, hooks: bool) -> str:
    return "_prof" if profile else ("_hooks" if hooks else "")


def _compile(src: str, force: bool, profile: bool = False, hooks: bool = False) -> str:
    obj = os.path.join(OBJ + _variant(profile, hooks), os.path.splitext(src)[0] + ".o")
    path = os.path.join(CSRC, src)
    newest = max(os.path.getmtime(p) for p in [path] + _deps())
    if not force and os.path.exists(obj) and os.path.getmtime(obj) >= newest:
        return obj
    defs = (["-DSR_PROFILE"] if profile else []) + (["-DSR_TEST_HOOKS"] if (hooks or profile) else [])
    cmd = [HIPCC] + FLAGS + defs + ["-x", "hip", "-c", path, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    return obj


def build(force: bool = False, profile: bool = False, hooks: bool = False) -> str:
    """The product library exports the entry points of include/stingray_sampler.h and nothing else.
    hooks=True builds libstingray_sampler_hooks.so instead: the same sources with the test and measurement hooks of
    include/stingray_sampler_test.h compiled in (-DSR_TEST_HOOKS); the tests call its hooks on contexts and batches of
    the product library (tests/helpers.py).  profile=True builds libstingray_sampler_prof.so: the hooks plus the
    kernels' phase timestamps (-DSR_PROFILE; sr_debug_set_profile).  STINGRAY_SAMPLER_LIB=<path> makes the Python
    mirror load another build."""
    os.makedirs(OBJ + _variant(profile, hooks), exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    lib = LIB.replace(".so", "_prof.so") if profile else (LIB.replace(".so", "_hooks.so") if hooks else LIB)
    with ThreadPoolExecutor(max_workers=4) as ex:
        objs = list(ex.map(lambda s: _compile(s, force, profile, hooks), SOURCES))
    if force or not os.path.exists(lib) or any(os.path.getmtime(o) > os.path.getmtime(lib) for o in objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    return lib


CPP_TEST_SRC = os.path.join(HERE, "..", "..", "tests", "cpp", "host_mirror_test.cpp")
CPP_TEST_BIN = os.path.join(HERE, "..", "..", "tests", "cpp", "host_mirror_test")


def build_cpp_test(oracle_lib: str) -> str:
    """Compiles the C++ host-mirror test (g++; links the C ABI library and, as its checker, the oracle)."""
    root = os.path.normpath(os.path.join(HERE, "..", ".."))
    cmd = ["g++", "-std=c++17", "-O1", "-o", os.path.normpath(CPP_TEST_BIN), os.path.normpath(CPP_TEST_SRC),
           "-I" + os.path.join(root, "include"), "-I" + os.path.join(root, "oracle"),
           "-I/opt/rocm/include", "-D__HIP_PLATFORM_AMD__", "-L/opt/rocm/lib", "-lamdhip64",
           "-L" + LIB_DIR, "-lstingray_sampler", "-L" + os.path.dirname(os.path.abspath(oracle_lib)), "-lstingray_oracle",
           "-Wl,-rpath,$ORIGIN/../../opentail/stingray_amd/lib", "-Wl,-rpath,$ORIGIN/../../oracle/_build",
           "-Wl,-rpath,/opt/rocm/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"g++ failed for the host-mirror test:\n{r.stdout}\n{r.stderr}")
    return os.path.normpath(CPP_TEST_BIN)


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, profile="--profile" in sys.argv, hooks="--hooks" in sys.argv))
