"""Builds librllama_hip.so (the C-ABI library with the gfx950 kernels) in-tree with hipcc.

    python -m rllama_amd.build [--force]

The library lands next to this file so that it travels with the source tree; nothing is installed.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "_obj")
LIB = os.path.join(HERE, "librllama_hip.so")

SOURCES = ["gemv.hip", "attention.hip", "gemm.hip", "gemm_dma.hip", "gemm_kgroup.hip", "attn_prefill.hip", "prefill.hip", "prefill_f32.hip", "misc.hip", "sampler.hip", "api.hip", "api_ops.hip"]
HEADERS = ["kernels.h", "device_utils.h", "gemv_device.h", "gemm_epilogue.h", "synth.h", "api_internal.h", os.path.join("..", "..", "include", "rllama_hip.h")]  # relative to csrc/

HIPCC = os.environ.get("HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    # packed fp32 instructions are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _sources():
    return [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]


def _stale() -> bool:
    if not os.path.exists(LIB):
        return True
    t = os.path.getmtime(LIB)
    deps = [os.path.join(CSRC, s) for s in _sources()] + [os.path.join(CSRC, h) for h in HEADERS] + [__file__]
    return any(os.path.exists(d) and os.path.getmtime(d) > t for d in deps)


def _compile(src: str) -> str:
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + r.stdout + r.stderr)
    warn = "\n".join(l for l in (r.stdout + r.stderr).splitlines() if "packed-fp32-ops" not in l and l.strip())
    if warn:
        sys.stderr.write(warn + "\n")
    return obj


def build(force: bool = False) -> str:
    if not force and not _stale():
        return LIB
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=4) as ex:
        objs = list(ex.map(_compile, _sources()))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs, "-lpthread"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + " ".join(cmd) + "\n" + r.stdout + r.stderr)
    return LIB


HOST_BIN = os.path.join(HERE, "host", "rllama_generate")


def build_host(force: bool = False) -> str:
    """Compiles the C++ host example (header-only mirror of the reference API + the token loop) against the library."""
    src = os.path.join(HERE, "host", "generate_main.cpp")
    hdrs = [os.path.join(HERE, "host", h) for h in ("rllama_hip.hpp", "model_files.hpp", "tokenizer.hpp", "file_tools.hpp")]
    if not force and os.path.exists(HOST_BIN) and all(os.path.getmtime(HOST_BIN) >= os.path.getmtime(f) for f in (src, *hdrs, LIB)):
        return HOST_BIN
    cmd = ["g++", "-O2", "-std=c++17", "-Wall", "-Wextra", src, "-o", HOST_BIN, "-L" + HERE, "-lrllama_hip", "-Wl,-rpath,$ORIGIN/.."]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("host build failed:\n" + " ".join(cmd) + "\n" + r.stdout + r.stderr)
    return HOST_BIN


ASAN_BIN = os.path.join(HERE, "host", "rllama_check_files_asan")
ASAN_FLAGS = ["-O1", "-g", "-fno-omit-frame-pointer", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-static-libasan", "-static-libubsan"]


def build_host_asan(force: bool = False) -> str:
    """The host-only file readers (pickle subset, params.json, shard joining, tokenizer model file) as a program built with
    AddressSanitizer and UndefinedBehaviorSanitizer.  CPU code only: nothing of the device library is in it."""
    src = os.path.join(HERE, "host", "check_files_main.cpp")
    hdrs = [os.path.join(HERE, "host", h) for h in ("rllama_hip.hpp", "model_files.hpp", "tokenizer.hpp", "file_tools.hpp")]
    if not force and os.path.exists(ASAN_BIN) and all(os.path.getmtime(ASAN_BIN) >= os.path.getmtime(f) for f in (src, *hdrs)):
        return ASAN_BIN
    cmd = ["g++", *ASAN_FLAGS, "-std=c++17", "-Wall", "-Wextra", src, "-o", ASAN_BIN]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("sanitizer build of the host readers failed:\n" + " ".join(cmd) + "\n" + r.stdout + r.stderr)
    return ASAN_BIN


if __name__ == "__main__":
    if "--host-asan" in sys.argv:
        print(build_host_asan(force=True))
    else:
        print(build(force="--force" in sys.argv))
        print(build_host(force="--force" in sys.argv))
