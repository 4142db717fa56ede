"""Builds libferrum_hip.so (gfx950 only) from ferrum_amd/csrc with hipcc.

Run as ``python -m ferrum_amd.build``.  Objects land in ``ferrum_amd/build/``
and the shared library in ``ferrum_amd/lib/``; both are git-ignored.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys

from . import isa_check

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libferrum_hip.so")

SOURCES = ["capi.hip", "dequant.hip", "gemv.hip", "gemv_stream.hip", "probe.hip", "gemm.hip", "gemm_skinny.hip", "moe.hip", "norm.hip"]

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    # packed-f32 VALU forms stay off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def _compile(src: str, extra: list[str]) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc(), *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{proc.stdout}\n{proc.stderr}")
    warnings = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l).strip()
    if warnings:
        sys.stderr.write(warnings + "\n")
    return obj


def _assembly(src: str, extra: list[str]) -> str:
    """The device assembly hipcc writes for one of this library's sources, as text."""
    out = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".s")
    cmd = [hipcc(), *[f for f in FLAGS if f != "-fPIC"], *extra, "-S", "--offload-device-only",
           os.path.join(CSRC, src), "-o", out]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc -S failed for {src}:\n{proc.stdout}\n{proc.stderr}")
    with open(out) as f:
        return f.read()


def check_toolchain() -> str:
    """The hipcc release in use; a release other than the validated one is reported on stderr
    (the check of the generated code below and the GPU parity tests are then the gate)."""
    proc = subprocess.run([hipcc(), "--version"], capture_output=True, text=True)
    release = isa_check.hipcc_release(proc.stdout)
    if release != isa_check.VALIDATED_HIPCC:
        sys.stderr.write(f"ferrum_amd.build: hipcc {release or '(unknown)'} is not the release the hand-scheduled kernels "
                         f"were validated with ({isa_check.VALIDATED_HIPCC}); run the GPU parity tests before use\n")
    return release


def build(extra_flags: list[str] | None = None, jobs: int = 8, output: str | None = None) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    extra = list(extra_flags or [])
    check_toolchain()
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        # the sources with hand-scheduled loads are also compiled to assembly text, which is checked
        # for what the compiler must not have done around those loads
        texts = {s: pool.submit(_assembly, s, extra) for s in isa_check.CHECKED_SOURCES}
        objs = list(pool.map(lambda s: _compile(s, extra), SOURCES))
        broken = [v for s, t in texts.items() for v in isa_check.violations(t.result(), s)]
    if broken:
        raise RuntimeError("the generated code breaks an invariant of the hand-scheduled loads:\n" + "\n".join(broken[:40]))
    target = output or LIB_PATH
    tmp = target + ".tmp"
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, target)
    return target


def build_host_test() -> str:
    """Compiles the C++ host-side test (g++, no HIP headers needed) against the
    built library and the CPU oracle; the GPU test suite runs the binary."""
    root = os.path.dirname(HERE)
    src = os.path.join(root, "tests", "cpp", "host_mirror_test.cpp")
    out = os.path.join(root, "tests", "cpp", "host_mirror_test")
    cmd = ["g++", "-std=c++17", "-O2", "-Wall", "-I" + os.path.join(root, "include"), src, "-o", out,
           "-L" + LIB_DIR, "-lferrum_hip", "-L" + os.path.join(root, "oracle"), "-lferrum_oracle",
           "-Wl,-rpath,$ORIGIN/../../ferrum_amd/lib", "-Wl,-rpath,$ORIGIN/../../oracle",
           "-Wl,-rpath,/opt/rocm/lib"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"g++ failed for the host test:\n{proc.stdout}\n{proc.stderr}")
    return out


def build_gguf_probe(sanitize: bool = False) -> str:
    """Compiles tests/cpp/gguf_probe.cpp (the C++ GGUF reader's CPU test
    program; host code only, nothing to link).  `sanitize` builds a second
    binary under AddressSanitizer and UBSan, any report of which is fatal."""
    root = os.path.dirname(HERE)
    out = os.path.join(root, "tests", "cpp", "gguf_probe_san" if sanitize else "gguf_probe")
    flags = ["-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all"] if sanitize else ["-O2"]
    cmd = ["g++", "-std=c++17", *flags, "-Wall", "-Werror", "-I" + os.path.join(root, "include"),
           os.path.join(root, "tests", "cpp", "gguf_probe.cpp"), "-o", out]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"g++ failed for the GGUF probe:\n{proc.stdout}\n{proc.stderr}")
    return out


if __name__ == "__main__":
    print(build(sys.argv[1:]))
