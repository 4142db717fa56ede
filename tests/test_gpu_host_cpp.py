"""Runs the C++ host-side test program (tests/cpp/host_mirror_test.cpp over
include/ferrum_hip.hpp) on the GPU.  The binary is built with the libraries by
``__graft_entry__.build()``; it checks itself against the CPU oracle."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "cpp", "host_mirror_test")


@pytest.mark.gpu
def test_cpp_host_side_matches_the_oracle():
    if not os.path.exists(BINARY):
        from ferrum_amd import build
        build.build_host_test()
    proc = subprocess.run([BINARY], capture_output=True, text=True, timeout=150)
    print(proc.stdout)
    print(proc.stderr)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "0 failure(s)" in proc.stdout


def test_cpp_header_compiles_standalone(tmp_path):
    src = tmp_path / "probe.cpp"
    src.write_text('#include "ferrum_hip.hpp"\nint main() { return sizeof(ferrum::Device) == 0; }\n')
    include = os.path.join(os.path.dirname(HERE), "include")
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Werror", "-fsyntax-only", "-I" + include, str(src)], check=True)
