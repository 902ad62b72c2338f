"""The C++ host side above the C ABI (include/jitllm_hip.hpp): it compiles as strict C++17 on its
own, and a C++ program that uses the reference's projection seams through it
(tests/cpp/host_mirror_check.cpp, built by __graft_entry__.build()) holds every result to the CPU
oracle on a GPU, or -- without one -- gets the library's errors as exceptions."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "_build", "host_mirror_check")


def built():
    if not os.path.exists(EXE):
        import sys
        sys.path.insert(0, ROOT)
        from oracle import pyoracle
        pyoracle.build(force=False)
        import __graft_entry__ as entry
        entry.build_cpp_host_check()
    return EXE


def test_the_header_is_strict_cxx17_on_its_own(tmp_path):
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("no C++ compiler")
    src = tmp_path / "only_the_header.cpp"
    src.write_text('#include "jitllm_hip.hpp"\nint main() { return jitllm::check(0), 0; }\n')
    subprocess.run([gxx, "-std=c++17", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only",
                    "-I", os.path.join(ROOT, "include"), str(src)], check=True)


def test_errors_arrive_as_exceptions_without_a_device():
    if os.path.exists("/dev/kfd"):
        pytest.skip("a GPU is present: the parity run covers the binary")
    out = subprocess.run([built(), "--no-device"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert out.stdout.count(" ok") == 4 and "FAILED" not in out.stdout


@pytest.mark.gpu
def test_cpp_host_holds_every_projection_to_the_oracle():
    print("[gpu-case] C++ host mirror check", flush=True)
    out = subprocess.run([built()], capture_output=True, text=True, timeout=300)
    print(out.stdout[-6000:])
    assert out.returncode == 0, out.stdout[-4000:] + out.stderr[-2000:]
    assert "[cpp-host] all ok" in out.stdout and "FAILED" not in out.stdout
    assert out.stdout.count("[cpp-host]") > 40
