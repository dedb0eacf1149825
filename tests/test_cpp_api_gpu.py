"""The C++ tape interface (include/paperkiln_amd.hpp) exercised by a C++ program that links the shared library:
tests/cpp/tape_api_check.cpp, built by __graft_entry__.build() with plain g++. The CPU half checks that the header
stands on its own; the GPU half runs the program."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "tape_api_check")


def test_public_cpp_header_needs_no_hip_header(tmp_path):
    """`#include "paperkiln_amd.hpp"` alone compiles with g++ and no ROCm include path."""
    src = tmp_path / "only_header.cpp"
    src.write_text('#include "paperkiln_amd.hpp"\n'
                   "pk::Var (*fa)(const pk::Var&, const pk::Var&, const pk::Var&, float, int64_t, bool) = "
                   "&pk::ops::fused_attention;\n"
                   "pk::Var (*ck)(const std::function<pk::Var(const pk::Var&)>&, const pk::Var&) = &pk::checkpoint;\n"
                   "int main() { return fa && ck ? 0 : 1; }\n")
    subprocess.check_call(["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src)])


@pytest.mark.gpu
def test_cpp_program_against_the_shared_library():
    if not os.path.exists(EXE):
        pytest.fail(f"{EXE} not built: run __graft_entry__.build()")
    out = subprocess.run([EXE], capture_output=True, text=True, timeout=120)
    print(out.stdout[-3000:], out.stderr[-1000:], flush=True)
    assert out.returncode == 0 and "tape_api_check PASSED" in out.stdout
