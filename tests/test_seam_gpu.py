"""The reference's device seam as compiled code: paperkiln_amd/adapter/microtorch_hip_seam.cpp stands in for
src/device.cpp + src/device_cache.cpp of the reference. The CPU half checks that the adapter compiles against the
reference's own headers (only where the reference tree is present); the GPU half runs oracle/_ref/seam_check, the
reference's untouched tape sources linked with the adapter and libpaperkiln_amd.so (built by oracle/Makefile where
the reference tree is present; the binary travels, the reference does not)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference"
EXE = os.path.join(ROOT, "oracle", "_ref", "seam_check")


def test_adapter_compiles_against_the_reference_headers():
    if not os.path.isdir(os.path.join(REF, "include", "microtorch")):
        pytest.skip("reference tree absent")
    subprocess.check_call(["g++", "-std=c++17", "-fsyntax-only", "-w", "-I", os.path.join(REF, "include"),
                           "-I", os.path.join(REF, "third_party", "transformer_cpp", "include"),
                           "-I", os.path.join(ROOT, "include"),
                           os.path.join(ROOT, "paperkiln_amd", "adapter", "microtorch_hip_seam.cpp")])


@pytest.mark.gpu
def test_reference_tape_over_the_hip_seam():
    if not os.path.exists(EXE):
        pytest.skip("oracle/_ref/seam_check not built (reference tree absent at build time)")
    out = subprocess.run([EXE], capture_output=True, text=True, timeout=300)
    print(out.stdout[-6000:], out.stderr[-1000:], flush=True)
    assert out.returncode == 0 and "seam_check PASSED" in out.stdout
