"""The C++ twin tests (bare-cuda-4gib_amd/csrc/twin): every kernel family of the library beside a plain C++
reference, in a program of its own that links the library as any C program would -- no Python, no torch between
the test and the kernels.  Here the program is run family by family; twin/CMakeLists.txt registers the same
families with ctest."""
import os
import re
import subprocess

import pytest

from bare_cuda_4gib_amd.csrc import build

FAMILIES = ["embed", "rmsnorm", "swiglu", "gemm_generic", "gemm_skinny", "gemm_skinny_norms", "gemm_mfma",
            "attention_generic", "attention_mfma", "qkv_fused", "argmax", "sampling"]


def program() -> str:
    path = build.twins_path()
    if not os.path.exists(path):
        build.build_twins(verbose=True)
    return path


def test_the_families_are_the_same_everywhere():
    """The program's own list, ctest's list and this file's are one list."""
    if not build.is_built():
        pytest.skip("the kernel library is not built here")
    listed = subprocess.run([program(), "--list"], capture_output=True, text=True, timeout=60)
    assert listed.returncode == 0 and listed.stdout.split() == FAMILIES
    cmake = open(os.path.join(build.TWIN_DIR, "CMakeLists.txt")).read()
    in_cmake = re.search(r"foreach\(family IN ITEMS ([^)]*)\)", cmake).group(1).split()
    assert in_cmake == FAMILIES


@pytest.mark.gpu
@pytest.mark.parametrize("family", FAMILIES)
def test_kernels_beside_their_cpp_twins(family):
    done = subprocess.run([program(), family], capture_output=True, text=True, timeout=110)
    assert done.returncode == 0 and f"PASS: {family}" in done.stdout, done.stdout[-3000:] + done.stderr[-2000:]


@pytest.mark.gpu
def test_a_name_the_program_does_not_know():
    done = subprocess.run([program(), "no_such_family"], capture_output=True, text=True, timeout=60)
    assert done.returncode == 2 and "--list" in done.stdout
