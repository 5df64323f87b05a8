"""Callers written against the public headers alone, built by the host compilers: C99 programs on
the C ABI (tests/c_abi/ivf_pq_roundtrip.c, tests/c_abi/core_c_api.c) and C++17 programs on the C++
interface (tests/c_abi/ivf_pq_cpp_caller.cpp, tests/c_abi/ivf_pq_helpers.cpp).  Without a GPU: the headers compile (as pedantic C99 / C++17)
and the programs link against the library; on the GPU they run."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
PROGRAMS = {"ivf_pq_roundtrip": ("gcc", "-std=c99", "ivf_pq_roundtrip.c"),
            "core_c_api": ("gcc", "-std=c99", "core_c_api.c"),
            "ivf_pq_cpp_caller": ("g++", "-std=c++17", "ivf_pq_cpp_caller.cpp"),
            "ivf_pq_helpers": ("g++", "-std=c++17", "ivf_pq_helpers.cpp")}


def _compile(name, out):
    compiler, std, src = PROGRAMS[name]
    cmd = [compiler, std, "-Wall", "-Werror", "-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(ROOT, "include"),
           "-isystem", os.path.join(ROCM, "include"), os.path.join(ROOT, "tests", "c_abi", src),
           "-L" + os.path.join(ROOT, "cuvs_amd"), "-lcuvs_c", "-L" + os.path.join(ROCM, "lib"), "-lamdhip64",
           "-Wl,-rpath," + os.path.join(ROOT, "cuvs_amd"), "-Wl,-rpath," + os.path.join(ROCM, "lib"), "-o", out]
    done = subprocess.run(cmd, capture_output=True, text=True)
    assert done.returncode == 0, done.stderr


def test_headers_compile_as_c_and_the_programs_link(tmp_path):
    headers = ["cuvs/core/c_api.h", "cuvs/version_config.h", "cuvs/neighbors/ivf_pq.h", "cuvs/neighbors/refine.h",
               "cuvs/neighbors/knn_merge_parts.h"]
    probe = tmp_path / "probe.c"
    probe.write_text("".join(f"#include <{h}>\n" for h in headers) + "int main(void) { return 0; }\n")
    done = subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-D__HIP_PLATFORM_AMD__",
                           "-I" + os.path.join(ROOT, "include"), "-isystem", os.path.join(ROCM, "include"),
                           "-fsyntax-only", str(probe)], capture_output=True, text=True)
    assert done.returncode == 0, done.stderr
    for name in PROGRAMS:
        _compile(name, str(tmp_path / name))


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(PROGRAMS))
def test_program_runs(tmp_path, name):
    exe = str(tmp_path / name)
    _compile(name, exe)
    done = subprocess.run([exe, str(tmp_path / "index.bin")], capture_output=True, text=True, timeout=120)
    assert done.returncode == 0, done.stdout + done.stderr
    assert any(line.startswith("ok") for line in done.stdout.splitlines()), done.stdout
