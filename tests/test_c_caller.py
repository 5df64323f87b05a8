"""A C99 program against the public headers: they must compile as C, link against the library, and
(on the GPU) carry a build / search / save / load / search round trip (tests/c_abi/ivf_pq_roundtrip.c)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "c_abi", "ivf_pq_roundtrip.c")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


def _compile(out):
    cmd = ["gcc", "-std=c99", "-Wall", "-Werror", "-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(ROOT, "include"),
           "-I" + os.path.join(ROCM, "include"), SRC, "-L" + os.path.join(ROOT, "cuvs_amd"), "-lcuvs_c",
           "-L" + os.path.join(ROCM, "lib"), "-lamdhip64", "-Wl,-rpath," + os.path.join(ROOT, "cuvs_amd"),
           "-Wl,-rpath," + os.path.join(ROCM, "lib"), "-o", out]
    subprocess.run(cmd, check=True, capture_output=True, text=True)


def test_headers_compile_as_c_and_the_program_links(tmp_path):
    headers = ["cuvs/core/c_api.h", "cuvs/neighbors/ivf_pq.h", "cuvs/neighbors/refine.h",
               "cuvs/neighbors/knn_merge_parts.h"]
    probe = tmp_path / "probe.c"
    probe.write_text("".join(f"#include <{h}>\n" for h in headers) + "int main(void) { return 0; }\n")
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-D__HIP_PLATFORM_AMD__",
                    "-I" + os.path.join(ROOT, "include"), "-isystem", os.path.join(ROCM, "include"),
                    "-fsyntax-only", str(probe)], check=True, capture_output=True, text=True)
    _compile(str(tmp_path / "ivf_pq_roundtrip"))


@pytest.mark.gpu
def test_c_program_round_trip(tmp_path):
    exe = str(tmp_path / "ivf_pq_roundtrip")
    _compile(exe)
    done = subprocess.run([exe, str(tmp_path / "index.bin")], capture_output=True, text=True, timeout=120)
    assert done.returncode == 0, done.stdout + done.stderr
    assert done.stdout.startswith("ok")
