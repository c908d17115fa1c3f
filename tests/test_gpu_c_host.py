"""The C ABI from a compiled host that is neither Python nor torch: `tests/c_host/matmul_host.c`.

What the Rust `Rocm` device would do through its FFI block -- create, allocate (zeroed and zero-deferred), copy in,
`matmat_forward` / `matmat_backward` on the literals of the reference's `test_matmul_normal`
(dfdx-core/src/tensor_ops/matmul/mod.rs:368-410), copy out, compare, use the allocation cache, walk the error codes,
destroy -- as a plain-C program built with gcc against `include/dfdx_rocm.h` and linked with `-ldfdx_rocm`.  The CPU
test builds it (header, link line and exported symbols agree); the GPU test runs it in a fresh child process.
"""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
SRC_DIR = os.path.join(HERE, "c_host")
EXE = os.path.join(SRC_DIR, "matmul_host")
LIB = os.path.join(os.path.dirname(HERE), "dfdx_amd", "lib", "libdfdx_rocm.so")


def test_c_host_builds_against_the_public_header(tmp_path):
    if not os.path.exists(LIB):
        pytest.skip("libdfdx_rocm.so is not built")
    out = tmp_path / "matmul_host"
    rocm_lib = "/opt/rocm/lib"
    cmd = ["gcc", "-std=c99", "-O1", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I" + os.path.join(os.path.dirname(HERE), "include"),
           os.path.join(SRC_DIR, "matmul_host.c"), "-o", str(out), "-L" + os.path.dirname(LIB), "-ldfdx_rocm", "-lm",
           "-Wl,-rpath-link," + rocm_lib]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    assert out.exists()


@pytest.mark.gpu
def test_c_host_runs_the_reference_literals():
    if not os.path.exists(EXE):   # normally built beforehand (make -C tests/c_host, or __graft_entry__.build())
        subprocess.check_call(["make", "-C", SRC_DIR])
    print("[gpu-case] c host program", EXE, flush=True)
    res = subprocess.run([EXE], capture_output=True, text=True, timeout=120)
    print(res.stdout)
    assert res.returncode == 0, f"exit {res.returncode}\n{res.stdout}\n{res.stderr}"
    assert "c host ok" in res.stdout
