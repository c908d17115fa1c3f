"""CPU-side checks of the C-ABI boundary: the shared library loads, exports every symbol that
include/dfdx_rocm.h declares (and nothing is declared that is not exported), the ctypes mirror of the
descriptor struct has the C layout, and calls fail cleanly -- never crash -- without a GPU."""
import ctypes
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "dfdx_rocm.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dfdx_rocm_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_all_exported():
    from dfdx_amd.rocm import EXPORTS, load_library

    lib = load_library()
    declared = declared_symbols()
    assert len(declared) >= 20
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in dfdx_rocm.h but not exported"
    assert sorted(EXPORTS) == declared, "python binding list and header disagree"


def test_integration_binding_lists_every_symbol():
    """INTEGRATION.md's Rust `extern "C"` block declares every exported symbol except the four test / tooling aids it
    names as left out."""
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    block = text[text.index('extern "C" {'):]
    block = block[:block.index("```")]
    bound = set(re.findall(r"pub fn (dfdx_rocm_[a-z0-9_]+)\(", block))
    left_out = {"dfdx_rocm_gemm_plan", "dfdx_rocm_gemm_time", "dfdx_rocm_gemm_time_rotating", "dfdx_rocm_mfma_variant_count", "dfdx_rocm_cache_stats"}
    assert bound == set(declared_symbols()) - left_out
    for name in left_out:
        assert name in text[:text.index('extern "C" {')]   # named where the binding says what it leaves out


def test_every_declaration_cites_the_reference():
    """Each block of declarations names the reference interface it replaces (file:line)."""
    text = open(HEADER).read()
    for needle in ("cpu_kernel.rs:38-50", "cuda_kernel.rs:153-181", "matmul/mod.rs:116-131", "matmul/mod.rs:197-212",
                   "matmul/mod.rs:234-249", "matmul/mod.rs:273-288", "linear.rs:82-89", "cuda/device.rs:259-266",
                   "bias1d.rs:62-78", "utilities/cpu_kernels.rs:164-203", "softmax.rs:70-83", "mul/cpu_kernel.rs:\n * 5-17",
                   "reshape_to/mod.rs:90-115", "conv2d/mod.rs:31-55", "multi_head_attention.rs:\n * 105-146",
                   "storage_traits.rs:41-77", "tensor/cache.rs:36-149"):
        assert needle in text, needle


def test_desc_struct_layout_matches_c(tmp_path):
    from dfdx_amd.rocm import GemmDesc

    src = tmp_path / "layout.c"
    src.write_text(
        '#include <stdio.h>\n#include <stddef.h>\n#include "dfdx_rocm.h"\n'
        "int main(void){printf(\"%zu %zu %zu %zu %zu %zu %zu\\n\", sizeof(dfdx_rocm_gemm_desc),"
        "offsetof(dfdx_rocm_gemm_desc,m), offsetof(dfdx_rocm_gemm_desc,a), offsetof(dfdx_rocm_gemm_desc,b),"
        "offsetof(dfdx_rocm_gemm_desc,c), offsetof(dfdx_rocm_gemm_desc,bias), offsetof(dfdx_rocm_gemm_desc,kernel));return 0;}\n")
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    got = [int(x) for x in subprocess.check_output([str(exe)]).split()]
    want = [ctypes.sizeof(GemmDesc), GemmDesc.m.offset, GemmDesc.a.offset, GemmDesc.b.offset, GemmDesc.c.offset,
            GemmDesc.bias.offset, GemmDesc.kernel.offset]
    assert got == want


def test_conv2d_op_layout_matches_c(tmp_path):
    """dfdx_rocm_conv2d_op is twelve size_t in the reference's field order (conv2d/mod.rs:14-29)."""
    from dfdx_amd.rocm import Conv2DOp

    src = tmp_path / "conv.c"
    src.write_text(
        '#include <stdio.h>\n#include <stddef.h>\n#include "dfdx_rocm.h"\n'
        "int main(void){printf(\"%zu %zu %zu %zu %zu\\n\", sizeof(dfdx_rocm_conv2d_op), offsetof(dfdx_rocm_conv2d_op,kernel),"
        "offsetof(dfdx_rocm_conv2d_op,groups), offsetof(dfdx_rocm_conv2d_op,chan_in), offsetof(dfdx_rocm_conv2d_op,w_out));return 0;}\n")
    exe = tmp_path / "conv"
    subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    got = [int(x) for x in subprocess.check_output([str(exe)]).split()]
    assert got == [ctypes.sizeof(Conv2DOp), Conv2DOp.kernel.offset, Conv2DOp.groups.offset, Conv2DOp.chan_in.offset,
                   Conv2DOp.w_out.offset]
    assert [n for n, _ in Conv2DOp._fields_] == ["kernel", "stride", "padding", "dilation", "groups", "batch", "chan_in",
                                                 "chan_out", "h_in", "h_out", "w_in", "w_out"]


def test_header_compiles_as_c_and_cxx(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#include "dfdx_rocm.h"\nint main(void){return DFDX_ROCM_OK;}\n')
    subprocess.check_call(["gcc", "-std=c99", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", str(src),
                           "-o", str(tmp_path / "t.o")])
    subprocess.check_call(["g++", "-std=c++11", "-Werror", "-I", os.path.join(ROOT, "include"), "-x", "c++", "-c", str(src),
                           "-o", str(tmp_path / "t2.o")])


def test_calls_fail_cleanly_without_a_device():
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from dfdx_amd import Rocm
    from dfdx_amd.rocm import load_library

    lib = load_library()
    ctx = ctypes.c_void_p()
    assert lib.dfdx_rocm_create(0, None, ctypes.byref(ctx)) == -3  # DFDX_ROCM_ERR_NO_DEVICE
    assert ctx.value is None
    assert lib.dfdx_rocm_gemm(None, None) == -1
    assert lib.dfdx_rocm_synchronize(None) == -1
    # the entry points around the matmuls refuse a null context the same way
    i64, vp = ctypes.c_int64, ctypes.c_void_p
    assert lib.dfdx_rocm_bias_forward(None, 0, i64(1), i64(1), vp(), vp(), vp()) == -1
    assert lib.dfdx_rocm_bias_backward(None, 0, i64(1), i64(1), vp(), vp()) == -1
    assert lib.dfdx_rocm_softmax_forward(None, 0, i64(1), i64(1), vp(), ctypes.c_float(1.0), vp()) == -1
    assert lib.dfdx_rocm_reshape_forward(None, 0, 1, vp(), vp(), vp(), vp()) == -1
    assert lib.dfdx_rocm_scalar_mul_forward(None, 0, i64(1), vp(), ctypes.c_double(1.0), vp()) == -1
    assert lib.dfdx_rocm_conv2d_forward(None, 0, vp(), vp(), vp(), vp()) == -1
    assert b"gfx950" in lib.dfdx_rocm_strerror(-3)
    assert lib.dfdx_rocm_mfma_variant_count(1) >= 6
    with pytest.raises(RuntimeError):  # the Python mirror refuses too: there is no CPU fallback
        Rocm(0)


def test_product_code_does_not_touch_the_oracle():
    """Nothing under dfdx_amd/ or include/ may import, load or name the oracle."""
    for base in ("dfdx_amd", "include"):
        for dirpath, _, files in os.walk(os.path.join(ROOT, base)):
            for f in files:
                if f.endswith((".py", ".cpp", ".hip", ".h", "Makefile")):
                    text = open(os.path.join(dirpath, f), errors="ignore").read()
                    assert "oracle" not in text.lower(), os.path.join(dirpath, f)
