"""The C-ABI library loads without a GPU and exports exactly what include/bmt_hip.h declares;
the ctypes face offers the names bmtrain.C has on this path.  No GPU launcher is called."""
import ctypes
import os
import re

import pytest

from conftest import ROOT

HEADER = os.path.join(ROOT, "include", "bmt_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"BMT_API\s+[\w\s\*]+?\b(\w+)\s*\(", text)))


def test_header_declares_the_hot_path_surface():
    names = declared_symbols()
    for stem in ("has_nan_inf", "adam", "adam_cpu", "cross_entropy_forward", "cross_entropy_backward_inplace",
                 "fused_sumexp", "fused_softmax_inplace"):
        for ty in ("fp16", "bf16"):
            assert f"{stem}_{ty}_launcher" in names
    for extra in ("is_bf16_supported", "to_fp16_from_fp32", "to_bf16_from_fp32", "bmt_hip_last_error"):
        assert extra in names


def test_library_exports_every_declared_symbol():
    import bmtrain_amd.C as C
    lib = ctypes.CDLL(C.LIBRARY_PATH)
    for name in declared_symbols():
        assert hasattr(lib, name), name
    assert sorted(C.EXPORTED_SYMBOLS) == declared_symbols()
    assert C.is_bf16_supported() == 1


def test_python_face_has_the_reference_names():
    import bmtrain_amd.C as C
    # names registered by the reference in csrc/bind.cpp:4-20 (NCCL wrappers excluded)
    for name in ("to_fp16_from_fp32", "to_bf16_from_fp32", "is_bf16_supported", "has_nan_inf_fp16_launcher",
                 "has_nan_inf_bf16_launcher", "adam_fp16_launcher", "adam_bf16_launcher", "adam_cpu_fp16_launcher",
                 "adam_cpu_bf16_launcher", "cross_entropy_forward_fp16_launcher", "cross_entropy_forward_bf16_launcher",
                 "cross_entropy_backward_inplace_fp16_launcher", "cross_entropy_backward_inplace_bf16_launcher",
                 "fused_sumexp_fp16_launcher", "fused_sumexp_bf16_launcher", "fused_softmax_inplace_fp16_launcher",
                 "fused_softmax_inplace_bf16_launcher"):
        assert callable(getattr(C, name)), name


def test_argument_count_is_checked_and_degenerate_sizes_are_noops():
    import bmtrain_amd.C as C
    with pytest.raises(TypeError):
        C.adam_bf16_launcher(1, 0, 0)
    # n <= 0 returns before anything touches a device (adam_cuda.cu:91,118; has_inf_nan.cu:108,128)
    C.adam_bf16_launcher(0, 0, 0, 0, 0, 0, 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.0, 0.1, 0.001, 0)
    C.adam_fp16_launcher(-5, 0, 0, 0, 0, 0, 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.0, 0.1, 0.001, 0)
    C.has_nan_inf_fp16_launcher(0, 0, 0, 0, 0)
    C.has_nan_inf_bf16_launcher(0, 0, 0, 0, 0)
    C.cross_entropy_forward_fp16_launcher(0, 10, 0, 0, 0, 0, -100, 0)
    C.cross_entropy_backward_inplace_bf16_launcher(4, 0, 0, 0, 0, -100, 0)
    with pytest.raises(RuntimeError, match="null pointer"):
        C.adam_cpu_fp16_launcher(4, 0, 0, 0, 0, 0, 0, 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.0, 0.1, 0.001)
    # refused on the host before any device call: a softmax output inside the logits (cross_entropy.cu:30-36 reads
    # input[target] after the softmax row has been stored, so the forward is not an in-place operation there either)
    for softmax in (0x10000, 0x10000 + 2 * 4 * 16 - 2, 0x10000 - 2 * 4 * 16 + 2):
        with pytest.raises(RuntimeError, match="softmax overlaps input"):
            C.cross_entropy_forward_bf16_launcher(4, 16, 0x10000, 0x40000, softmax, 0x50000, -100, 0)


def test_header_is_plain_c_and_the_documented_bindings_compile(tmp_path):
    """include/bmt_hip.h is the boundary: it must compile as C99 on its own and link against the library, and the
    pybind11 forwarding module that the integration guide shows a maintainer of the reference (the replacement for
    csrc/bind.cpp:3-35, the guide's one C++ listing) must compile against the header exactly as printed there."""
    import subprocess
    import sysconfig
    import pybind11
    import bmtrain_amd.C as C
    include = os.path.join(ROOT, "include")
    c_file = tmp_path / "uses_header.c"
    c_file.write_text('#include "bmt_hip.h"\nint main(void) { return is_bf16_supported() == 1 ? 0 : 1; }\n')
    lib_dir = os.path.dirname(C.LIBRARY_PATH)
    exe = tmp_path / "uses_header"
    subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Werror", "-I", include, str(c_file), "-o", str(exe), "-L", lib_dir,
                    "-lbmt_hip", "-Wl,-rpath," + lib_dir], check=True, capture_output=True)
    assert subprocess.run([str(exe)]).returncode == 0
    doc = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    stub = re.search(r"```cpp\n(.*?)```", doc, flags=re.S).group(1)
    assert "PYBIND11_MODULE(C, m)" in stub
    cpp_file = tmp_path / "bind.cpp"
    cpp_file.write_text(stub)
    subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-Werror", "-I", include, "-I", pybind11.get_include(),
                    "-I", sysconfig.get_paths()["include"], str(cpp_file)], check=True, capture_output=True)
