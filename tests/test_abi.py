"""CPU-side checks of the drop-in boundary: the C-ABI library loads without a GPU and exports
every symbol include/tensorlib_amd.h declares; the Python binding covers each of them; the
product package never reaches into the oracle.  No compute call is made here."""
import ctypes
import os
import re
import subprocess

import pytest

from tensorlib_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_is_built_in_tree():
    assert os.path.exists(_lib.LIB_PATH), "run __graft_entry__.build() first"
    assert _lib.LIB_PATH.startswith(ROOT)


def test_every_declared_symbol_is_exported():
    handle = ctypes.CDLL(_lib.LIB_PATH)
    declared = _lib.declared_symbols()
    assert len(declared) >= 30
    missing = [s for s in declared if not hasattr(handle, s)]
    assert not missing, missing


def test_binding_covers_the_header_exactly():
    assert sorted(_lib._PROTOS) == _lib.declared_symbols()


def test_llama2_driver_exports_its_header():
    import re as _re
    from tensorlib_amd import llama2
    text = open(os.path.join(ROOT, "include", "tensorlib_llama2.h")).read()
    text = _re.sub(r"/\*.*?\*/", "", text, flags=_re.S)
    declared = sorted(set(_re.findall(r"\b(tlm_[a-z0-9_]+)\s*\(", text)))
    assert sorted(llama2._PROTOS) == declared
    ctypes.CDLL(_lib.LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    handle = ctypes.CDLL(llama2.LLAMA2_LIB_PATH)
    assert not [s for s in declared if not hasattr(handle, s)]


def test_tokenizer_exports_its_header():
    from tensorlib_amd import llama2, tokenizer
    text = open(os.path.join(ROOT, "include", "tensorlib_tokenizer.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = sorted(set(re.findall(r"\b(tlt_[a-z0-9_]+)\s*\(", text)))
    assert sorted(tokenizer._PROTOS) == declared
    ctypes.CDLL(_lib.LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    handle = ctypes.CDLL(llama2.LLAMA2_LIB_PATH)
    assert not [s for s in declared if not hasattr(handle, s)]


def test_header_cites_the_reference_for_each_hot_path_entry():
    text = open(_lib.HEADER).read()
    for sym in ["tl_matmul2d_f16", "tl_gemv_f16", "tl_hgemm_f16", "tl_rms_norm_f16", "tl_apply_rotary_emb_f16",
                "tl_softmax_f16", "tl_contiguous_f16", "tl_set_item_ewise_f16", "tl_argmax_f16"]:
        i = text.index(f"int {sym}(")
        comment = text[text.rfind("/*", 0, i):i]
        assert re.search(r"\.(hpp|cpp|cu|cuh):\d+", comment), f"{sym} lacks a reference citation"


def test_status_and_version_calls_work_without_a_gpu():
    handle = ctypes.CDLL(_lib.LIB_PATH)
    handle.tl_version.restype = ctypes.c_char_p
    handle.tl_last_error.restype = ctypes.c_char_p
    assert b"gfx950" in handle.tl_version()
    assert handle.tl_device_cu_count() == 0
    assert handle.tl_set_gemv_variant(10 ** 6) != 0      # host-side validation only
    assert b"out of range" in handle.tl_last_error()
    handle.tl_gemv_variant_name.restype = ctypes.c_char_p
    assert handle.tl_gemv_variant_name(0) == b"auto"
    assert handle.tl_gemv_variant_name(-1) is None


def test_product_never_imports_the_oracle():
    """Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may touch oracle/."""
    pkg = os.path.join(ROOT, "tensorlib_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".hpp", ".cpp", "Makefile")):
                src = open(os.path.join(dirpath, f), errors="ignore").read()
                assert "oracle" not in src.lower(), os.path.join(dirpath, f)


REFERENCE_INCLUDE = "/root/reference/tensorLib/include"


@pytest.mark.skipif(not os.path.exists(os.path.join(REFERENCE_INCLUDE, "device", "Device.hpp")),
                    reason="the reference tree is not present (it never is on the GPU box)")
def test_adaptor_overrides_every_pure_virtual_of_the_reference_interface(tmp_path):
    """include/tl_hip_device.hpp compiled against the reference's own Device.hpp
    (tensorLib/include/device/Device.hpp:13-101): deriving from Device<dtype> with every method marked
    `override`, and instantiating HIP<half>, HIP<int> and HIP<float>, only compiles when each pure virtual is
    overridden with a matching signature.  Syntax check only: nothing is linked or run."""
    src = tmp_path / "adaptor_check.cpp"
    src.write_text(
        '#include "tl_hip_device.hpp"\n'
        "template class HIP<tl::half>;\n"
        "template class HIP<int>;\n"
        "template class HIP<float>;\n"
        "Device<tl::half>* make_h(size_t n) { return new HIP<tl::half>(n); }\n"
        "Device<int>* make_i(size_t n) { return new HIP<int>(n); }\n"
        "Device<float>* make_f(size_t n) { return new HIP<float>(n); }\n")
    cxx = "/opt/rocm/lib/llvm/bin/clang++"      # needs _Float16 on the host, which g++ 11 lacks
    proc = subprocess.run([cxx, "-std=c++17", "-fsyntax-only", "-Wall", "-Werror=overloaded-virtual",
                           "-DTL_HAVE_TENSORLIB_DEVICE_HPP", "-I", os.path.join(ROOT, "include"), "-I", REFERENCE_INCLUDE,
                           str(src)], capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-3000:]
