"""Loader of libtensorlib_amd.so with typed ctypes prototypes for every C-ABI entry point."""
from __future__ import annotations

import ctypes
import os
import re
import subprocess

_PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(_PKG)
CSRC = os.path.join(_PKG, "csrc")
LIB_PATH = os.path.join(_PKG, "lib", "libtensorlib_amd.so")
HEADER = os.path.join(ROOT, "include", "tensorlib_amd.h")


class TensorLibError(RuntimeError):
    """A tl_* entry point returned a non-zero status."""


def build_library(clean: bool = False) -> str:
    """Compile csrc/*.hip for gfx950 with hipcc (cross-compiles without a GPU)."""
    if clean:
        subprocess.run(["make", "-C", CSRC, "clean"], check=True, capture_output=True)
    proc = subprocess.run(["make", "-C", CSRC, "-j8"], capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("building libtensorlib_amd.so failed:\n" + proc.stdout[-4000:] + proc.stderr[-4000:])
    return LIB_PATH


def declared_symbols() -> list[str]:
    """Names of all functions declared in include/tensorlib_amd.h."""
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tl_[a-z0-9_]+)\s*\(", text)))


_c = ctypes
_vp, _sz, _i, _f, _u16 = _c.c_void_p, _c.c_size_t, _c.c_int, _c.c_float, _c.c_uint16
_ip = _c.POINTER(_c.c_int)

# name -> (restype, argtypes); status-returning functions have restype int
_PROTOS = {
    "tl_init": (_i, [_i]),
    "tl_last_error": (_c.c_char_p, []),
    "tl_version": (_c.c_char_p, []),
    "tl_device_cu_count": (_i, []),
    "tl_set_stream": (_i, [_vp]),
    "tl_get_stream": (_vp, []),
    "tl_malloc": (_i, [_c.POINTER(_vp), _sz]),
    "tl_free": (_i, [_vp]),
    "tl_memcpy_h2d": (_i, [_vp, _vp, _sz]),
    "tl_memcpy_d2h": (_i, [_vp, _vp, _sz]),
    "tl_memcpy_d2d": (_i, [_vp, _vp, _sz]),
    "tl_synchronize": (_i, []),
    "tl_reset_scratch": (_i, []),
    "tl_matmul2d_f16": (_i, [_vp, _vp, _vp, _sz, _sz, _sz]),
    "tl_gemv_f16": (_i, [_vp, _vp, _vp, _sz, _sz]),
    "tl_hgemm_f16": (_i, [_vp, _vp, _vp, _sz, _sz, _sz]),
    "tl_gemv_f16_stamped": (_i, [_vp, _vp, _vp, _sz, _sz, _vp, _sz, _ip]),
    "tl_hgemm_silu_mul_f16": (_i, [_vp, _vp, _vp, _vp, _sz, _sz, _sz]),
    "tl_matmul2d_batched_f16": (_i, [_vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _sz, _sz]),
    "tl_matmul2d_f32": (_i, [_vp, _vp, _vp, _sz, _sz, _sz]),
    "tl_set_gemv_variant": (_i, [_i]),
    "tl_set_hgemm_variant": (_i, [_i]),
    "tl_gemv_variant_name": (_c.c_char_p, [_i]),
    "tl_hgemm_variant_name": (_c.c_char_p, [_i]),
    "tl_set_gemv_grid_waves_per_cu": (_i, [_i]),
    "tl_set_hgemm_splits": (_i, [_i]),
    "tl_set_hgemm_splitk_merge": (_i, [_i]),
    "tl_set_hgemm_agpr_kernels": (_i, [_i]),
    "tl_set_hgemm_stamps": (_i, [_vp, _sz]),
    "tl_hgemm_last_split_in_launch": (_i, []),
    "tl_hgemm_last_plan": (_i, [_c.POINTER(_c.c_int), _c.POINTER(_c.c_int)]),
    "tl_set_hgemm_k_rotation": (_i, [_i, _i]),
    "tl_set_hgemm_tile_band": (_i, [_i]),
    "tl_set_hgemm_fewrows": (_i, [_i]),
    "tl_set_prefill_attention_variant": (_i, [_i]),
    "tl_set_decode_attention_merge": (_i, [_i]),
    "tl_set_decode_attention_chunk": (_i, [_i]),
    "tl_measure_mfma_rate_f16": (_i, [_i, _c.POINTER(_c.c_double)]),
    "tl_rms_norm_f16": (_i, [_vp, _vp, _vp, _f, _i, _i]),
    "tl_apply_rotary_emb_f16": (_i, [_vp, _vp, _i, _i, _i, _i, _i]),
    "tl_softmax_f16": (_i, [_vp, _vp, _sz, _sz]),
    "tl_silu_f16": (_i, [_vp, _vp, _sz]),
    "tl_binary_f16": (_i, [_vp, _vp, _vp, _sz, _i]),
    "tl_binary_scalar_f16": (_i, [_vp, _vp, _u16, _sz, _i]),
    "tl_contiguous_f16": (_i, [_vp, _vp, _ip, _ip, _i, _sz, _sz]),
    "tl_set_item_ewise_f16": (_i, [_vp, _vp, _ip, _ip, _i, _sz, _sz]),
    "tl_argmax_f16": (_i, [_vp, _vp, _sz, _sz]),
    "tl_embedding_f16": (_i, [_vp, _vp, _vp, _i, _i, _i]),
    "tl_full_f16": (_i, [_vp, _u16, _sz]),
    "tl_silu_mul_f16": (_i, [_vp, _vp, _vp, _sz]),
    "tl_decode_attention_f16": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "tl_causal_mask_f16": (_i, [_vp, _i, _i, _i]),
    "tl_gemv_silu_mul_f16": (_i, [_vp, _vp, _vp, _sz, _sz]),
    "tl_prefill_rope_qkv_f16": (_i, [_vp, _vp, _vp, _vp, _sz, _vp, _vp, _vp, _i, _i, _i, _i]),
    "tl_prefill_rope_qkv_vt_f16": (_i, [_vp, _vp, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _i, _i, _i, _i]),
    "tl_hgemm_prefill_rope_qkv_vt_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _sz]),
    "tl_scaled_causal_softmax_f16": (_i, [_vp, _u16, _i, _i, _i]),
    "tl_silu_mul_rows_f16": (_i, [_vp, _vp, _sz, _sz]),
    "tl_gather_vt_f16": (_i, [_vp, _vp, _i, _i, _i, _i]),
    "tl_prefill_attention_f16": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i]),
    "tl_gemv_add_rms_norm_f16": (_i, [_vp, _vp, _vp, _f, _vp, _vp, _vp, _sz, _sz]),
    "tl_hgemm_add_rms_norm_f16": (_i, [_vp, _vp, _vp, _vp, _f, _vp, _vp, _sz, _sz, _sz]),
    "tl_decode_attention_rope_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i]),
    "tl_decode_attention_rope_static_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i]),
    "tl_rope_table_f16": (_i, [_vp, _i, _i]),
    "tl_rope_qk_store_kv_f16": (_i, [_vp, _vp, _vp, _i, _i, _i]),
    "tl_add_rms_norm_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _f, _i, _i]),
}

_lib = None


def lib() -> ctypes.CDLL:
    """Load the shared library (never builds, never falls back)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise TensorLibError(
            f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C tensorlib_amd/csrc`; there is no CPU fallback")
    # torch bundles its own HIP runtime with the same soname; importing it first makes this
    # library bind to the runtime torch uses, so device pointers are shared.
    try:
        import torch  # noqa: F401
    except Exception:  # torch is plumbing only; the library also works without it
        pass
    handle = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    for name, (res, args) in _PROTOS.items():
        fn = getattr(handle, name)
        fn.restype = res
        fn.argtypes = args
    _lib = handle
    return _lib


def check(status: int, what: str = "") -> None:
    if status != 0:
        msg = lib().tl_last_error().decode(errors="replace")
        raise TensorLibError(f"{what or 'tl call'} failed ({status}): {msg}")
