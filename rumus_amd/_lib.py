"""ctypes binding of ``librumus_hip.so`` (the C ABI declared in include/rumus_hip.h).

There is no fallback: if the library is missing or a call fails, an exception is
raised.  ``build()`` compiles it in-tree with hipcc for gfx950.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "librumus_hip.so")
CSRC = os.path.join(_HERE, "csrc")

OK, EINVAL, EHIP = 0, 1, 2


class RumusError(RuntimeError):
    """A non-zero status from the C ABI (the reference panics in these cases)."""

    def __init__(self, code: int, message: str):
        super().__init__(f"rumus_hip status {code}: {message}")
        self.code = code


def build(jobs: int = 8) -> str:
    """Compile every HIP source into ``librumus_hip.so`` (always recompiles)."""
    subprocess.check_call(["make", "-C", CSRC, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", CSRC, f"-j{jobs}"], stdout=subprocess.DEVNULL)
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("hipcc did not produce librumus_hip.so")
    return LIB_PATH


_u32, _u64, _i32, _vp = C.c_uint32, C.c_uint64, C.c_int, C.c_void_p

# name -> (restype, argtypes); mirrors include/rumus_hip.h one to one
PROTOTYPES = {
    "rumus_hip_init": (_i32, [_i32]),
    "rumus_hip_last_error": (C.c_char_p, []),
    "rumus_hip_version": (C.c_char_p, []),
    "rumus_hip_sync": (_i32, [_vp]),
    "rumus_hip_workspace_reserve": (_i32, [_vp, _u64]),
    "rumus_hip_shutdown": (_i32, []),
    "rumus_hip_q8_buf_size": (_u64, [_u64, _u32]),
    "rumus_hip_q8_quantize": (_i32, [_vp, _vp, _u32, _u32, _vp]),
    "rumus_hip_q8_dequantize": (_i32, [_vp, _vp, _u32, _u32, _vp]),
    "rumus_hip_q8_dequantize_kn": (_i32, [_vp, _vp, _u32, _u32, _u32, _vp]),
    "rumus_hip_matmul_q8": (_i32, [_vp, _vp, _vp, _u32, _u32, _u32, _u32, _vp]),
    "rumus_hip_q8_dense_layout": (_i32, [_vp, _u32, _u32, _u32, _vp, _vp, _vp]),
    "rumus_hip_matmul_q8_dense": (_i32, [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _vp]),
    "rumus_hip_add_bias": (_i32, [_vp, _vp, _vp, _u32, _u32, _vp]),
    "rumus_hip_transpose_f32": (_i32, [_vp, _vp, _u32, _u32, _vp]),
    "rumus_hip_i8_quantize_rows": (_i32, [_vp, _vp, _vp, _u32, _u32, _vp]),
    "rumus_hip_i8_quantize_cols_t": (_i32, [_vp, _vp, _vp, _u32, _u32, _vp]),
    "rumus_hip_i8_gemm": (_i32, [_vp] * 7 + [_u32] * 3 + [_vp]),
    "rumus_hip_w4_quantize_pack": (_i32, [_vp, _u32, _u32, _u32, _vp, _vp, _vp, _vp]),
    "rumus_hip_w4_quantize_pack_sym": (_i32, [_vp, _u32, _u32, _u32, _vp, _vp, _vp, _vp]),
    "rumus_hip_w4_quantize_pack_awq": (_i32, [_vp, _u32, _u32, _u32, _vp, _vp, _vp, _vp]),
    "rumus_hip_f16_to_f32": (_i32, [_vp, _vp, _u64, _vp]),
    "rumus_hip_matmul_q8_f16": (_i32, [_vp, _vp, _vp, _u32, _u32, _u32, _u32, _vp]),
    "rumus_hip_qmatmul_int4_f16": (_i32, [_vp] * 7 + [_u32] * 6 + [_vp]),
    "rumus_hip_f16_staging_reserve": (_i32, [_vp, _u64]),
    "rumus_hip_w4_qzeros_unpack": (_i32, [_vp, _u32, _u32, _vp, _vp]),
    "rumus_hip_w4_decode_layout": (_i32, [_vp, _vp, _vp, _u32, _u32, _u32, _vp, _vp, _vp, _vp]),
    "rumus_hip_qmatmul_int4_decode": (_i32, [_vp] * 7 + [_u32] * 6 + [_vp]),
    "rumus_hip_qmatmul_int4_decode_max_rows": (_u32, [_u32, _u32]),
    "rumus_hip_w4_decode_layout_zp4": (_i32, [_vp, _vp, _vp, _u32, _u32, _u32, _vp, _vp, _vp, _vp]),
    "rumus_hip_qmatmul_int4_decode_zp4": (_i32, [_vp] * 7 + [_u32] * 6 + [_vp]),
    "rumus_hip_qmatmul_int4_decode_swiglu": (_i32, [_vp] * 6 + [_u32] * 6 + [_vp]),
    "rumus_hip_qmatmul_int4_decode_block": (_i32, [_vp, _vp, C.c_float, _i32] + [_vp] * 6 + [_u32] * 6 + [_vp]),
    "rumus_hip_qmatmul_int4_zp4": (_i32, [_vp] * 7 + [_u32] * 6 + [_vp]),
    "rumus_hip_qmatmul_int4": (_i32, [_vp] * 7 + [_u32] * 6 + [_vp]),
    "rumus_hip_qmatmul_int4_t": (_i32, [_vp] * 5 + [_u32] * 6 + [_vp]),
    "rumus_hip_w4_actorder_prepare": (_i32, [_vp, _vp, _u32, _u32, _u32, _vp, _vp, _vp]),
    "rumus_hip_qmatmul_int4_perm": (_i32, [_vp] * 7 + [_u32] * 6 + [_vp]),
    "rumus_hip_qmatmul_int4_perm_static": (_i32, [_vp] * 7 + [_u32] * 6 + [_vp]),
    "rumus_hip_static_scratch_bytes": (_u64, []),
    "rumus_hip_rmsnorm": (_i32, [_vp, _vp, _vp, _u32, _u32, C.c_float, _vp]),
    "rumus_hip_add_rmsnorm": (_i32, [_vp, _vp, _vp, _vp, _vp, _u32, _u32, C.c_float, _vp]),
    "rumus_hip_swiglu": (_i32, [_vp, _vp, _vp, _u64, _vp]),
    "rumus_hip_swiglu_rows": (_i32, [_vp, _vp, _u32, _u32, _vp]),
    "rumus_hip_add": (_i32, [_vp, _vp, _vp, _u64, _vp]),
    "rumus_hip_i8_gemm_workspace_size": (_u64, [_u32, _u32, _u32]),
    "rumus_hip_kv_append": (_i32, [_vp] * 4 + [_u32] * 6 + [C.POINTER(C.c_uint64), _vp]),
    "rumus_hip_attention_decode_append": (_i32, [_vp] * 6 + [_u32] * 5 + [C.POINTER(C.c_uint64), _vp]),
    "rumus_hip_attention": (_i32, [_vp] * 4 + [_u32] * 5 + [C.POINTER(C.c_uint64), _i32, _vp]),
}

_lib = None


def lib() -> C.CDLL:
    """Load the shared library (once) and attach the prototypes."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C rumus_amd/csrc`; there is no fallback path")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


def check(status: int) -> None:
    if status != OK:
        raise RumusError(status, lib().rumus_hip_last_error().decode())


def call(name: str, *args) -> None:
    """Call an int-returning entry point and raise on a non-zero status."""
    check(getattr(lib(), name)(*args))
