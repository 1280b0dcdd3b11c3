"""ctypes binding of libflexattn.so (the C ABI declared in include/flexattn.h).

The library is the only compute path: if it is missing or a call fails, this
module raises -- there is no CPU or eager fallback.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("FLEXATTN_LIB") or os.path.join(_HERE, "libflexattn.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

FLEX_F32, FLEX_F16, FLEX_BF16 = 0, 1, 2
SCORE_IDENTITY, SCORE_CHECKERBOARD, SCORE_ALIBI, SCORE_TANH_SOFTCAP, SCORE_REL_BIAS, SCORE_AFFINE = range(6)
MASK_BAND, MASK_BITS = 0, 1
FLAG_ROUND_S, FLAG_STRICT, FLAG_FORCE_GENERIC, FLAG_BWD_ONLY_DQ, FLAG_BWD_ONLY_DKV, FLAG_PARITY = 1, 2, 4, 8, 16, 32
FLAG_UNROUNDED = 64
INT_MIN, INT_MAX = -(2 ** 31), 2 ** 31 - 1


class FlexScoreMod(C.Structure):
    _fields_ = [("kind", C.c_int32), ("p0", C.c_float), ("p1", C.c_float),
                ("i0", C.c_int32), ("i1", C.c_int32),
                ("mul", C.c_void_p), ("add", C.c_void_p),
                ("stride_b", C.c_int64), ("stride_h", C.c_int64), ("stride_q", C.c_int64)]


class FlexMask(C.Structure):
    _fields_ = [("kind", C.c_int32), ("lo", C.c_int32), ("hi", C.c_int32), ("sink", C.c_int32),
                ("q_offset", C.c_int32), ("pad_", C.c_int32), ("bits", C.c_void_p),
                ("bits_stride_b", C.c_int64), ("bits_stride_h", C.c_int64), ("bits_stride_q", C.c_int64),
                ("bits_t", C.c_void_p),
                ("bits_t_stride_b", C.c_int64), ("bits_t_stride_h", C.c_int64), ("bits_t_stride_kv", C.c_int64),
                ("blk", C.c_void_p),
                ("blk_stride_b", C.c_int64), ("blk_stride_h", C.c_int64), ("blk_stride_q", C.c_int64)]


class FlexTileLists(C.Structure):
    _fields_ = [("kv_num", C.c_void_p), ("kv_idx", C.c_void_p),
                ("full_kv_num", C.c_void_p), ("full_kv_idx", C.c_void_p),
                ("q_num", C.c_void_p), ("q_idx", C.c_void_p),
                ("full_q_num", C.c_void_p), ("full_q_idx", C.c_void_p),
                ("q_block", C.c_int32), ("kv_block", C.c_int32),
                ("n_q_blocks", C.c_int32), ("n_kv_blocks", C.c_int32),
                ("stride_b", C.c_int64), ("stride_h", C.c_int64)]


class FlexAttnParams(C.Structure):
    _fields_ = [("dtype", C.c_int32),
                ("B", C.c_int32), ("Hq", C.c_int32), ("Hkv", C.c_int32), ("Lq", C.c_int32),
                ("Lkv", C.c_int32), ("D", C.c_int32), ("Dv", C.c_int32),
                ("q_stride", C.c_int64 * 3), ("k_stride", C.c_int64 * 3),
                ("v_stride", C.c_int64 * 3), ("o_stride", C.c_int64 * 3),
                ("scale", C.c_float), ("flags", C.c_int32),
                ("score", FlexScoreMod), ("mask", FlexMask), ("tiles", FlexTileLists),
                ("tiles_bwd", FlexTileLists), ("q_index_base", C.c_int32), ("pad_", C.c_int32),
                ("d_lse2", C.c_void_p)]


EXPORTS = [
    "flexattn_abi_version", "flexattn_last_error", "flexattn_preferred_tiles", "flexattn_kernel_family",
    "flexattn_block_mask_workspace_bytes", "flexattn_block_mask_build",
    "flexattn_fwd_workspace_bytes", "flexattn_fwd",
    "flexattn_bwd_workspace_bytes", "flexattn_bwd",
    "flexattn_decode_workspace_bytes", "flexattn_decode", "flexattn_decode_static",
]

_lib: Optional[C.CDLL] = None


class FlexAttnError(RuntimeError):
    pass


def build(verbose: bool = False) -> str:
    """Compile libflexattn.so for gfx950 with hipcc (cross-compiles without a GPU)."""
    jobs = str(min(16, os.cpu_count() or 8))
    subprocess.run(["make", "-C", CSRC_DIR, "clean"], check=True, capture_output=not verbose)
    r = subprocess.run(["make", "-C", CSRC_DIR, "-j", jobs], capture_output=True, text=True)
    if r.returncode != 0:
        raise FlexAttnError("building libflexattn.so failed:\n" + r.stdout[-4000:] + r.stderr[-8000:])
    return LIB_PATH


def lib() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FlexAttnError(
            f"{LIB_PATH} is missing: build it with `make -C {CSRC_DIR}` "
            "(or __graft_entry__.build()); there is no fallback path")
    L = C.CDLL(LIB_PATH)
    L.flexattn_abi_version.restype = C.c_int
    L.flexattn_last_error.restype = C.c_char_p
    L.flexattn_preferred_tiles.argtypes = [C.c_int32] * 6 + [C.POINTER(C.c_int32)] * 2
    L.flexattn_kernel_family.argtypes = [C.POINTER(FlexAttnParams), C.c_int32]
    L.flexattn_block_mask_workspace_bytes.restype = C.c_size_t
    L.flexattn_block_mask_workspace_bytes.argtypes = [C.c_int32] * 4
    L.flexattn_block_mask_build.argtypes = ([C.POINTER(FlexMask)] + [C.c_int32] * 6 +
                                            [C.c_void_p] * 8 + [C.c_void_p, C.c_void_p])
    L.flexattn_fwd_workspace_bytes.restype = C.c_size_t
    L.flexattn_fwd_workspace_bytes.argtypes = [C.POINTER(FlexAttnParams)]
    L.flexattn_fwd.argtypes = [C.POINTER(FlexAttnParams)] + [C.c_void_p] * 7
    L.flexattn_bwd_workspace_bytes.restype = C.c_size_t
    L.flexattn_bwd_workspace_bytes.argtypes = [C.POINTER(FlexAttnParams)]
    L.flexattn_bwd.argtypes = [C.POINTER(FlexAttnParams)] + [C.c_void_p] * 11
    L.flexattn_decode_workspace_bytes.restype = C.c_size_t
    L.flexattn_decode_workspace_bytes.argtypes = [C.POINTER(FlexAttnParams), C.c_int32]
    L.flexattn_decode.argtypes = [C.POINTER(FlexAttnParams)] + [C.c_void_p] * 5 + [C.c_int32, C.c_void_p, C.c_void_p]
    L.flexattn_decode_static.argtypes = [C.POINTER(FlexAttnParams)] + [C.c_void_p] * 5 + [C.c_int32, C.c_void_p]
    _lib = L
    return L


def check(rc: int, who: str) -> None:
    if rc != 0:
        msg = lib().flexattn_last_error().decode("utf-8", "replace")
        raise FlexAttnError(f"{who} failed (code {rc}): {msg}")
