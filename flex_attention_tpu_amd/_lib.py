"""ctypes binding of libflexattn.so (the C ABI declared in include/flexattn.h).

The library is the only compute path of this package: importing this module fails loudly when the
shared object has not been built (``python -m flex_attention_tpu_amd.build``); there is no
fallback implementation.
"""
from __future__ import annotations

import ctypes as C
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libflexattn.so")

OK = 0
EINVAL = -22
ENOTSUP = -95
ELAUNCH = -5

BF16 = 0
F32 = 1

SCORE_NONE = 0
SCORE_ALIBI = 1
SCORE_SOFTCAP = 2
SCORE_ALIBI_TILE = 3
SCORE_CUSTOM = 4

MASK_CAUSAL = 1
MASK_WINDOW = 2
MASK_DOC = 4
MASK_S2 = 8
MASK_CUSTOM = 16

FLAG_COMPILED_LOOP = 1

PASS_FWD = 0
PASS_DQ = 1
PASS_DKV = 2


class ScoreSpecC(C.Structure):
    _fields_ = [
        ("kind", C.c_int32),
        ("cap", C.c_float),
        ("slope", C.c_float),
        ("mod_q", C.c_int32),
        ("mod_k", C.c_int32),
        ("reserved", C.c_int32),
        ("slopes", C.c_void_p),
    ]


class MaskSpecC(C.Structure):
    _fields_ = [
        ("flags", C.c_int32),
        ("window", C.c_int32),
        ("stride", C.c_int32),
        ("doc_batches", C.c_int32),
        ("doc_q", C.c_void_p),
        ("doc_k", C.c_void_p),
        ("doc_q_range", C.c_void_p),
        ("doc_k_range", C.c_void_p),
    ]


class BlockMapC(C.Structure):
    _fields_ = [
        ("state", C.c_void_p),
        ("kv_cnt", C.c_void_p),
        ("kv_idx", C.c_void_p),
        ("q_cnt", C.c_void_p),
        ("q_idx", C.c_void_p),
        ("nq", C.c_int32),
        ("nk", C.c_int32),
        ("block_q", C.c_int32),
        ("block_k", C.c_int32),
    ]


class BiasC(C.Structure):
    _fields_ = [
        ("ptr", C.c_void_p),
        ("stride_b", C.c_int64),
        ("stride_h", C.c_int64),
        ("dtype", C.c_int32),
        ("reserved", C.c_int32),
    ]


class DsIndexC(C.Structure):
    _fields_ = [
        ("col", C.c_void_p),
        ("rank", C.c_void_p),
        ("pairs", C.c_int64),
    ]


class FwdParamsC(C.Structure):
    _fields_ = [
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p),
        ("o", C.c_void_p),
        ("l", C.c_void_p), ("m", C.c_void_p),
        ("B", C.c_int32), ("Hq", C.c_int32), ("Hkv", C.c_int32),
        ("Sq", C.c_int32), ("Sk", C.c_int32), ("D", C.c_int32),
        ("dtype", C.c_int32),
        ("sm_scale", C.c_float),
        ("flags", C.c_int32),
        ("reserved", C.c_int32),
        ("score", ScoreSpecC),
        ("mask", MaskSpecC),
        ("map", BlockMapC),
        ("ab", BiasC),
    ]


class BwdParamsC(C.Structure):
    _fields_ = [
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("dout", C.c_void_p),
        ("l", C.c_void_p), ("m", C.c_void_p), ("delta", C.c_void_p),
        ("dq", C.c_void_p),
        ("dk", C.c_void_p), ("dv", C.c_void_p),
        ("B", C.c_int32), ("Hq", C.c_int32), ("Hkv", C.c_int32),
        ("Sq", C.c_int32), ("Sk", C.c_int32), ("D", C.c_int32),
        ("dtype", C.c_int32),
        ("sm_scale", C.c_float),
        ("flags", C.c_int32),
        ("reserved", C.c_int32),
        ("score", ScoreSpecC),
        ("mask", MaskSpecC),
        ("map", BlockMapC),
        ("ab", BiasC),
        ("ds", C.c_void_p),
        ("ds_bytes", C.c_int64),
        ("ds_index", DsIndexC),
        ("dab", C.c_void_p),
        ("o", C.c_void_p),
        ("delta_out", C.c_void_p),
    ]


EXPORTS = (
    "flexattn_version",
    "flexattn_last_error_string",
    "flexattn_tile_shape",
    "flexattn_build_block_mask",
    "flexattn_build_ds_index",
    "flexattn_fwd",
    "flexattn_fwd_noalloc",
    "flexattn_bwd_delta",
    "flexattn_bwd_ds_bytes",
    "flexattn_bwd_dq",
    "flexattn_bwd_dkv",
    "flexattn_bwd",
    "flexattn_custom_tag",
)

_lib = None
_custom_libs = {}


def _bind(lib: C.CDLL) -> C.CDLL:
    lib.flexattn_version.restype = C.c_int
    lib.flexattn_last_error_string.restype = C.c_char_p
    lib.flexattn_custom_tag.restype = C.c_char_p
    lib.flexattn_tile_shape.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
    lib.flexattn_build_block_mask.argtypes = [
        C.POINTER(MaskSpecC), C.c_int32, C.c_int32, C.c_int32, C.c_int32,
        C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    lib.flexattn_build_ds_index.argtypes = [C.POINTER(BlockMapC), C.c_void_p, C.c_void_p, C.c_void_p]
    lib.flexattn_fwd.argtypes = [C.POINTER(FwdParamsC), C.c_void_p]
    lib.flexattn_fwd_noalloc.argtypes = [C.POINTER(FwdParamsC), C.c_void_p]
    lib.flexattn_bwd_delta.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_int32, C.c_void_p]
    lib.flexattn_bwd_dq.argtypes = [C.POINTER(BwdParamsC), C.c_void_p]
    lib.flexattn_bwd_ds_bytes.argtypes = [C.POINTER(BwdParamsC)]
    lib.flexattn_bwd_ds_bytes.restype = C.c_int64
    lib.flexattn_bwd_dkv.argtypes = [C.POINTER(BwdParamsC), C.c_void_p]
    lib.flexattn_bwd.argtypes = [C.POINTER(BwdParamsC), C.POINTER(BwdParamsC), C.c_void_p]
    for name in ("flexattn_tile_shape", "flexattn_build_block_mask", "flexattn_build_ds_index", "flexattn_fwd", "flexattn_fwd_noalloc", "flexattn_bwd_delta",
                 "flexattn_bwd_dq", "flexattn_bwd_dkv", "flexattn_bwd"):
        getattr(lib, name).restype = C.c_int
    return lib


def load() -> C.CDLL:
    """Loads libflexattn.so once; raises ImportError if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m flex_attention_tpu_amd.build` "
            "(hipcc, gfx950). This package has no other compute path.")
    _lib = _bind(C.CDLL(LIB_PATH))
    return _lib


def load_for(score_code=None, mask_code=None) -> C.CDLL:
    """The library whose kernels contain the given compiled closures (compiler.CustomCode objects, or None):
    libflexattn.so when there is none, else the functor library of the pair, compiled with hipcc at first
    use and cached on disk (compiler.build_functor_library)."""
    if score_code is None and mask_code is None:
        return load()
    from . import compiler
    key = compiler.functor_key(score_code, mask_code)
    lib = _custom_libs.get(key)
    if lib is None:
        path = compiler.build_functor_library(score_code, mask_code)
        lib = _bind(C.CDLL(path))
        tag = lib.flexattn_custom_tag().decode()
        if tag != key:
            raise ImportError(f"{path} was built for functor {tag!r}, expected {key!r}: delete it and call again")
        _custom_libs[key] = lib
    return lib


def check(rc: int, lib=None) -> None:
    """Maps a status code to the exception class the reference raises in the same situation."""
    if rc == OK:
        return
    msg = (lib or load()).flexattn_last_error_string().decode("utf-8", "replace")
    if rc == EINVAL:
        raise ValueError(msg)
    if rc == ENOTSUP:
        raise NotImplementedError(msg)
    raise RuntimeError(f"flexattn error {rc}: {msg}")


_tile_shapes = {}


def tile_shape(pass_id: int, dtype: int, D: int):
    """(block_q, block_k) of the kernels of a pass (a property of the library: asked once per combination)."""
    key = (pass_id, dtype, D)
    hit = _tile_shapes.get(key)
    if hit is None:
        bq, bk = C.c_int32(0), C.c_int32(0)
        check(load().flexattn_tile_shape(pass_id, dtype, D, C.byref(bq), C.byref(bk)))
        hit = _tile_shapes[key] = (bq.value, bk.value)
    return hit
