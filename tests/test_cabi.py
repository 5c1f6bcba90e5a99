"""The C-ABI shared library loads, exports every symbol include/flexattn.h declares, and rejects
bad arguments with error codes (no GPU work is launched by these tests)."""
import ctypes as C
import os
import re

import pytest
import torch

from flex_attention_tpu_amd import _lib

HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "flexattn.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(flexattn_[a-z_0-9]+)\s*\(", text)))


def test_every_declared_symbol_is_exported(lib):
    names = _declared_symbols()
    assert len(names) >= 8
    for n in names:
        assert hasattr(lib, n), f"{n} declared in flexattn.h but not exported"
    assert sorted(_lib.EXPORTS) == names


def test_version_matches_header(lib):
    ver = int(re.search(r"#define FLEXATTN_VERSION (\d+)", open(HEADER).read()).group(1))
    assert lib.flexattn_version() == ver


def test_struct_sizes_follow_c_layout():
    # pointers 8-byte aligned, no surprises in the ctypes mirrors
    assert C.sizeof(_lib.ScoreSpecC) == 32
    assert C.sizeof(_lib.MaskSpecC) == 48
    assert C.sizeof(_lib.BlockMapC) == 56
    assert C.sizeof(_lib.BiasC) == 32
    assert C.sizeof(_lib.FwdParamsC) == 6 * 8 + 10 * 4 + 32 + 48 + 56 + 32
    assert C.sizeof(_lib.DsIndexC) == 24
    assert C.sizeof(_lib.BwdParamsC) == 10 * 8 + 10 * 4 + 32 + 48 + 56 + 32 + 16 + 24 + 8 + 16


def test_tile_shapes(lib):
    assert _lib.tile_shape(_lib.PASS_FWD, _lib.BF16, 128)[0] % 64 == 0
    for p in (_lib.PASS_FWD, _lib.PASS_DQ, _lib.PASS_DKV):
        bq, bk = _lib.tile_shape(p, _lib.F32, 64)
        assert bq > 0 and bk > 0
    with pytest.raises(NotImplementedError):
        _lib.tile_shape(_lib.PASS_FWD, _lib.BF16, 96)
    # bf16 head dimension 256 runs on the tiles of 128; beyond that, and float32 beyond 128, there is no kernel
    for p in (_lib.PASS_FWD, _lib.PASS_DQ, _lib.PASS_DKV):
        assert _lib.tile_shape(p, _lib.BF16, 256) == _lib.tile_shape(p, _lib.BF16, 128)
    for dtype, D in ((_lib.BF16, 384), (_lib.F32, 256)):
        with pytest.raises(NotImplementedError):
            _lib.tile_shape(_lib.PASS_FWD, dtype, D)
    from flex_attention_tpu_amd._common import kernel_head_dim
    assert [kernel_head_dim(D, torch.bfloat16) for D in (1, 64, 128, 129, 192, 256)] == [128, 128, 128, 256, 256, 256]
    assert [kernel_head_dim(D, torch.float32) for D in (1, 64, 65, 128)] == [64, 64, 128, 128]
    for dtype, D in ((torch.bfloat16, 257), (torch.float32, 129)):
        with pytest.raises(NotImplementedError):
            kernel_head_dim(D, dtype)
    with pytest.raises(ValueError):
        _lib.tile_shape(7, _lib.BF16, 128)


def test_error_codes_and_messages(lib):
    assert lib.flexattn_fwd(None, None) == _lib.EINVAL
    assert b"NULL" in lib.flexattn_last_error_string()
    assert lib.flexattn_bwd_dq(None, None) == _lib.EINVAL
    assert lib.flexattn_bwd_dkv(None, None) == _lib.EINVAL
    assert lib.flexattn_bwd_delta(None, None, None, 1, 128, 0, None) == _lib.EINVAL
    m = _lib.MaskSpecC(_lib.MASK_WINDOW, 0, 0, 0, None, None)
    dummy = C.create_string_buffer(64)
    rc = lib.flexattn_build_block_mask(C.byref(m), 256, 256, 128, 128, dummy, None, None, None, None, None)
    assert rc == _lib.EINVAL and b"window" in lib.flexattn_last_error_string()
    m = _lib.MaskSpecC(_lib.MASK_CAUSAL, 0, 0, 0, None, None)
    rc = lib.flexattn_build_block_mask(C.byref(m), 250, 256, 128, 128, dummy, None, None, None, None, None)
    assert rc == _lib.EINVAL and b"divisible" in lib.flexattn_last_error_string()
    # shape errors are caught before any launch
    p = _lib.FwdParamsC()
    p.q = p.k = p.v = p.o = C.addressof(dummy)
    p.B, p.Hq, p.Hkv, p.Sq, p.Sk, p.D, p.dtype = 1, 3, 2, 128, 128, 128, _lib.BF16
    assert lib.flexattn_fwd(C.byref(p), None) == _lib.EINVAL
    assert b"multiple" in lib.flexattn_last_error_string()
    p.Hq = 2
    p.Sq = 100
    assert lib.flexattn_fwd(C.byref(p), None) == _lib.EINVAL
    p.Sq, p.D = 128, 96
    assert lib.flexattn_fwd(C.byref(p), None) == _lib.ENOTSUP
    with pytest.raises(NotImplementedError):
        _lib.check(_lib.ENOTSUP)
    with pytest.raises(ValueError):
        _lib.check(_lib.EINVAL)


def test_ds_exchange_sizes_and_argument_checks(lib):
    """flexattn_bwd_ds_bytes looks at shapes, dtype, score, flags and the number of kept tile pairs only (one 32 KB
    block per query head and pair); a dS buffer on a request whose kernels exchange nothing, one without its
    index, or one that is too small, is refused before any launch."""
    dummy = C.create_string_buffer(64)
    p = _lib.BwdParamsC()
    p.B, p.Hq, p.Hkv, p.Sq, p.Sk, p.D, p.dtype, p.sm_scale = 2, 4, 2, 256, 384, 128, _lib.BF16, 0.125
    assert lib.flexattn_bwd_ds_bytes(C.byref(p)) == 0          # no kept pairs named
    p.ds_index.pairs = 5
    assert lib.flexattn_bwd_ds_bytes(C.byref(p)) == 2 * 4 * 5 * 128 * 128 * 2
    p.ds_index.pairs = 2 * 3 + 1                                # more pairs than the 2 x 3 tiles of the shape
    assert lib.flexattn_bwd_ds_bytes(C.byref(p)) == 0
    p.ds_index.pairs = 6
    assert lib.flexattn_bwd_ds_bytes(C.byref(p)) == 2 * 4 * 256 * 384 * 2   # every pair kept: the dense size
    p.score.kind = _lib.SCORE_SOFTCAP
    assert lib.flexattn_bwd_ds_bytes(C.byref(p)) == 2 * 4 * 256 * 384 * 2
    # the dk/dv kernel with a compiled main loop exports too: the tile-local position bias, the global one where kv
    # heads are grouped, any score on request; the global bias's dk/dv stream (one q head per kv head) does not
    for kind in (_lib.SCORE_ALIBI, _lib.SCORE_ALIBI_TILE):
        p.score.kind = kind
        assert lib.flexattn_bwd_ds_bytes(C.byref(p)) == 2 * 4 * 256 * 384 * 2
    p.score.kind, p.Hkv = _lib.SCORE_ALIBI, 4
    assert lib.flexattn_bwd_ds_bytes(C.byref(p)) == 0
    p.score.kind, p.Hkv = _lib.SCORE_NONE, 2
    p.flags = _lib.FLAG_COMPILED_LOOP
    assert lib.flexattn_bwd_ds_bytes(C.byref(p)) == 2 * 4 * 256 * 384 * 2
    p.flags, p.D = 0, 256
    assert lib.flexattn_bwd_ds_bytes(C.byref(p)) == 0          # (head dimension 256: no exchange)
    p.D, p.dtype = 128, _lib.F32
    assert lib.flexattn_bwd_ds_bytes(C.byref(p)) == 0
    p.dtype, p.Sq = _lib.BF16, 200          # not a multiple of the dk/dv tile
    assert lib.flexattn_bwd_ds_bytes(C.byref(p)) == 0
    p.Sq = 1025 * 128                       # more than 1024 tiles along a sequence
    assert lib.flexattn_bwd_ds_bytes(C.byref(p)) == 0
    assert lib.flexattn_bwd_ds_bytes(None) == 0
    # a buffer where none is exchanged, one without its index, and one that is too small
    p.Sq, p.dtype = 256, _lib.F32
    for f in ("q", "k", "v", "dout", "l", "m", "delta", "dq", "dk", "dv", "ds"):
        setattr(p, f, C.addressof(dummy))
    p.ds_bytes = 1 << 40
    for call in (lib.flexattn_bwd_dq, lib.flexattn_bwd_dkv):
        assert call(C.byref(p), None) == _lib.EINVAL and b"exchange no dS" in lib.flexattn_last_error_string()
    p.dtype = _lib.BF16
    for call in (lib.flexattn_bwd_dq, lib.flexattn_bwd_dkv):
        assert call(C.byref(p), None) == _lib.EINVAL and b"ds_index" in lib.flexattn_last_error_string()
    p.ds_index.col = p.ds_index.rank = C.addressof(dummy)
    p.ds_bytes = 2 * 4 * 256 * 384 * 2 - 1
    for call in (lib.flexattn_bwd_dq, lib.flexattn_bwd_dkv):
        assert call(C.byref(p), None) == _lib.EINVAL and b"needs" in lib.flexattn_last_error_string()
    # the whole backward from one call: both blocks are checked, and they must describe the same problem
    assert lib.flexattn_bwd(None, None, None) == _lib.EINVAL
    # the index builder checks its arguments
    assert lib.flexattn_build_ds_index(None, None, None, None) == _lib.EINVAL
    m = _lib.BlockMapC()
    assert lib.flexattn_build_ds_index(C.byref(m), C.addressof(dummy), C.addressof(dummy), None) == _lib.EINVAL
