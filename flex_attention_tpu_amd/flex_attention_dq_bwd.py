"""dq backward entry point, same name and argument list as the reference's
``flex_attention_bwd_dq`` (flex_attention_dq_bwd.py:114-267), on torch tensors."""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from ._common import (on_device, bias_c, check_blocks, check_doc_batches, check_qkv, check_rows, dtype_code, kernel_block_map, kernel_head_dim, library_for,
                      pad_seq, padded_len, mostly_partial_custom_mask, resolve_mask, score_spec_c, stream_of, tagged_closures)
from .block_mask import mask_spec_c


def compute_delta(o: torch.Tensor, do: torch.Tensor) -> torch.Tensor:
    """d = sum(o * do, axis=-1) in float32, [B, H, Sq] -- the reduction the reference leaves to the
    caller (flex_attention_dq_bwd.py:932, flash_attention_dkv_bwd.py:925), as one HIP launch."""
    if o.shape != do.shape or o.dtype != do.dtype or o.ndim != 4:
        raise ValueError("o and do must be rank-4 tensors of the same shape and dtype")
    if not (o.is_cuda and o.is_contiguous() and do.is_contiguous()):
        raise ValueError("o and do must be contiguous GPU tensors")
    B, H, S, D = o.shape
    if D not in (64, 128) and not (D == 256 and o.dtype == torch.bfloat16):   # (zero columns add nothing to the sum)
        D = kernel_head_dim(D, o.dtype)
        o, do = pad_seq(o, D, 3), pad_seq(do, D, 3)
    d = torch.empty(B, H, S, dtype=torch.float32, device=o.device)
    with on_device(o.device):
        _lib.check(_lib.load().flexattn_bwd_delta(o.data_ptr(), do.data_ptr(), d.data_ptr(), B * H * S, D,
                                                  dtype_code(o), stream_of(o)))
    return d


class DsBlocks:
    """dS of one dk/dv pass, as ``flash_attention_bwd_dkv(..., return_ds=True)`` leaves it for
    ``flex_attention_bwd_dq(..., ds=...)``: bf16 values in the kernels' own block layout, opaque to callers.
    The reference's two backward kernels each recompute S, dP and dS (flex_attention_dq_bwd.py:340-378,
    flash_attention_dkv_bwd.py:232-302); handing dS over leaves the dq pass one contraction instead of three."""

    def __init__(self, buf=None, shape=None, index=None, compiled_loop=False):
        # (compiled_loop: the flag of the dk/dv call; the dq call must carry the same one, the kernel family decides
        # whether the exported values already hold sm_scale)
        self.buf, self.shape, self.index, self.compiled_loop = buf, shape, index, compiled_loop


# The dS buffer is never allowed to take more than this share of the device's memory, and an out-of-memory error of
# the allocator is caught: the backward must not fail for want of memory where the recomputing dq pass would have worked.
DS_MEMORY_SHARE = 0.25
_total_memory = {}


def alloc_ds(nbytes: int, device):
    """The dS exchange buffer, or None when it does not fit comfortably: more than DS_MEMORY_SHARE of the device's
    memory, or an out-of-memory error from the allocator.  The caller then runs the two recomputing passes.  (The
    driver's figure of free memory is not asked per call: the query takes 0.2 ms and holds the launch path up.)"""
    dev = torch.device(device)
    total = _total_memory.get(dev)
    if total is None:
        total = _total_memory[dev] = torch.cuda.get_device_properties(dev).total_memory
    if nbytes > DS_MEMORY_SHARE * total:
        return None
    try:
        return torch.empty(nbytes, dtype=torch.uint8, device=dev)
    except torch.cuda.OutOfMemoryError:
        return None


def ds_exchange_pays(score_fn, mask_fn=None, segment_ids=None) -> bool:
    """Whether handing dS from the dk/dv pass to the dq pass is expected to shorten the backward: yes with the
    softcap score (eight element-wise operations per score in the recomputing dq kernel) and with masks that
    leave many partial tiles (documents, windows: the dq pass from dS does no mask work at all); no with plain
    scores under no mask or a plain causal one, where the export slows the dk/dv pass (writing S^2-sized dS costs
    it clock under the power limit) by as much as the dq pass gains.  Measured on MI355X, dq + dk/dv in ms,
    recomputing -> exchanging: softcap + documents, 16k tokens, GQA 4:1: 1.93 -> 1.47; documents, plain scores, same
    shape: 1.75 -> 1.34; five documents in B=4, H=32, S=4096: 1.09 -> 0.91; causal window 1025, B=2, H=16, S=8192:
    0.56 -> 0.49; softcap, causal, B=4, H=32, S=4096: 2.08 -> 1.86; plain causal, same shape: 1.67 -> 1.68; plain
    causal GQA 4:1, B=2, Hq=32, S=8192: 3.09 -> 3.17."""
    kind = getattr(getattr(score_fn, "spec", None), "kind", _lib.SCORE_NONE if score_fn is None else None)
    if kind in (_lib.SCORE_CUSTOM, _lib.SCORE_ALIBI_TILE):
        # kernels with a compiled main loop in both passes: the dq pass from dS is half the recomputing one's time
        # and evaluates no score function (a compiled closure then costs one backward pass its arithmetic, not two:
        # B=4, H=32, S=4096, dq + dk/dv in ms, a soft-cap closure 3.12 -> 2.62, the test suite's mixed_mod 5.05 -> 3.50)
        return True
    if kind not in (_lib.SCORE_NONE, _lib.SCORE_SOFTCAP):
        return False   # (the global position bias: its dk/dv stream exports nothing, its dq stream is fast)
    if kind == _lib.SCORE_SOFTCAP:
        return True
    if segment_ids is not None:
        return True
    flags = getattr(getattr(mask_fn, "spec", None), "flags", 0)
    return bool(flags & (_lib.MASK_WINDOW | _lib.MASK_DOC | _lib.MASK_S2))


def bwd_params(q, k, v, l, m, do, d, sm_scale, score_fn, spec, bm, mod_q, mod_k, dq=None, dk=None, dv=None,
               compiled_loop=False, ab_c=None):
    B, Hq, Sq, D = q.shape
    _, Hkv, Sk, _ = k.shape
    return _lib.BwdParamsC(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), do.data_ptr(), l.data_ptr(), m.data_ptr(), d.data_ptr(),
        dq.data_ptr() if dq is not None else None,
        dk.data_ptr() if dk is not None else None, dv.data_ptr() if dv is not None else None,
        B, Hq, Hkv, Sq, Sk, D, dtype_code(q), float(sm_scale), _lib.FLAG_COMPILED_LOOP if compiled_loop else 0, 0,
        score_spec_c(score_fn, Hq, q.device, mod_q, mod_k, sm_scale), mask_spec_c(spec, Sq, Sk, q.device), bm.as_c(),
        ab_c if ab_c is not None else _lib.BiasC())


def flex_attention_bwd_dq(q, k, v, ab, segment_ids, l, m, o, do, d, *, block_b, block_q, block_k_major,
                          block_k, sm_scale, debug, score_fn=None, mask_fn=None, block_mask_fn=None,
                          causal=False, compiled_loop=False, ds=None, return_dab=False, return_delta=False, _defer=False):
    """dq = sum_j dS_ij * d(score)/dq, with P_ij = exp(S_ij - m_i) / l_i recomputed from the saved
    statistics, dP = do v^T, dS = P (dP - d) (flex_attention_dq_bwd.py:340-378).  ``o`` is only
    shape-checked, as in the reference (:163); ``d`` is the caller's delta (see compute_delta).
    ``ds``: the DsBlocks of the dk/dv pass of the same arguments, if that pass returned one: dq is then
    sm_scale dS K, nothing is recomputed.
    ``d=None``: the call takes delta = sum(o * do) itself (the reference hands ``o`` to this function without using
    it, :163): the delta kernel runs in front of the dq kernel, one call through the C ABI instead of two;
    ``return_delta=True`` then returns (dq, d) so that the dk/dv pass can be given the same d.
    ``return_dab=True`` (needs ``ab``; excludes ``ds``) returns (dq, dab): the gradient of the additive bias in
    ab's shape and dtype, dab = P (dP - d) summed over the dimensions ``ab`` broadcasts -- the output the
    reference declares next to dk, dv (flash_attention_dkv_bwd.py:103-107,130-138) and its upstream dq kernel
    writes (jax_exp.py:1252-1255; there multiplied by sm_scale)."""
    B, Hq, Hkv, Sq, Sk, D = check_qkv(q, k, v, do)
    score_fn, mask_fn, block_mask_fn = tagged_closures(score_fn, mask_fn, block_mask_fn, block_q, block_k_major)
    if o is not None and tuple(o.shape) != tuple(q.shape):
        raise ValueError(f"o has shape {tuple(o.shape)}, expected {tuple(q.shape)}")
    fuse_delta = d is None
    if fuse_delta:
        if o is None or ds is not None:
            raise ValueError("d=None needs `o` (delta is then taken of o and do) and excludes `ds`")
        if o.dtype != q.dtype or not o.is_contiguous() or o.device != q.device:
            raise ValueError("o must be a contiguous tensor of q's dtype on q's device")
        d = torch.empty(B, Hq, Sq, dtype=torch.float32, device=q.device)
    for name, t in (("l", l), ("m", m), ("d", d)):
        check_rows(name, t, B, Hq, Sq, q.device)
    check_blocks(Sq, Sk, block_q=block_q, block_k_major=block_k_major, block_k=block_k)
    # ragged lengths: zero-padded to the kernels' tiles (padded rows carry l = 0: their probabilities vanish)
    Sq_p, Sk_p = padded_len(Sq), padded_len(Sk)
    spec = resolve_mask(mask_fn, block_mask_fn, causal, segment_ids, Sq, Sk, Sq_p, Sk_p)
    check_doc_batches(spec, B)   # (ids of shape [B, S]: the kernels mask every batch entry by its own row)
    q, do, k, v = pad_seq(q, Sq_p), pad_seq(do, Sq_p), pad_seq(k, Sk_p), pad_seq(v, Sk_p)
    l, m, d_p = pad_seq(l, Sq_p), pad_seq(m, Sq_p), pad_seq(d, Sq_p)
    D_user, D = D, kernel_head_dim(D, q.dtype)   # smaller head dimensions: zero-padded columns
    q, do, k, v = pad_seq(q, D, 3), pad_seq(do, D, 3), pad_seq(k, D, 3), pad_seq(v, D, 3)
    o_p = pad_seq(pad_seq(o, Sq_p), D, 3) if fuse_delta else None
    if ds is not None and (ds.buf is None or ds.index is None or ds.shape != (B, Hq, Sq_p, Sk_p) or ds.buf.device != q.device
                           or ds.compiled_loop != bool(compiled_loop)):
        raise ValueError("ds does not come from a dk/dv pass of these arguments")
    # (the dS blocks lie at the dk/dv kernel's tiles: the dq pass walks that map's row lists)
    bm = kernel_block_map(_lib.PASS_DKV if ds is not None else _lib.PASS_DQ, spec, q, Sq_p, Sk_p, D, score_fn)
    if ds is None and mostly_partial_custom_mask(spec, bm):
        compiled_loop = True
    dq = torch.empty_like(q)
    ab_c, ab_keep = bias_c(ab, B, Hq, Sq, Sk, Sq_p, Sk_p, q.device)
    p = bwd_params(q, k, v, l, m, do, d_p, sm_scale, score_fn, spec, bm, block_q or 1, block_k or 1, dq=dq,
                   compiled_loop=compiled_loop, ab_c=ab_c)
    if fuse_delta:
        p.delta, p.o, p.delta_out = None, o_p.data_ptr(), d_p.data_ptr()
    dab_full = None
    if return_dab:
        if ab is None or ds is not None:
            raise ValueError("return_dab needs the additive bias `ab` and excludes `ds`")
        # (only the tiles the block map visits are written: masked-out pairs have no gradient)
        dab_full = torch.zeros(B, Hq, Sq_p, Sk_p, dtype=torch.float32, device=q.device)
        p.dab = dab_full.data_ptr()
    if ds is not None:
        p.ds, p.ds_bytes = ds.buf.data_ptr(), ds.buf.numel()
        col, rank, pairs = ds.index   # (the index the dk/dv pass wrote the blocks by)
        p.ds_index = _lib.DsIndexC(col.data_ptr(), rank.data_ptr(), pairs)
    if return_delta and return_dab:
        raise ValueError("return_delta and return_dab exclude each other")
    lib = library_for(score_fn, spec)
    keep = (q, k, v, do, l, m, d_p, o_p, ab_keep, bm, dab_full)   # what the parameter block points at

    def finish():
        """The call's results from the kernels' output buffers (cuts padding off, reduces the bias gradient)."""
        out, d_out = dq, d
        if Sq_p != Sq or D != D_user:
            out = out[:, :, :Sq, :D_user].contiguous()
        if fuse_delta and d_p is not d:
            d_out = d_p[:, :, :Sq].contiguous()
        if not return_dab:
            return (out, d_out) if return_delta else out
        dab = dab_full[:, :, :Sq, :Sk]
        if ab.shape[0] == 1 and B > 1:
            dab = dab.sum(0, keepdim=True)
        if ab.shape[1] == 1 and Hq > 1:
            dab = dab.sum(1, keepdim=True)
        return out, dab.to(ab.dtype).contiguous()

    if _defer:   # (flex_attention_bwd launches this pass together with the dk/dv pass)
        return {"params": p, "lib": lib, "finish": finish, "keep": keep, "delta": d if d_p is d else None}
    with on_device(q.device):
        _lib.check(lib.flexattn_bwd_dq(C.byref(p), stream_of(q)), lib)
    return finish()
