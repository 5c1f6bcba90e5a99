"""Flex-attention forward entry point, same name and argument list as the reference's
``_flex_attention_impl`` (flex_attention_kernel.py:66-193), on torch tensors.

The reference builds a Pallas grid and traces ``score_fn`` / ``mask_fn`` / ``block_mask_fn`` into
the kernel; here the closures' ``.spec`` selects a compiled HIP functor, the block map is built on
the GPU once per mask, and one ``flexattn_fwd`` launch does the rest on the current stream.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from ._common import (on_device, bias_c, check_blocks, check_doc_batches, check_qkv, dtype_code, kernel_block_map, kernel_head_dim, library_for, pad_seq,
                      padded_len, mostly_partial_custom_mask, resolve_mask, score_spec_c, stream_of, tagged_closures)
from .block_mask import mask_spec_c


def _flex_attention_impl(q, k, v, ab, segment_ids, save_residuals, causal, sm_scale, block_b, block_q,
                         block_k_major, block_k, debug, block_mask_fn, mask_fn, score_fn, *, compiled_loop=False):
    """Returns ``o`` (q.dtype) or ``(o, l, m)`` with float32 ``l, m`` of shape [B, H, Sq].

    Semantics (flex_attention_kernel.py:248-319): S = score_mod(sm_scale * q k^T) + ab; masked
    positions are excluded; m = rowmax S, l = sum exp(S - m), o = exp(S - m) v / l.
    Unlike the reference's flex forward, ``causal=True`` is honoured (ANDed with ``mask_fn``), as
    flash_attention_fwd_ref.py:78-86 and the dense reference do.  ``compiled_loop=True`` (not in the
    reference) selects the bf16 kernel with a compiled main loop instead of the generated instruction
    stream, for comparisons.
    """
    B, Hq, Hkv, Sq, Sk, D = check_qkv(q, k, v)
    check_blocks(Sq, Sk, block_q=block_q, block_k_major=block_k_major, block_k=block_k)
    score_fn, mask_fn, block_mask_fn = tagged_closures(score_fn, mask_fn, block_mask_fn, block_q, block_k_major)
    # ragged lengths: the tensors are zero-padded to the kernels' tiles, a key bound drops the padded keys
    # and the padded query rows are cut off again
    Sq_p, Sk_p = padded_len(Sq), padded_len(Sk)
    spec = resolve_mask(mask_fn, block_mask_fn, causal, segment_ids, Sq, Sk, Sq_p, Sk_p)
    check_doc_batches(spec, B)   # (ids of shape [B, S]: the kernels mask every batch entry by its own row)
    q, k, v = pad_seq(q, Sq_p), pad_seq(k, Sk_p), pad_seq(v, Sk_p)
    D_user, D = D, kernel_head_dim(D, q.dtype)   # smaller head dimensions: zero-padded columns
    q, k, v = pad_seq(q, D, 3), pad_seq(k, D, 3), pad_seq(v, D, 3)
    bm = kernel_block_map(_lib.PASS_FWD, spec, q, Sq_p, Sk_p, D, score_fn)
    compiled_loop = compiled_loop or mostly_partial_custom_mask(spec, bm)
    ab_c, ab_keep = bias_c(ab, B, Hq, Sq, Sk, Sq_p, Sk_p, q.device)
    o = torch.empty_like(q)
    l = m = None
    if save_residuals:
        l = torch.empty(B, Hq, Sq_p, dtype=torch.float32, device=q.device)
        m = torch.empty(B, Hq, Sq_p, dtype=torch.float32, device=q.device)
    p = _lib.FwdParamsC(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
        l.data_ptr() if l is not None else None, m.data_ptr() if m is not None else None,
        B, Hq, Hkv, Sq_p, Sk_p, D, dtype_code(q), float(sm_scale), _lib.FLAG_COMPILED_LOOP if compiled_loop else 0, 0,
        score_spec_c(score_fn, Hq, q.device, block_q or 1, block_k or 1, sm_scale),
        mask_spec_c(spec, Sq_p, Sk_p, q.device), bm.as_c(), ab_c)
    with on_device(q.device):
        lib = library_for(score_fn, spec)
        _lib.check(lib.flexattn_fwd(C.byref(p), stream_of(q)), lib)
    if Sq_p != Sq or D != D_user:
        o = o[:, :, :Sq, :D_user].contiguous()
        if save_residuals:
            l, m = l[:, :, :Sq].contiguous(), m[:, :, :Sq].contiguous()
    if debug:
        print(f"[flexattn_fwd] B={B} Hq={Hq} Hkv={Hkv} Sq={Sq} Sk={Sk} D={D} dtype={q.dtype} "
              f"mask_flags={spec.flags} tiles_run={int((bm.state != 0).sum())}/{bm.nq * bm.nk}")
    return (o, l, m) if save_residuals else o
