"""dk/dv backward entry point, same name and argument list as the reference's
``flash_attention_bwd_dkv`` (flex_attention_dkv_kernel.py:23-174), plus the ``mask_fn`` /
``block_mask_fn`` keywords of its mask-aware twin (flash_attention_dkv_bwd.py:27-48)."""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from ._common import (on_device, bias_c, check_blocks, check_doc_batches, check_qkv, check_rows, kernel_block_map, kernel_head_dim, library_for, pad_seq,
                      padded_len, resolve_mask, stream_of, tagged_closures)
from .flex_attention_dq_bwd import DsBlocks, alloc_ds, bwd_params


def flash_attention_bwd_dkv(k, v, q, ab, segment_ids, l, m, di, do, *, block_b=None, block_q, block_q_major,
                            block_k_major, block_k, sm_scale, causal, debug, score_fn=None, mask_fn=None,
                            block_mask_fn=None, compiled_loop=False, return_ds=False, _defer=False):
    """(dk, dv): dv = P^T do, dk = dS^T * d(score)/dk with P recomputed from (l, m) and
    dS = P (dP - di) (flex_attention_dkv_kernel.py:237-272).  With grouped KV heads the gradients
    of all query heads of a group are summed inside the kernel.  ``causal`` is honoured
    (the reference's north-star file ignores it; its mask-aware twin gets the same effect from
    ``mask_fn``).  ``return_ds=True`` returns (dk, dv, ds): ds is the pass's dS as a DsBlocks for
    ``flex_attention_bwd_dq(..., ds=ds)``, or None when the kernels of the call exchange nothing (fp32, head
    dimension 256, the global position bias with one query head per kv head) or the device has too little free memory for the buffer (one 32 KB
    block per query head and kept pair of 128 x 128 tiles): the dq pass then recomputes as usual."""
    B, Hq, Hkv, Sq, Sk, D = check_qkv(q, k, v, do)
    score_fn, mask_fn, block_mask_fn = tagged_closures(score_fn, mask_fn, block_mask_fn, block_q, block_k_major)
    for name, t in (("l", l), ("m", m), ("di", di)):
        check_rows(name, t, B, Hq, Sq, q.device)
    check_blocks(Sq, Sk, block_q=block_q, block_k_major=block_k_major, block_k=block_k,
                 block_q_major=block_q_major)
    # ragged lengths: zero-padded to the kernels' tiles (padded rows carry l = 0 and dO = 0: they add nothing)
    Sq_p, Sk_p = padded_len(Sq), padded_len(Sk)
    spec = resolve_mask(mask_fn, block_mask_fn, causal, segment_ids, Sq, Sk, Sq_p, Sk_p)
    check_doc_batches(spec, B)   # (ids of shape [B, S]: the kernels mask every batch entry by its own row)
    q, do, k, v = pad_seq(q, Sq_p), pad_seq(do, Sq_p), pad_seq(k, Sk_p), pad_seq(v, Sk_p)
    l, m, di = pad_seq(l, Sq_p), pad_seq(m, Sq_p), pad_seq(di, Sq_p)
    D_user, D = D, kernel_head_dim(D, q.dtype)   # smaller head dimensions: zero-padded columns
    q, do, k, v = pad_seq(q, D, 3), pad_seq(do, D, 3), pad_seq(k, D, 3), pad_seq(v, D, 3)
    bm = kernel_block_map(_lib.PASS_DKV, spec, q, Sq_p, Sk_p, D, score_fn)
    dk = torch.empty_like(k)
    dv = torch.empty_like(v)
    ab_c, ab_keep = bias_c(ab, B, Hq, Sq, Sk, Sq_p, Sk_p, q.device)
    p = bwd_params(q, k, v, l, m, do, di, sm_scale, score_fn, spec, bm, block_q or 1, block_k or 1, dk=dk, dv=dv,
                   compiled_loop=compiled_loop, ab_c=ab_c)
    ds = None
    lib = library_for(score_fn, spec)
    if _defer:   # (flex_attention_bwd launches this pass together with the dq pass: whole tiles only, no hand-over)
        if Sk_p != Sk or Sq_p != Sq or D != D_user or return_ds:
            return None
        return {"params": p, "lib": lib, "finish": lambda: (dk, dv), "keep": (q, k, v, do, l, m, di, ab_keep, bm)}
    with on_device(q.device):
        if return_ds:
            p.ds_index.pairs = 1   # (asks whether the kernels of the call exchange at all, before the index is built)
            if lib.flexattn_bwd_ds_bytes(C.byref(p)) > 0:
                p.ds_index = bm.ds_index_c()
                need = lib.flexattn_bwd_ds_bytes(C.byref(p))
                buf = alloc_ds(need, q.device)
                if buf is not None:
                    ds = DsBlocks(buf, (B, Hq, Sq_p, Sk_p), index=bm.ds_index(), compiled_loop=bool(compiled_loop))
                    p.ds, p.ds_bytes = buf.data_ptr(), need
            if ds is None:
                p.ds_index = _lib.DsIndexC()
        _lib.check(lib.flexattn_bwd_dkv(C.byref(p), stream_of(q)), lib)
    if Sk_p != Sk or D != D_user:
        dk, dv = dk[:, :, :Sk, :D_user].contiguous(), dv[:, :, :Sk, :D_user].contiguous()
    return (dk, dv, ds) if return_ds else (dk, dv)
