"""End-to-end differentiable flex attention: forward + delta + dq + dk/dv behind one
``torch.autograd.Function``.

The reference wires its three kernels together with ``jax.custom_vjp`` (upstream copy in
jax_exp.py:207-321: ``_flash_attention`` / ``_flash_attention_fwd`` saves ``(q, k, v, ab,
segment_ids, o, l, m)``; ``_flash_attention_bwd`` computes ``di = sum(o * do, -1)`` in float32 and
calls the dk/dv and the dq kernels).  This is the same wiring on the HIP entry points of this
package, with the flex arguments (``score_fn``, ``mask_fn`` / ``block_mask_fn``) of
flex_attention_kernel.py:66-83 carried through.
"""
from __future__ import annotations

import math
from typing import Callable, Optional, Tuple

import torch

from .flex_attention_dkv_kernel import flash_attention_bwd_dkv
from .flex_attention_dq_bwd import compute_delta, ds_exchange_pays, flex_attention_bwd_dq
from .flex_attention_kernel import _flex_attention_impl


# The backward hands dS from the dk/dv pass to the dq pass (DsBlocks in flex_attention_dq_bwd.py) when both
# gradients are wanted and the hand-over is expected to pay (ds_exchange_pays).  The buffer holds one 32 KB block
# per query head and kept pair of 128 x 128 tiles (what the mask skips takes no room); the dk/dv entry point
# declines it, and the dq pass recomputes, when it would take more than half of the free device memory.


def flex_attention_bwd(q, k, v, ab, segment_ids, l, m, o, do, *, block_q, block_k, sm_scale, causal=False, score_fn=None,
                       mask_fn=None, block_mask_fn=None, compiled_loop=False):
    """(dq, dk, dv) of one backward: delta = sum(o * do), the dq pass and the dk/dv pass (the sequence of the
    reference's custom_vjp wiring, jax_exp.py:276-321) from one call through the C ABI (flexattn_bwd): small
    problems are bound by the host's path to a launch.  No dS hand-over (see flash_attention_bwd_dkv(return_ds=True) for that) and no bias
    gradient (flex_attention_bwd_dq(return_dab=True))."""
    import ctypes as C
    from . import _lib
    from ._common import on_device, stream_of
    kw = dict(sm_scale=sm_scale, debug=False, score_fn=score_fn, mask_fn=mask_fn, block_mask_fn=block_mask_fn,
              compiled_loop=compiled_loop)
    dq_call = flex_attention_bwd_dq(q, k, v, ab, segment_ids, l, m, o, do, None, block_b=1, block_q=block_q,
                                    block_k_major=block_k, block_k=block_k, causal=causal, return_delta=True, _defer=True, **kw)
    dkv_call = None
    if dq_call is not None and dq_call["delta"] is not None:
        dkv_call = flash_attention_bwd_dkv(k, v, q, ab, segment_ids, l, m, dq_call["delta"], do, block_b=1, block_q=block_q,
                                           block_q_major=block_q, block_k_major=block_k, block_k=block_k, causal=causal,
                                           _defer=True, **kw)
    if dkv_call is None:   # (padded shapes, ids per batch entry: the passes one after the other)
        dq, di = flex_attention_bwd_dq(q, k, v, ab, segment_ids, l, m, o, do, None, block_b=1, block_q=block_q,
                                       block_k_major=block_k, block_k=block_k, causal=causal, return_delta=True, **kw)
        dk, dv = flash_attention_bwd_dkv(k, v, q, ab, segment_ids, l, m, di, do, block_b=1, block_q=block_q,
                                         block_q_major=block_q, block_k_major=block_k, block_k=block_k, causal=causal, **kw)
        return dq, dk, dv
    lib = dq_call["lib"]
    with on_device(q.device):
        _lib.check(lib.flexattn_bwd(C.byref(dq_call["params"]), C.byref(dkv_call["params"]), stream_of(q)), lib)
    dq, _ = dq_call["finish"]()
    dk, dv = dkv_call["finish"]()
    return dq, dk, dv


class _FlexAttention(torch.autograd.Function):
    """o = softmax(mask(score_mod(sm_scale q k^T))) v with the saved statistics (l, m) for the backward."""

    @staticmethod
    def forward(ctx, q, k, v, ab, opts):
        score_fn, mask_fn, block_mask_fn, segment_ids, causal, sm_scale, block_q, block_k = opts
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        o, l, m = _flex_attention_impl(q, k, v, ab, segment_ids, True, causal, sm_scale, 1, block_q, block_k, block_k,
                                       False, block_mask_fn, mask_fn, score_fn)
        ctx.save_for_backward(q, k, v, o, l, m, *([ab] if ab is not None else []))
        ctx.opts = opts
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, l, m, *rest = ctx.saved_tensors
        ab = rest[0] if rest else None
        score_fn, mask_fn, block_mask_fn, segment_ids, causal, sm_scale, block_q, block_k = ctx.opts
        want_dab = ab is not None and ctx.needs_input_grad[3]
        do = do.contiguous()
        dq = dk = dv = ds = dab = None
        want_dkv = ctx.needs_input_grad[1] or ctx.needs_input_grad[2]
        want_dq = ctx.needs_input_grad[0] or want_dab
        exchange = (want_dkv and ctx.needs_input_grad[0] and ab is None and q.dtype == torch.bfloat16 and
                    ds_exchange_pays(score_fn, mask_fn, segment_ids))
        # di = sum(o * do), float32 [B, H, Sq] (jax_exp.py:276-278): taken by the dq pass itself where that pass runs
        # first (no dS hand-over), else by its own launch
        di = None
        if want_dkv and ctx.needs_input_grad[0] and not want_dab and not exchange:
            dq, dk, dv = flex_attention_bwd(q, k, v, ab, segment_ids, l, m, o, do, block_q=block_q, block_k=block_k,
                                            sm_scale=sm_scale, causal=causal, score_fn=score_fn, mask_fn=mask_fn,
                                            block_mask_fn=block_mask_fn)
            return dq, dk, dv, None, None
        if want_dq and not exchange:
            dq = flex_attention_bwd_dq(q, k, v, ab, segment_ids, l, m, o, do, None, block_b=1, block_q=block_q,
                                       block_k_major=block_k, block_k=block_k, sm_scale=sm_scale, debug=False,
                                       score_fn=score_fn, mask_fn=mask_fn, block_mask_fn=block_mask_fn, causal=causal,
                                       return_dab=want_dab, return_delta=not want_dab)
            if want_dab:
                dq, dab = dq
            else:
                dq, di = dq
        if di is None and want_dkv:
            di = compute_delta(o, do)
        if want_dkv:
            dk, dv, ds = flash_attention_bwd_dkv(k, v, q, ab, segment_ids, l, m, di, do, block_b=1, block_q=block_q,
                                                 block_q_major=block_q, block_k_major=block_k, block_k=block_k,
                                                 sm_scale=sm_scale, causal=causal, debug=False, score_fn=score_fn,
                                                 mask_fn=mask_fn, block_mask_fn=block_mask_fn, return_ds=True) \
                if exchange else (*flash_attention_bwd_dkv(
                    k, v, q, ab, segment_ids, l, m, di, do, block_b=1, block_q=block_q, block_q_major=block_q,
                    block_k_major=block_k, block_k=block_k, sm_scale=sm_scale, causal=causal, debug=False,
                    score_fn=score_fn, mask_fn=mask_fn, block_mask_fn=block_mask_fn), None)
        if want_dq and exchange:
            dq = flex_attention_bwd_dq(q, k, v, ab, segment_ids, l, m, o, do, di, block_b=1, block_q=block_q,
                                       block_k_major=block_k, block_k=block_k, sm_scale=sm_scale, debug=False,
                                       score_fn=score_fn, mask_fn=mask_fn, block_mask_fn=block_mask_fn, causal=causal,
                                       ds=ds)
        return dq if ctx.needs_input_grad[0] else None, dk, dv, dab, None


def flex_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, score_fn: Optional[Callable] = None,
                   mask_fns: Optional[Tuple[Callable, Callable]] = None, *, segment_ids=None, causal: bool = False,
                   sm_scale: Optional[float] = None, block_q: int = 128, block_k: int = 128,
                   ab: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Differentiable flex attention on ``[B, H, S, D]`` GPU tensors (k, v may have fewer heads: GQA).

    ``score_fn``   closure from ``scores`` (or ``util.make_jax_score_fn`` / ``compiler.compile_score_mod``), a plain
                   Python function ``f(q_tile, k_tile)`` or ``f(s, b, h, q_idx, kv_idx)`` (compiled at first use), or None
    ``mask_fns``   ``(mask_fn, block_mask_fn)`` pair from ``masks`` (or ``compiler.compile_mask_fn``), a pair whose
                   ``mask_fn(q_idx, k_idx)`` is a plain Python function (compiled at first use, the block closure
                   derived from it), such a function alone, or None
    ``segment_ids`` / ``causal``   as in the three entry points (ANDed with ``mask_fns``)
    ``sm_scale``   default 1 / sqrt(D)
    ``ab``         additive bias on the logits, [B or 1, H or 1, Sq, Sk]; a bias that requires grad receives
                   dab = P (dP - delta), summed over the dimensions it broadcasts (the output the reference declares
                   next to dk, dv, flash_attention_dkv_bwd.py:103-107,130-138)
    Gradients flow to q, k, v and ab (``torch.autograd.grad`` / ``.backward()``); higher-order
    differentiation is not supported, as in the reference (jax_exp.py:243-244).
    """
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(q.shape[-1])
    if callable(mask_fns):   # (a bare mask function instead of a pair)
        mask_fn, block_mask_fn = mask_fns, None
    else:
        mask_fn, block_mask_fn = mask_fns if mask_fns is not None else (None, None)
    from ._common import tagged_closures
    score_fn, mask_fn, block_mask_fn = tagged_closures(score_fn, mask_fn, block_mask_fn, block_q, block_k)
    opts = (score_fn, mask_fn, block_mask_fn, segment_ids, bool(causal), float(sm_scale), int(block_q), int(block_k))
    return _FlexAttention.apply(q, k, v, ab, opts)
