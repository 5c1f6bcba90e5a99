"""Host-side helpers shared by the three entry points: argument checks and C struct assembly."""
from __future__ import annotations

import warnings
import weakref
from typing import Callable, Optional

import numpy as np
import torch

from . import _lib
from .block_mask import LRU, BlockMap, build_block_map, mask_spec_c, raw_stream, spec_of
from .masks import DocIds, MaskSpec
from .scores import ScoreSpec

_slopes_cache = LRU(16)   # (slopes, device) -> float32 device array
_segment_cache = LRU(16)  # id(tensor) -> (weak reference, tensor version, DocIds)


def dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return _lib.BF16
    if t.dtype == torch.float32:
        return _lib.F32
    raise NotImplementedError(f"dtype {t.dtype} is not supported (bfloat16 and float32 are)")


def check_qkv(q, k, v, *others):
    """Shape / layout checks in the spirit of the reference's rank asserts
    (flex_attention_dq_bwd.py:161-164); returns (B, Hq, Hkv, Sq, Sk, D)."""
    for name, t in (("q", q), ("k", k), ("v", v)) + tuple((f"arg{i}", o) for i, o in enumerate(others)):
        if not isinstance(t, torch.Tensor):
            raise TypeError(f"{name} must be a torch.Tensor")
        if t.ndim != 4:
            raise ValueError(f"{name} must have rank 4 [batch, heads, seq, head_dim], got {tuple(t.shape)}")
        if not t.is_cuda:
            raise ValueError(f"{name} must live on the GPU (got {t.device}); this package has no CPU path")
        if not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous")
        if t.dtype != q.dtype:
            raise ValueError(f"{name} has dtype {t.dtype}, expected {q.dtype}")
    B, Hq, Sq, D = q.shape
    Bk, Hkv, Sk, Dk = k.shape
    if v.shape != k.shape:
        raise ValueError(f"k {tuple(k.shape)} and v {tuple(v.shape)} differ")
    if Bk != B or Dk != D:
        raise ValueError(f"q {tuple(q.shape)} and k {tuple(k.shape)} disagree on batch or head_dim")
    if Hq % Hkv:
        raise ValueError(f"query heads {Hq} not a multiple of kv heads {Hkv}")
    for o in others:
        if tuple(o.shape) != tuple(q.shape):
            raise ValueError(f"expected shape {tuple(q.shape)}, got {tuple(o.shape)}")
    return B, Hq, Hkv, Sq, Sk, D


def check_rows(name, t, B, Hq, Sq, device):
    if not isinstance(t, torch.Tensor) or tuple(t.shape) != (B, Hq, Sq):
        raise ValueError(f"{name} must be a float32 tensor of shape {(B, Hq, Sq)}")
    if t.dtype != torch.float32 or not t.is_contiguous() or t.device != device:
        raise ValueError(f"{name} must be contiguous float32 on {device}")


def check_blocks(Sq, Sk, block_q=None, block_k_major=None, block_k=None, block_q_major=None):
    """Block sizes are tuning hints in the reference; here they are validated only
    (the device tiles are the kernels' own)."""
    def _div(name, blk, n):
        if blk is None:
            return
        if not isinstance(blk, (int, np.integer)) or blk <= 0:
            raise ValueError(f"{name}={blk!r} must be a positive int")
        if n % SEQ_ALIGN:
            return  # ragged length: the tensors are padded to the tile; the reference floors silently here (flex_attention_kernel.py:91)
        if n % blk:
            raise ValueError(f"{name}={blk} does not divide sequence length {n}")
    _div("block_q", block_q, Sq)
    _div("block_q_major", block_q_major, Sq)
    _div("block_k_major", block_k_major, Sk)
    _div("block_k", block_k, Sk)
    if block_k is not None and block_k_major is not None and block_k_major % block_k:
        raise ValueError(f"block_k={block_k} does not divide block_k_major={block_k_major}")
    if block_q is not None and block_q_major is not None and block_q_major % block_q:
        raise ValueError(f"block_q={block_q} does not divide block_q_major={block_q_major}")


def _doc_ids_of(ids) -> DocIds:
    """DocIds (host copy + hash) of one id array.  A DocIds passes through, and a tensor seen before (same
    object, unchanged) is answered from a small cache, so that a training step does not copy the ids to the
    host and hash them once per pass."""
    if isinstance(ids, DocIds):
        return ids
    key = id(ids)
    if isinstance(ids, torch.Tensor):
        hit = _segment_cache.get(key)
        if hit is not None and hit[0]() is ids and hit[1] == ids._version:
            return hit[2]
    t = torch.as_tensor(ids).detach().cpu()
    if t.ndim == 2 and bool((t == t[:1]).all()):
        t = t[0]   # (equal rows: one row serves the batch)
    if t.ndim not in (1, 2):
        raise ValueError("segment_ids must be a 1-D (or [B, S]) array of ids")
    doc = DocIds(t.numpy().astype(np.int64))
    if isinstance(ids, torch.Tensor):
        _segment_cache.put(key, (weakref.ref(ids), ids._version, doc))
    return doc


def segment_doc_ids(segment_ids):
    """(q ids, kv ids or None) of a ``segment_ids`` argument: one id array for both sides (1-D, or [B, S]: a row
    per batch entry, mha_reference.py:65-73), or an object with ``.q`` / ``.kv`` arrays (the reference's
    SegmentIds, jax_exp.py:37-51), which may differ and need not be sorted."""
    if hasattr(segment_ids, "q") and hasattr(segment_ids, "kv") and not isinstance(segment_ids, DocIds):
        dq = _doc_ids_of(segment_ids.q)
        dk = dq if segment_ids.kv is segment_ids.q else _doc_ids_of(segment_ids.kv)
        return dq, (None if dk == dq else dk)
    return _doc_ids_of(segment_ids), None


_tagged_closures = weakref.WeakKeyDictionary()   # plain Python closure -> its compiled (tagged) form


def _remembered(fn):
    try:
        return _tagged_closures.get(fn)
    except TypeError:   # (a callable that cannot be weakly referenced or hashed: compiled again at every call;
        return None     #  the functor libraries themselves are cached by their source)


def _remember(fn, compiled) -> None:
    try:
        _tagged_closures[fn] = compiled
    except TypeError:
        pass


def tagged_closures(score_fn, mask_fn, block_mask_fn, block_q, block_k):
    """(score_fn, mask_fn, block_mask_fn) with plain Python closures replaced by their compiled forms, so that a
    caller may hand the entry points the functions themselves, as the reference's callers hand theirs to its
    kernels (flex_attention_kernel.py:248-255, 278-288): a score function of two arguments is the reference's tile
    form (util.make_jax_score_fn), one of five the element-wise ``score_mod(s, b, h, q_idx, kv_idx)``
    (compiler.compile_score_mod); a ``mask_fn(q_idx, k_idx)`` goes to compiler.compile_mask_fn at the call's block
    sizes, which also derives the block closure (a block closure without a mask function cannot be compiled: it
    says which tiles run, not which elements).  Closures that carry a ``.spec`` pass through; the compiled form of
    a function object is kept while the function lives."""
    import inspect

    def arity(fn):
        try:
            ps = inspect.signature(fn).parameters.values()
        except (TypeError, ValueError):
            return -1
        return sum(1 for p in ps if p.kind in (p.POSITIONAL_ONLY, p.POSITIONAL_OR_KEYWORD) and p.default is p.empty)
    if score_fn is not None and not isinstance(getattr(score_fn, "spec", None), ScoreSpec):
        hit = _remembered(score_fn)
        if hit is None:
            n = arity(score_fn)
            if n == 2:
                from . import util
                hit = util.make_jax_score_fn(score_fn)
            elif n == 5:
                from . import compiler
                hit = compiler.compile_score_mod(score_fn)
            else:
                raise NotImplementedError("score_fn must take (q_tile, k_tile) or (s, b, h, q_idx, kv_idx), or come from "
                                          "flex_attention_tpu_amd.scores / util.make_jax_score_fn / compiler.compile_score_mod")
            _remember(score_fn, hit)
        score_fn = hit
    if mask_fn is not None and getattr(mask_fn, "spec", None) is None:
        key = (int(block_q or SEQ_ALIGN), int(block_k or SEQ_ALIGN))
        per_fn = _remembered(mask_fn)
        if per_fn is None:
            per_fn = {}
            _remember(mask_fn, per_fn)
        if key not in per_fn:
            from . import compiler
            per_fn[key] = compiler.compile_mask_fn(mask_fn, *key)
        mask_fn, block_mask_fn = per_fn[key]
    return score_fn, mask_fn, block_mask_fn


def check_doc_batches(spec: MaskSpec, B: int) -> None:
    """Document ids with a row per batch entry must have one for every entry of the call."""
    for d in (spec.doc_ids, spec.doc_ids_k):
        if d is not None and d.batches not in (1, B):
            raise ValueError(f"segment ids have {d.batches} rows for a batch of {B}")


def bias_c(ab, B: int, Hq: int, Sq: int, Sk: int, Sq_p: int, Sk_p: int, device):
    """(BiasC, tensor to keep alive) of the additive bias ``ab``: [B or 1, Hq or 1, Sq, Sk], float32 or
    bfloat16, added to the logits behind the score function (mha_reference.py:50-51).  Zero-padded along with
    q and k when the lengths are ragged (padded keys are masked anyway)."""
    if ab is None:
        return _lib.BiasC(), None
    if not isinstance(ab, torch.Tensor) or ab.ndim != 4:
        raise ValueError("ab must be a 4-D tensor [B or 1, H or 1, Sq, Sk]")
    if ab.shape[0] not in (1, B) or ab.shape[1] not in (1, Hq) or tuple(ab.shape[2:]) != (Sq, Sk):
        raise ValueError(f"ab has shape {tuple(ab.shape)}, expected [{B} or 1, {Hq} or 1, {Sq}, {Sk}]")
    if ab.dtype not in (torch.float32, torch.bfloat16):
        raise NotImplementedError(f"ab dtype {ab.dtype} is not supported (float32 or bfloat16)")
    if ab.device != device:
        raise ValueError("ab must live on the device of q")
    ab = pad_seq(pad_seq(ab, Sq_p, dim=2), Sk_p, dim=3).contiguous()
    sb = 0 if ab.shape[0] == 1 else ab.stride(0)
    sh = 0 if ab.shape[1] == 1 else ab.stride(1)
    return _lib.BiasC(ab.data_ptr(), sb, sh, _lib.F32 if ab.dtype == torch.float32 else _lib.BF16, 0), ab


def resolve_mask(mask_fn, block_mask_fn, causal, segment_ids, Sq, Sk, Sq_pad=None, Sk_pad=None) -> MaskSpec:
    """Single MaskSpec for the closures, the ``causal`` flag and ``segment_ids`` (AND of all).  ``Sq_pad`` /
    ``Sk_pad``: the lengths the tensors are padded to for the kernels (ragged lengths).  Padded keys must
    receive no probability: they get a document id of their own (the document mask is switched on for
    the call if it was not), so that the kernels need no separate length bound."""
    Sq_pad, Sk_pad = Sq_pad or Sq, Sk_pad or Sk
    spec = spec_of(mask_fn, block_mask_fn)
    if causal:
        spec = spec.combine(MaskSpec(flags=_lib.MASK_CAUSAL))
    if segment_ids is not None:
        dq, dk = segment_doc_ids(segment_ids)
        if len(dq) != Sq or len(dk if dk is not None else dq) != Sk:
            raise ValueError(f"segment_ids must have one id per position ({Sq} q, {Sk} kv); give an object with "
                             ".q / .kv arrays when the two lengths differ")
        spec = spec.combine(MaskSpec(flags=_lib.MASK_DOC, doc_ids=dq, doc_ids_k=dk))
    if Sq_pad != Sq or Sk_pad != Sk:
        if spec.flags & _lib.MASK_DOC:
            ids_q = spec.doc_ids.array
            ids_k = (spec.doc_ids_k if spec.doc_ids_k is not None else spec.doc_ids).array
            if ids_q.shape[-1] < Sq or ids_k.shape[-1] < Sk:
                raise ValueError(f"document ids cover {ids_q.shape[-1]} q / {ids_k.shape[-1]} kv positions, need {Sq} / {Sk}")
            ids_q, ids_k = ids_q[..., :Sq], ids_k[..., :Sk]
        else:
            ids_q, ids_k = np.zeros(Sq, np.int32), np.zeros(Sk, np.int32)
        pad_id = int(max(ids_q.max(initial=0), ids_k.max(initial=0))) + 1    # an id no query carries

        def tail(a, n):   # (pad widths of the sequence axis; rows per batch entry keep their axis)
            return [(0, 0)] * (a.ndim - 1) + [(0, n)]
        dq_p = DocIds(np.pad(ids_q, tail(ids_q, Sq_pad - Sq), mode="edge"))
        dk_p = DocIds(np.pad(ids_k, tail(ids_k, Sk_pad - Sk), constant_values=pad_id))
        spec = MaskSpec(spec.flags | _lib.MASK_DOC, spec.window, spec.stride, dq_p, spec.custom, None if dk_p == dq_p else dk_p)
    return spec


SEQ_ALIGN = 128   # every kernel's tiles divide it


def padded_len(n: int) -> int:
    return (n + SEQ_ALIGN - 1) // SEQ_ALIGN * SEQ_ALIGN


def kernel_head_dim(D: int, dtype) -> int:
    """Head dimension the kernels run a call of head dimension D at: bf16 128 or 256, fp32 64 or 128.  Others
    are zero-padded to the next of these (dot products and the output columns that are kept do not change); the
    reference itself refuses head dimensions that are not multiples of 128 (flex_attention_kernel.py:302-306)."""
    if D <= 0:
        raise ValueError(f"head_dim must be positive, got {D}")
    if dtype == torch.float32:
        if D > 128:
            raise NotImplementedError(f"float32 head_dim {D} is not supported (at most 128)")
        return 64 if D <= 64 else 128
    if D > 256:
        raise NotImplementedError(f"head_dim {D} is not supported (at most 256)")
    return 128 if D <= 128 else 256


def pad_seq(t: torch.Tensor, n: int, dim: int = 2) -> torch.Tensor:
    """`t` zero-padded to n positions along `dim` (a copy only when padding is needed)."""
    have = t.shape[dim]
    if have == n:
        return t
    shape = list(t.shape)
    shape[dim] = n
    out = t.new_zeros(shape)
    out.narrow(dim, 0, have).copy_(t)
    return out


def score_spec_c(score_fn: Optional[Callable], Hq: int, device, mod_q: int, mod_k: int, sm_scale=None) -> _lib.ScoreSpecC:
    """C view of the score closure's spec.  ``mod_q``/``mod_k`` are the tile edges the reference
    would call a tile-local score function with (block_q, block_k)."""
    if score_fn is None:
        return _lib.ScoreSpecC(_lib.SCORE_NONE, 0.0, 0.0, 1, 1, 0, None)
    if sm_scale is not None and float(sm_scale) != 1.0 and getattr(score_fn, "spec", None) is not None \
            and score_fn.spec.kind != _lib.SCORE_NONE:
        # the reference's three kernels and its dense reference disagree about sm_scale next to a score_fn
        # (flex_attention_kernel.py:249-255 ignores it, flex_attention_dq_bwd.py:340-345 multiplies the
        # function's result); they coincide with this build's score_mod(sm_scale * <q, k>) only at 1
        warnings.warn("score_fn with sm_scale != 1: this build computes score_mod(sm_scale * <q, k>); the reference's "
                      "forward ignores sm_scale here and its backward kernels scale the function's result",
                      UserWarning, stacklevel=3)
    spec = getattr(score_fn, "spec", None)
    if not isinstance(spec, ScoreSpec):
        raise NotImplementedError(
            "score_fn must come from flex_attention_tpu_amd.scores factories, util.make_jax_score_fn or "
            "compiler.compile_score_mod / compile_score_fn (which compile a Python function into the kernels)")
    slopes_ptr = None
    if spec.kind == _lib.SCORE_ALIBI:
        slopes = spec.slopes
        if slopes is None and spec.slopes_open is not None:
            if Hq > len(spec.slopes_open):
                raise NotImplementedError(f"the compiled ALiBi closure was checked for {len(spec.slopes_open)} heads, the call has {Hq}")
            slopes = spec.slopes_open[:Hq]
        if slopes is None or len(slopes) != Hq:
            raise ValueError(f"ALiBi has {0 if slopes is None else len(slopes)} slopes for {Hq} heads")
        key = (slopes, str(device))
        t = _slopes_cache.get(key)
        if t is None:
            t = torch.tensor(slopes, dtype=torch.float32, device=device)
            _slopes_cache.put(key, t)
        slopes_ptr = t.data_ptr()
    return _lib.ScoreSpecC(spec.kind, spec.cap, spec.slope, int(mod_q), int(mod_k), 0, slopes_ptr)


def kernel_block_map(pass_id: int, spec: MaskSpec, q: torch.Tensor, Sq: int, Sk: int, D: int, score_fn=None) -> BlockMap:
    bq, bk = _lib.tile_shape(pass_id, dtype_code(q), D)
    if Sq % bq or Sk % bk:
        raise ValueError(f"sequence lengths ({Sq}, {Sk}) must be multiples of the kernel tile ({bq}, {bk})")
    return build_block_map(spec, Sq, Sk, bq, bk, q.device, score_code=score_code_of(score_fn))


def mostly_partial_custom_mask(spec: MaskSpec, bm: BlockMap) -> bool:
    """A compiled mask predicate that leaves most tiles partly masked (a checkerboard, a dilated pattern): the
    generated streams compute a partial step's keep bits in front of the step, one evaluation of the predicate per
    element with nothing to hide it behind, where the kernels with a compiled main loop evaluate it next to the
    other work-group's MFMAs.  The forward and the dq pass then take the compiled-loop kernels (measured on B=4,
    H=32, S=4096 with every tile partial: forward 3.81 -> 2.15 ms, dq 3.65 -> 2.55 ms; dk/dv stays on its stream,
    4.28 against 5.56 ms)."""
    return spec.custom is not None and bm.partial_share() > 0.5


def score_code_of(score_fn):
    """compiler.CustomCode of a compiled score closure, else None."""
    spec = getattr(score_fn, "spec", None)
    return getattr(spec, "custom", None)


def library_for(score_fn, spec: MaskSpec):
    """The library that holds the kernels of this call: libflexattn.so, or the functor library of the call's
    compiled closures (built at first use)."""
    return _lib.load_for(score_code_of(score_fn), spec.custom)


def stream_of(t: torch.Tensor) -> int:
    return raw_stream(t.device)


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_no_switch = _NoSwitch()


def on_device(device):
    """Context that makes `device` the current one for the launch; nothing to enter when it already is (the
    usual case: switching costs the launch path several microseconds, which small problems are bound by)."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _no_switch
    return torch.cuda.device(device)
