"""Mask factories with the reference's names and call signatures (masks.py of the reference).

Every factory returns ``(mask_fn, block_mask_fn)``:

* ``mask_fn(q_idx, k_idx) -> bool[Bq, Bk]`` on 1-D global index arrays (True = attend),
* ``block_mask_fn(q_block_idx, k_block_idx) -> bool`` "this tile must run",

exactly as the reference's closures do, so they can still be evaluated on index tensors (torch or
NumPy arrays, or plain ints for the block closure).  Each closure also carries ``.spec``, a
``MaskSpec`` the C layer understands; the HIP kernels never call back into Python.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Sequence, Tuple

import numpy as np
import torch

from . import _lib


class DocIds:
    """Immutable per-position document ids (int32) with a precomputed hash: one row [S] for every batch entry, or
    one row per entry, [B, S] (the reference's segment ids of shape [B, S], mha_reference.py:65-73)."""
    __slots__ = ("array", "_key", "_hash")

    def __init__(self, ids):
        arr = np.ascontiguousarray(np.asarray(ids, dtype=np.int32))
        if arr.ndim not in (1, 2):
            raise ValueError("document ids must be a 1-D (or [B, S]) array")
        arr.setflags(write=False)
        self.array = arr
        self._key = (arr.shape, arr.tobytes())
        self._hash = hash(self._key)

    @property
    def batches(self) -> int:
        """Rows of ids: 1 when all batch entries share them."""
        return 1 if self.array.ndim == 1 else self.array.shape[0]

    def rows(self, B: int) -> np.ndarray:
        """The ids as [B, S] (a shared row repeated)."""
        a = self.array if self.array.ndim == 2 else self.array[None, :]
        if a.shape[0] not in (1, B):
            raise ValueError(f"document ids have {a.shape[0]} rows for a batch of {B}")
        return np.ascontiguousarray(np.broadcast_to(a, (B, a.shape[1])))

    def __hash__(self):
        return self._hash

    def __eq__(self, other):
        return isinstance(other, DocIds) and self._key == other._key

    def __len__(self):
        return self.array.shape[-1]

    def is_sorted(self) -> bool:
        """Whether the ids are non-decreasing along the sequence (the reference's jagged mask: masks.py:88-103),
        in every row."""
        a = self.array
        return bool(a.shape[-1] < 2 or (a[..., 1:] >= a[..., :-1]).all())

    def ranges_in(self, other: "DocIds"):
        """int32 [len(self), 2] (with rows per batch entry on either side: [B, len(self), 2]): for every position of
        this array the first and last position of ``other`` (of the same batch entry) that carries the same id
        (first > last where there is none), or None when ``other`` is not sorted (the positions then form no
        interval).  The kernels mask partial tiles of a document mask from these bounds."""
        if not other.is_sorted():
            return None

        def one(mine, theirs):
            lo = np.searchsorted(theirs, mine, side="left")
            hi = np.searchsorted(theirs, mine, side="right") - 1
            return np.stack([lo, hi], axis=1).astype(np.int32)
        if self.batches == 1 and other.batches == 1:
            return np.ascontiguousarray(one(self.array.reshape(-1), other.array.reshape(-1)))
        B = max(self.batches, other.batches)
        mine, theirs = self.rows(B), other.rows(B)
        return np.ascontiguousarray(np.stack([one(mine[b], theirs[b]) for b in range(B)], axis=0))


@dataclass(frozen=True)
class MaskSpec:
    """Machine-readable mask: AND of the flagged terms (S2 stands alone, it contains its own
    window and causal terms)."""
    flags: int = 0
    window: int = 0
    stride: int = 0
    doc_ids: Optional[DocIds] = None      # ids of the q positions (and of the kv positions unless doc_ids_k is given)
    custom: Optional[object] = None       # compiler.CustomCode of a compiled mask closure (flag MASK_CUSTOM)
    doc_ids_k: Optional[DocIds] = None    # ids of the kv positions where they differ from the q side

    def combine(self, other: "MaskSpec") -> "MaskSpec":
        """Spec of the AND of two masks."""
        if self.custom is not None and other.custom is not None and self.custom != other.custom:
            raise NotImplementedError("two different compiled mask functions cannot be combined; AND them in one function")
        custom = self.custom if self.custom is not None else other.custom
        out = self._combine_builtin(other)
        flags = out.flags | ((self.flags | other.flags) & _lib.MASK_CUSTOM)
        doc_k = self.doc_ids_k if self.doc_ids is not None else other.doc_ids_k
        return MaskSpec(flags, out.window, out.stride, out.doc_ids, custom, doc_k)

    def _combine_builtin(self, other: "MaskSpec") -> "MaskSpec":
        if self.doc_ids is not None and other.doc_ids is not None and \
                (self.doc_ids != other.doc_ids or self.doc_ids_k != other.doc_ids_k):
            raise NotImplementedError("two different document masks cannot be combined")
        doc = self.doc_ids if self.doc_ids is not None else other.doc_ids
        if (self.flags | other.flags) & _lib.MASK_S2:
            s2, rest = (self, other) if self.flags & _lib.MASK_S2 else (other, self)
            if rest.flags & (_lib.MASK_WINDOW | _lib.MASK_S2):
                raise NotImplementedError("an S2 mask cannot be combined with another window or S2 mask")
            # S2 is already causal, so AND with causal changes nothing
            return MaskSpec(s2.flags | (rest.flags & _lib.MASK_DOC), s2.window, s2.stride, doc)
        if self.flags & other.flags & _lib.MASK_WINDOW:
            window = min(self.window, other.window)
        else:
            window = self.window or other.window
        return MaskSpec(self.flags | other.flags, window, 0, doc)


def _tag(fn, spec: MaskSpec):
    fn.spec = spec
    return fn


def _to_int(x):
    """bool / bool array -> int32 of the same container kind."""
    if isinstance(x, torch.Tensor):
        return x.to(torch.int32)
    if isinstance(x, np.ndarray) or isinstance(x, np.generic):
        return x.astype(np.int32)
    return int(x)


def _maximum(a, b):
    if isinstance(a, torch.Tensor) or isinstance(b, torch.Tensor):
        return torch.maximum(torch.as_tensor(a), torch.as_tensor(b))
    return np.maximum(a, b)


def _minimum(a, b):
    if isinstance(a, torch.Tensor) or isinstance(b, torch.Tensor):
        return torch.minimum(torch.as_tensor(a), torch.as_tensor(b))
    return np.minimum(a, b)


def place_holder(block_q, block_k_major):
    """No masking: both closures return True (reference masks.py:3-6)."""
    def p(q_block_idx, k_block_idx):
        return True
    _tag(p, MaskSpec())
    return p, p


def make_causal_mask_fns(block_q, block_k_major):
    """Causal mask (reference masks.py:8-30): keep q >= k; run a tile iff k_start <= q_end."""
    def causal_mask_fn(q_idx, k_idx):
        return q_idx[:, None] >= k_idx[None, :]

    def causal_block_mask_fn(q_block_idx, k_block_idx):
        k_start = k_block_idx * block_k_major
        q_end = (q_block_idx + 1) * block_q - 1
        return k_start <= q_end

    spec = MaskSpec(flags=_lib.MASK_CAUSAL)
    return _tag(causal_mask_fn, spec), _tag(causal_block_mask_fn, spec)


def make_sliding_window_mask_fns(block_q, block_k, window_size):
    """Sliding window (reference masks.py:33-83): keep q - k < window_size, with no causal bound
    of its own; run a tile iff q_start - k_end < window_size."""
    def sliding_window_mask_fn(q_idx, k_idx):
        dist = q_idx[:, None] - k_idx[None, :]
        return dist < window_size

    def sliding_window_block_mask_fn(q_block_idx, k_block_idx):
        q_start = q_block_idx * block_q
        k_end = (k_block_idx + 1) * block_k - 1
        return (q_start - k_end) < window_size

    spec = MaskSpec(flags=_lib.MASK_WINDOW, window=int(window_size))
    return _tag(sliding_window_mask_fn, spec), _tag(sliding_window_block_mask_fn, spec)


def _doc_ids_from_lengths(doc_lengths: Sequence[int]) -> DocIds:
    return DocIds(np.repeat(np.arange(len(doc_lengths), dtype=np.int32), np.asarray(doc_lengths, dtype=np.int64)))


def make_jagged_mask_fns(block_q, block_k, doc_lengths):
    """Document ("jagged") mask (reference masks.py:88-141): keep same document AND q >= k; run a
    tile iff the document ranges of the two blocks overlap AND k_start <= q_end."""
    boundaries = [0]
    for n in doc_lengths:
        boundaries.append(boundaries[-1] + int(n))
    boundaries = tuple(boundaries)

    def get_doc_id(idx):
        doc_id = 0
        for b in boundaries[1:]:
            doc_id = doc_id + _to_int(idx >= b)
        return doc_id

    def jagged_mask_fn(q_idx, k_idx):
        doc_q = get_doc_id(q_idx)
        doc_k = get_doc_id(k_idx)
        is_same_doc = doc_q[:, None] == doc_k[None, :]
        is_causal = q_idx[:, None] >= k_idx[None, :]
        return is_same_doc & is_causal

    def jagged_block_mask_fn(q_b, k_b):
        q_start, q_end = q_b * block_q, (q_b + 1) * block_q - 1
        k_start, k_end = k_b * block_k, (k_b + 1) * block_k - 1
        q_doc_min, q_doc_max = get_doc_id(q_start), get_doc_id(q_end)
        k_doc_min, k_doc_max = get_doc_id(k_start), get_doc_id(k_end)
        overlap_start = _maximum(q_doc_min, k_doc_min)
        overlap_end = _minimum(q_doc_max, k_doc_max)
        has_common_doc = overlap_start <= overlap_end
        is_causal = k_start <= q_end
        return has_common_doc & is_causal

    spec = MaskSpec(flags=_lib.MASK_DOC | _lib.MASK_CAUSAL, doc_ids=_doc_ids_from_lengths(doc_lengths))
    return _tag(jagged_mask_fn, spec), _tag(jagged_block_mask_fn, spec)


def make_s2_mask_fns(block_q, block_k, window_size, stride):
    """S2 local + strided mask (reference masks.py:143-179): keep (0 <= q-k < window) or
    (k % stride == 0 and q >= k); run a tile iff k_start <= q_end (the stride term of the
    reference's block closure is always true)."""
    def s2_mask_fn(q_idx, k_idx):
        dist = q_idx[:, None] - k_idx[None, :]
        is_local = (dist >= 0) & (dist < window_size)
        is_strided = (k_idx % stride == 0)
        is_causal = q_idx[:, None] >= k_idx[None, :]
        return is_local | (is_strided[None, :] & is_causal)

    def s2_block_mask_fn(q_b, k_b):
        q_start = q_b * block_q
        k_start = k_b * block_k
        k_end = k_start + block_k - 1
        q_end = q_start + block_q - 1
        is_causal = k_start <= q_end
        in_window = (q_start - k_end) < window_size
        has_stride = True
        return (is_causal & in_window) | (is_causal & has_stride)

    spec = MaskSpec(flags=_lib.MASK_S2, window=int(window_size), stride=int(stride))
    return _tag(s2_mask_fn, spec), _tag(s2_block_mask_fn, spec)


# ------------------------------------------------------------------------------------------------
# Additions the benchmark configurations need and the reference lacks.
# ------------------------------------------------------------------------------------------------
def and_masks(*pairs):
    """AND-composes ``(mask_fn, block_mask_fn)`` pairs, e.g. causal AND sliding window."""
    mask_fns = [p[0] for p in pairs]
    block_fns = [p[1] for p in pairs]

    def and_mask_fn(q_idx, k_idx):
        out = mask_fns[0](q_idx, k_idx)
        for f in mask_fns[1:]:
            out = out & f(q_idx, k_idx)
        return out

    def and_block_mask_fn(q_b, k_b):
        out = block_fns[0](q_b, k_b)
        for f in block_fns[1:]:
            out = out & f(q_b, k_b)
        return out

    spec = mask_fns[0].spec
    for f in mask_fns[1:]:
        spec = spec.combine(f.spec)
    return _tag(and_mask_fn, spec), _tag(and_block_mask_fn, spec)


def make_causal_sliding_window_mask_fns(block_q, block_k, window_size):
    """Causal AND sliding window: keep 0 <= q - k < window_size."""
    return and_masks(make_causal_mask_fns(block_q, block_k),
                     make_sliding_window_mask_fns(block_q, block_k, window_size))


def make_document_mask_fns(block_q, block_k, segment_ids, causal=True):
    """Document mask from a per-position id array (non-decreasing ids), optionally causal."""
    ids = np.asarray(segment_ids.cpu() if isinstance(segment_ids, torch.Tensor) else segment_ids).astype(np.int64)
    if ids.ndim != 1:
        raise ValueError("segment_ids must be 1-D")
    if np.any(np.diff(ids) < 0):
        raise NotImplementedError("segment ids must be non-decreasing along the sequence")
    lengths = np.diff(np.flatnonzero(np.concatenate(([True], ids[1:] != ids[:-1], [True]))))
    mask_fn, block_fn = make_jagged_mask_fns(block_q, block_k, [int(x) for x in lengths])
    if causal:
        return mask_fn, block_fn
    t_ids = torch.from_numpy(ids)

    def doc_mask_fn(q_idx, k_idx):
        return t_ids[q_idx][:, None] == t_ids[k_idx][None, :]

    def doc_block_mask_fn(q_b, k_b):
        q_start, q_end = q_b * block_q, (q_b + 1) * block_q - 1
        k_start, k_end = k_b * block_k, (k_b + 1) * block_k - 1
        lo = _maximum(t_ids[q_start], t_ids[k_start])
        hi = _minimum(t_ids[q_end], t_ids[k_end])
        return lo <= hi

    spec = MaskSpec(flags=_lib.MASK_DOC, doc_ids=mask_fn.spec.doc_ids)
    return _tag(doc_mask_fn, spec), _tag(doc_block_mask_fn, spec)
