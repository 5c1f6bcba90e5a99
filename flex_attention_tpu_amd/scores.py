"""Score-mod factories with the reference's names (scores.py of the reference).

Each factory returns a closure ``score_fn(q_tile, k_tile) -> [Bq, Bk]`` on torch tensors, as the
reference's closures are on jnp arrays, and tags it with ``.spec`` (a ``ScoreSpec``) that selects
the compiled functor inside the HIP kernels.  Convention of this build for ``sm_scale``:
the kernels compute ``score_mod(sm_scale * <q, k>)``; every reference driver uses ``sm_scale=1``
with score functions, where all conventions coincide.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import _lib


@dataclass(frozen=True)
class ScoreSpec:
    kind: int = _lib.SCORE_NONE
    cap: float = 0.0
    slope: float = 0.0
    slopes: Optional[Tuple[float, ...]] = None  # per-head slopes (global ALiBi)
    # (global ALiBi of a compiled closure whose slope is a function of the head's index: the slopes of heads 0, 1, ...
    # as far as they were checked; a call takes the first Hq of them)
    slopes_open: Optional[Tuple[float, ...]] = None
    custom: Optional[object] = None             # compiler.CustomCode of a compiled closure (kind SCORE_CUSTOM)


def _tag(fn, spec):
    fn.spec = spec
    return fn


def make_alibi_score_fn(slope=0.5):
    """Tile-local ALiBi of the reference (scores.py:3-11): q k^T - slope * |row - col| with row/col
    counted inside the tile the kernel hands over (block_q x block_k)."""
    def alibi_score(q_tile, k_tile):
        score = q_tile @ k_tile.T
        m, n = q_tile.shape[0], k_tile.shape[0]
        dist = (torch.arange(m)[:, None] - torch.arange(n)[None, :]).abs()
        return score - (slope * dist).to(score.dtype)
    return _tag(alibi_score, ScoreSpec(kind=_lib.SCORE_ALIBI_TILE, slope=float(slope)))


def make_softcap_score_fn(cap=30.0):
    """Tanh soft-cap (scores.py:13-18): cap * tanh(q k^T / cap)."""
    def softcap_score(q_tile, k_tile):
        logits = q_tile @ k_tile.T
        return cap * torch.tanh(logits / cap)
    return _tag(softcap_score, ScoreSpec(kind=_lib.SCORE_SOFTCAP, cap=float(cap)))


def alibi_slopes(num_heads: int):
    """slope_h = 2^(-8 (h+1) / H) for h = 0 .. H-1."""
    return tuple(2.0 ** (-8.0 * (h + 1) / num_heads) for h in range(num_heads))


def make_alibi_global_score_fn(num_heads: int, slopes=None):
    """True ALiBi with global token indices and one slope per head:
    score + slope_h * (kv_idx - q_idx).  The tile callable form cannot see the head or the global
    position, so calling the closure directly evaluates head 0 at offset 0; the kernels and the
    dense checker use ``.spec``."""
    slopes = tuple(float(s) for s in (slopes if slopes is not None else alibi_slopes(num_heads)))

    def alibi_global_score(q_tile, k_tile, head=0, q_start=0, k_start=0):
        score = q_tile @ k_tile.T
        qi = q_start + torch.arange(q_tile.shape[0])[:, None]
        kj = k_start + torch.arange(k_tile.shape[0])[None, :]
        return score + (slopes[head] * (kj - qi)).to(score.dtype)
    return _tag(alibi_global_score, ScoreSpec(kind=_lib.SCORE_ALIBI, slopes=slopes))
