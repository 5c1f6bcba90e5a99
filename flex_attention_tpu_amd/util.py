"""``make_jax_score_fn`` of the reference's util.py:150-189, for the HIP back end.

The reference AST-rewrites a user score function ``f(q_tile, k_tile) -> [Bq, Bk]`` into
``lax.dot_general`` form so that Pallas can trace it into the kernel.  A HIP kernel cannot trace
Python, so the function is compiled ahead of time instead:

* if it equals one of the functors the generated-stream kernels carry (plain ``q k^T``, tile-local
  ALiBi, tanh soft-cap) it is tagged with that functor's spec and gets those kernels.  The match is
  numeric: the function is evaluated on two independent probe tiles of different shapes, the
  constants (cap, slope) are recovered from the first and must reproduce the second;
* anything else goes through ``compiler.compile_score_fn``: its source is rewritten into an
  expression tree, differentiated, printed as a HIP functor and compiled into the kernels with a
  compiled main loop (hipcc at first use, cached on disk).  Constructs the rewriter does not
  understand raise ``NotImplementedError`` naming the construct.

Functions already tagged by ``flex_attention_tpu_amd.scores`` or the compiler pass through unchanged.
"""
from __future__ import annotations

import torch

from . import _lib
from .scores import ScoreSpec


def _tagged(fn, spec):
    def score_fn(q_tile, k_tile):
        return fn(q_tile, k_tile)
    score_fn.spec = spec
    score_fn.__name__ = getattr(fn, "__name__", "score_fn")
    score_fn.__wrapped__ = fn
    return score_fn


def _probe(user_fn, m, n, d, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(m, d, generator=g, dtype=torch.float64)
    k = torch.randn(n, d, generator=g, dtype=torch.float64)
    q[0] *= 40.0  # a row of large logits saturates a soft-cap and exposes its cap
    out = torch.as_tensor(user_fn(q, k)).to(torch.float64)
    s = q @ k.T
    if out.shape != s.shape:
        raise NotImplementedError(f"score function returned shape {tuple(out.shape)}, expected {tuple(s.shape)}")
    dist = (torch.arange(m)[:, None] - torch.arange(n)[None, :]).abs().to(torch.float64)
    return s, out, dist


def _matches(spec: ScoreSpec, s, out, dist) -> bool:
    tol = 1e-9 * (1.0 + float(s.abs().max()))
    if spec.kind == _lib.SCORE_NONE:
        return float((out - s).abs().max()) <= tol
    if spec.kind == _lib.SCORE_ALIBI_TILE:
        return float((s - spec.slope * dist - out).abs().max()) <= tol
    return float((out - spec.cap * torch.tanh(s / spec.cap)).abs().max()) <= 1e-9 * (1.0 + spec.cap)


def _recognise(user_fn):
    """ScoreSpec of the stream-kernel functor the function equals, or None."""
    s, out, dist = _probe(user_fn, 24, 40, 16, 1234)
    cands = [ScoreSpec(kind=_lib.SCORE_NONE)]
    slope = float((s - out)[0, 1] / dist[0, 1])
    if slope != 0.0:
        cands.append(ScoreSpec(kind=_lib.SCORE_ALIBI_TILE, slope=slope))
    cap = float(out.abs().max())
    if cap > 0.0:
        # refine the cap on a moderate logit by bisection of cap * tanh(s / cap) = out
        i = int(torch.argmin((s.abs() - 0.5 * cap).abs()))
        s0, o0 = float(s.flatten()[i]), float(out.flatten()[i])
        lo, hi = 0.5 * cap, 2.0 * cap
        for _ in range(200):
            mid = 0.5 * (lo + hi)
            if mid * torch.tanh(torch.tensor(abs(s0) / mid, dtype=torch.float64)).item() < abs(o0):
                lo = mid
            else:
                hi = mid
        cands += [ScoreSpec(kind=_lib.SCORE_SOFTCAP, cap=float(round(c, 9))) for c in (cap, 0.5 * (lo + hi))]
    second = _probe(user_fn, 56, 72, 32, 99)   # another shape, depth and seed: a function that only looks like a
    for spec in cands:                         # closed form on the first probe does not pass
        if _matches(spec, s, out, dist) and _matches(spec, *second):
            return spec
    return None


def make_jax_score_fn(user_fn):
    """Returns ``user_fn`` tagged with the spec of the device functor that computes it."""
    if isinstance(getattr(user_fn, "spec", None), ScoreSpec):
        return user_fn
    try:
        spec = _recognise(user_fn)
    except NotImplementedError:
        raise
    except Exception as e:  # noqa: BLE001
        raise NotImplementedError(f"score function could not be evaluated on torch tiles: {e}") from e
    if spec is not None:
        return _tagged(user_fn, spec)
    from . import compiler
    return compiler.compile_score_fn(user_fn)
