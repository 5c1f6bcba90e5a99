"""``make_jax_score_fn`` of the reference's util.py:150-189, for the HIP back end.

The reference AST-rewrites a user score function ``f(q_tile, k_tile) -> [Bq, Bk]`` into
``lax.dot_general`` form so that Pallas can trace it into the kernel.  A HIP kernel cannot trace
Python; the kernels carry compiled functors instead (plain, tile-local ALiBi, tanh soft-cap, global
ALiBi).  This adapter therefore *recognises* which functor a user function is: it evaluates the
function on probe tiles (float64 torch tensors) and matches the result against each functor's
closed form, recovering the constants (cap, slope) from the probe values.  Functions already tagged
by ``flex_attention_tpu_amd.scores`` pass through unchanged.  Anything else raises
``NotImplementedError`` -- a general Python-to-HIP functor compiler is future work.
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


def make_jax_score_fn(user_fn):
    """Returns ``user_fn`` tagged with the ``ScoreSpec`` of the compiled functor it equals."""
    if isinstance(getattr(user_fn, "spec", None), ScoreSpec):
        return user_fn
    g = torch.Generator().manual_seed(1234)
    m, n, d = 24, 40, 16
    q = torch.randn(m, d, generator=g, dtype=torch.float64)
    k = torch.randn(n, d, generator=g, dtype=torch.float64)
    q[0] *= 40.0  # a row of large logits saturates a soft-cap and exposes its cap
    try:
        out = torch.as_tensor(user_fn(q, k)).to(torch.float64)
    except Exception as e:  # noqa: BLE001
        raise NotImplementedError(f"score function could not be evaluated on torch tiles: {e}") from e
    s = q @ k.T
    if out.shape != s.shape:
        raise NotImplementedError(f"score function returned shape {tuple(out.shape)}, expected {tuple(s.shape)}")
    tol = 1e-9 * (1.0 + float(s.abs().max()))
    if float((out - s).abs().max()) <= tol:
        return _tagged(user_fn, ScoreSpec(kind=_lib.SCORE_NONE))
    # tile-local ALiBi: out = s - slope * |row - col|
    dist = (torch.arange(m)[:, None] - torch.arange(n)[None, :]).abs().to(torch.float64)
    diff = s - out
    slope = float(diff[0, 1] / dist[0, 1])
    if slope != 0.0 and float((diff - slope * dist).abs().max()) <= tol:
        return _tagged(user_fn, ScoreSpec(kind=_lib.SCORE_ALIBI_TILE, slope=slope))
    # soft-cap: out = cap * tanh(s / cap); |out| -> cap where |s| is large
    cap = float(out.abs().max())
    if cap > 0.0:
        # refine cap on a moderate logit by bisection of cap*tanh(s/cap) = out
        i = int(torch.argmin((s.abs() - 0.5 * cap).abs()))
        s0, o0 = float(s.flatten()[i]), float(out.flatten()[i])
        lo, hi = 0.5 * cap, 2.0 * cap
        for _ in range(200):
            mid = 0.5 * (lo + hi)
            val = mid * torch.tanh(torch.tensor(abs(s0) / mid, dtype=torch.float64)).item()
            if val < abs(o0):
                lo = mid
            else:
                hi = mid
        for c in (cap, 0.5 * (lo + hi)):
            if float((out - c * torch.tanh(s / c)).abs().max()) <= 1e-7 * (1.0 + c):
                return _tagged(user_fn, ScoreSpec(kind=_lib.SCORE_SOFTCAP, cap=float(round(c, 9))))
    raise NotImplementedError(
        "score function is none of the compiled functors (q k^T, q k^T - slope*|i-j| tile-local, "
        "cap*tanh(q k^T/cap)); use flex_attention_tpu_amd.scores factories")
