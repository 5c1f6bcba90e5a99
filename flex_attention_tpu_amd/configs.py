"""The five benchmark configurations (synthetic inputs, masks and score mods) as plain data.

Inputs are drawn from ``torch.Generator(device="cpu").manual_seed(seed)``: Q, K, V, dO ~ N(0,1)
as independent float32 draws in that order, then cast to the configuration's dtype.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

from . import masks, scores


@dataclass(frozen=True)
class AttnConfig:
    name: str
    dtype: torch.dtype
    B: int
    Hq: int
    Hkv: int
    S: int
    D: int
    mask: str = "none"        # none | causal | causal_window | document
    window: int = 0           # causal_window: keep 0 <= i - j <= window
    score: str = "none"       # none | alibi | softcap
    cap: float = 30.0
    seed: int = 0
    block: int = 128          # block size handed to the mask factories / entry points

    @property
    def sm_scale(self) -> float:
        return 1.0 / math.sqrt(self.D)


CONFIGS: Dict[str, AttnConfig] = {
    "cfg1": AttnConfig("cfg1", torch.float32, 1, 4, 4, 512, 64),
    "cfg2": AttnConfig("cfg2", torch.bfloat16, 4, 32, 32, 4096, 128, mask="causal"),
    "cfg3": AttnConfig("cfg3", torch.bfloat16, 4, 32, 32, 4096, 128, mask="causal"),
    "cfg4": AttnConfig("cfg4", torch.bfloat16, 2, 16, 16, 8192, 128, mask="causal_window", window=1024,
                       score="alibi"),
    "cfg5": AttnConfig("cfg5", torch.bfloat16, 1, 32, 8, 16384, 128, mask="document", score="softcap", cap=30.0),
}

# Not one of the reference's configurations: the FLOPs of cfg2 at head dimension 256 (half the heads), which the
# reference's kernels accept (flex_attention_kernel.py:302-306) and none of its drivers runs.  bench.py reports it
# next to the others.
EXTRA_CONFIGS: Dict[str, AttnConfig] = {
    "d256": AttnConfig("d256", torch.bfloat16, 4, 16, 16, 4096, 256, mask="causal"),
}


def make_inputs(cfg: AttnConfig, device="cpu"):
    g = torch.Generator(device="cpu").manual_seed(cfg.seed)
    q = torch.randn(cfg.B, cfg.Hq, cfg.S, cfg.D, generator=g, dtype=torch.float32).to(cfg.dtype)
    k = torch.randn(cfg.B, cfg.Hkv, cfg.S, cfg.D, generator=g, dtype=torch.float32).to(cfg.dtype)
    v = torch.randn(cfg.B, cfg.Hkv, cfg.S, cfg.D, generator=g, dtype=torch.float32).to(cfg.dtype)
    do = torch.randn(cfg.B, cfg.Hq, cfg.S, cfg.D, generator=g, dtype=torch.float32).to(cfg.dtype)
    return tuple(t.to(device) for t in (q, k, v, do))


def segment_lengths(total_len: int, lo: int = 512, hi: int = 4096, seed: int = 0) -> List[int]:
    """Document lengths uniform in [lo, hi] summing to total_len: draw ``rng.integers(lo, hi+1)``
    until the sum reaches total_len, clip the last, merge a tail shorter than ``lo`` into its
    predecessor (numpy ``default_rng(seed)``)."""
    rng = np.random.default_rng(seed)
    lens, tot = [], 0
    while tot < total_len:
        n = min(int(rng.integers(lo, hi + 1)), total_len - tot)
        lens.append(n)
        tot += n
    if len(lens) > 1 and lens[-1] < lo:
        tail = lens.pop()
        lens[-1] += tail
    return lens


def mask_fns(cfg: AttnConfig):
    """(mask_fn, block_mask_fn) of the configuration, or (None, None)."""
    if cfg.mask == "none":
        return None, None
    if cfg.mask == "causal":
        return masks.make_causal_mask_fns(cfg.block, cfg.block)
    if cfg.mask == "causal_window":
        # |i - j| <= window together with causal  ==  0 <= i - j < window + 1
        return masks.make_causal_sliding_window_mask_fns(cfg.block, cfg.block, cfg.window + 1)
    if cfg.mask == "document":
        return masks.make_jagged_mask_fns(cfg.block, cfg.block, segment_lengths(cfg.S, seed=cfg.seed))
    raise ValueError(cfg.mask)


def score_fn(cfg: AttnConfig):
    if cfg.score == "none":
        return None
    if cfg.score == "alibi":
        return scores.make_alibi_global_score_fn(cfg.Hq)
    if cfg.score == "softcap":
        return scores.make_softcap_score_fn(cfg.cap)
    raise ValueError(cfg.score)


def n_pairs_per_head(cfg: AttnConfig) -> float:
    """Unmasked (i, j) pairs per head under the benchmark's FLOP convention (causal counts S^2/2)."""
    S = cfg.S
    if cfg.mask == "none":
        return float(S) * S
    if cfg.mask == "causal":
        return S * S / 2.0
    if cfg.mask == "causal_window":
        w = cfg.window + 1
        return float(sum(min(i + 1, w) for i in range(S)))
    if cfg.mask == "document":
        return float(sum(n * (n + 1) // 2 for n in segment_lengths(S, seed=cfg.seed)))
    raise ValueError(cfg.mask)


def flops_fwd(cfg: AttnConfig) -> float:
    """Algorithmic forward FLOPs: 4 * B * Hq * D * N_pairs (backward = 2.5x)."""
    return 4.0 * cfg.B * cfg.Hq * cfg.D * n_pairs_per_head(cfg)
