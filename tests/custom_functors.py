"""Score and mask closures that the tests compile into the kernels (compiler.py).  They live in a
module of their own so that the build step can compile their functor libraries ahead of the GPU
tests (`__graft_entry__.build()` calls `prebuild()`), which then find them cached."""
import torch

SLOPES = (0.25, 0.0625, 0.015625, 0.00390625)
PREFIX = 96


def alibi_mod(s, b, h, q_idx, kv_idx):
    """global ALiBi written by hand: must equal the built-in functor"""
    return s + SLOPES[h] * (kv_idx - q_idx)


def softcap_mod(s, b, h, q_idx, kv_idx):
    return 20.0 * torch.tanh(s / 20.0)


def mixed_mod(s, b, h, q_idx, kv_idx):
    """a bit of everything: a condition on the indices, abs, a per-head table, min"""
    near = torch.abs(q_idx - kv_idx) < 64
    t = torch.where(near, s, 0.5 * s - 0.25)
    return torch.minimum(t, 3.0 + 0.1 * s) + 0.01 * SLOPES[h] * (q_idx % 7) + 0.2 * torch.tanh(0.5 * s) * (b + 1)


def alibi_symmetric_mod(s, b, h, q_idx, kv_idx):
    """a distance penalty on both sides with the usual slopes computed from the head's index (a power with a
    variable exponent): none of the kernels' own functors"""
    return s - 2.0 ** (-8.0 * (h + 1) / 4) * torch.abs(q_idx - kv_idx)


def alibi_formula_mod(s, b, h, q_idx, kv_idx):
    """global ALiBi with the slopes computed from the head's index: recognised as the kernels' own functor"""
    return s + 2.0 ** (-8.0 * (h + 1) / 4) * (kv_idx - q_idx)


def elementary_mod(s, b, h, q_idx, kv_idx):
    """every elementary function the compiler knows once (sigmoid, exp, sqrt, log, abs), clamp, maximum, //"""
    gate = torch.sigmoid(0.5 * s) * torch.exp(-0.1 * torch.abs(s))
    r = torch.sqrt(1.0 + 0.01 * torch.abs(q_idx - kv_idx)) - torch.log(1.0 + s * s)
    return torch.clamp(s * gate + 0.2 * r, min=-4.0, max=6.0) + 0.05 * torch.maximum(s, 0.1 * (kv_idx // 64 - q_idx // 64))


def softcap30_mod(s, b, h, q_idx, kv_idx):
    return 30.0 * torch.tanh(s / 30.0)


def causal_window_mask(q_idx, k_idx):
    d = q_idx[:, None] - k_idx[None, :]
    return (d >= 0) & (d < 200)


def prefix_lm_mask(q_idx, k_idx):
    """causal, plus a bidirectional prefix"""
    return (q_idx[:, None] >= k_idx[None, :]) | (k_idx[None, :] < PREFIX)


def checker_mask(q_idx, k_idx):
    """keep a key when it shares the query's 32-block parity, or lies within 16 positions before it"""
    d = q_idx[:, None] - k_idx[None, :]
    return ((q_idx[:, None] // 32) % 2 == (k_idx[None, :] // 32) % 2) | ((d >= 0) & (d < 16))


def squared_tile(q_tile, k_tile):
    """tile form of the reference (scores.py): not one of the built-in functors"""
    s = q_tile @ k_tile.T
    return s - 0.05 * s ** 2


def tile_local_distance(q_tile, k_tile):
    """tile-local indices as in the reference's ALiBi (scores.py:3-11), with another profile"""
    m, n = q_tile.shape[0], k_tile.shape[0]
    dist = torch.abs(torch.arange(m)[:, None] - torch.arange(n)[None, :])
    return torch.matmul(q_tile, k_tile.T) - 0.01 * torch.minimum(dist, torch.tensor(50))


def compiled():
    """name -> (score closure or None, (mask_fn, block_mask_fn) or None), compiled at 128 x 128 granularity."""
    from flex_attention_tpu_amd import compiler, util
    return {
        # (written to equal the kernels' own functors: compiled regardless, to compare the two)
        "alibi_mod": (compiler.compile_score_mod(alibi_mod, recognise=False), None),
        "softcap_mod": (compiler.compile_score_mod(softcap_mod, recognise=False), None),
        "mixed_mod": (compiler.compile_score_mod(mixed_mod), None),
        "alibi_symmetric_mod": (compiler.compile_score_mod(alibi_symmetric_mod), None),
        "elementary_mod": (compiler.compile_score_mod(elementary_mod), None),
        "prefix_lm": (None, compiler.compile_mask_fn(prefix_lm_mask, 128, 128)),
        "checker": (None, compiler.compile_mask_fn(checker_mask, 128, 128)),
        "mixed_mod+prefix_lm": (compiler.compile_score_mod(mixed_mod), compiler.compile_mask_fn(prefix_lm_mask, 128, 128)),
        "squared_tile": (util.make_jax_score_fn(squared_tile), None),
        "tile_local_distance": (util.make_jax_score_fn(tile_local_distance), None),
    }


def prebuild(force=False):
    """Compiles the functor library of every pair above (hipcc, gfx950; cached on disk unless `force`)."""
    from flex_attention_tpu_amd import compiler
    paths = []
    for name, (score, mask) in compiled().items():
        sc = score.spec.custom if score is not None else None
        mc = mask[0].spec.custom if mask is not None else None
        paths.append(compiler.build_functor_library(sc, mc, force=force))
    return paths
