"""Shared test helpers: oracle keyword construction and tolerance checks."""
import torch

from oracle import mha_oracle as O

# north-star tolerances
BF16_ABS, BF16_REL = 2e-2, 1e-2
F32_ABS, F32_REL = 1e-5, 1e-5


def oracle_kwargs(cfg):
    """Oracle keywords equivalent to a flex_attention_tpu_amd.configs.AttnConfig."""
    return O.kwargs_for_config(cfg)


def assert_close(name, test, ref, dtype):
    """rel-L2 (benchmark_fwd.py:81-83 of the reference) and max-abs against the tolerance of the
    dtype.  The absolute bound scales with max|ref| when that exceeds 1: a bf16 result cannot
    resolve finer than 2^-9 relative, so 2e-2 absolute is unreachable for |values| > 4 even for a
    correctly rounded output."""
    abs_tol, rel_tol = (BF16_ABS, BF16_REL) if dtype == torch.bfloat16 else (F32_ABS, F32_REL)
    scale = max(1.0, float(ref.abs().max()))
    ma, rl = O.max_abs(test, ref), O.rel_l2(test, ref)
    assert rl <= rel_tol, f"{name}: rel-L2 {rl:.3e} > {rel_tol:.1e} (max-abs {ma:.3e})"
    assert ma <= abs_tol * scale, f"{name}: max-abs {ma:.3e} > {abs_tol:.1e} * {scale:.2f} (rel-L2 {rl:.3e})"
    return ma, rl
