"""Pins the CPU oracle against independent routines (none of these retype its formulas):
torch SDPA, torch.logsumexp, autograd through an independently written softmax, central finite
differences, repeat_interleave reduction of GQA, brute-force masks, and committed golden vectors."""
import math
import os

import numpy as np
import pytest
import torch

from oracle import mha_oracle as O

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _inputs(B=1, Hq=2, Hkv=2, S=64, D=16, seed=3):
    return O.make_inputs(B, Hq, Hkv, S, S, D, dtype=torch.float64, seed=seed)


@pytest.mark.parametrize("causal", [False, True])
def test_forward_matches_sdpa(causal):
    q, k, v, _ = _inputs()
    out = O.mha_reference(q, k, v, sm_scale=0.3, causal=causal)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=causal, scale=0.3)
    assert (out - ref).abs().max() < 1e-12


def test_residuals_match_logsumexp():
    q, k, v, _ = _inputs()
    _, l, m = O.mha_reference(q, k, v, sm_scale=0.25, save_residuals=True, causal=True)
    s = torch.einsum("bhqc,bhkc->bhqk", q, k) * 0.25
    s = s.masked_fill(~torch.ones(64, 64, dtype=torch.bool).tril(), float("-inf"))
    assert (m - s.max(-1).values).abs().max() < 1e-12
    assert ((m + l.log()) - torch.logsumexp(s, -1)).abs().max() < 1e-12


@pytest.mark.parametrize("causal", [False, True])
def test_backward_matches_autograd_of_sdpa(causal):
    q, k, v, do = _inputs()
    o, l, m = O.mha_reference(q, k, v, sm_scale=0.3, save_residuals=True, causal=causal)
    dq, dk, dv = O.mha_bwd_reference(q, k, v, o, do, l, m, causal=causal, sm_scale=0.3)
    qd, kd, vd = [x.clone().requires_grad_() for x in (q, k, v)]
    r = torch.nn.functional.scaled_dot_product_attention(qd, kd, vd, is_causal=causal, scale=0.3)
    gq, gk, gv = torch.autograd.grad(r, (qd, kd, vd), do)
    for a, b in ((dq, gq), (dk, gk), (dv, gv)):
        assert (a - b).abs().max() < 1e-11


def test_backward_finite_differences_softcap_window():
    """A dropped term, wrong sign or transposed operand in the backward fails this."""
    B, H, S, D = 1, 1, 8, 4
    q, k, v, do = O.make_inputs(B, H, H, S, S, D, dtype=torch.float64, seed=5)
    kw = dict(sm_scale=0.7, causal=True, window_size=5, score_mod=O.score_mod_softcap(2.0))
    o, l, m = O.mha_reference(q, k, v, save_residuals=True, **kw)
    dq, dk, dv = O.mha_bwd_reference(q, k, v, o, do, l, m, **kw)

    def loss(q_, k_, v_):
        return float((O.mha_reference(q_, k_, v_, **kw) * do).sum())

    eps = 1e-6
    for name, x, g in (("q", q, dq), ("k", k, dk), ("v", v, dv)):
        for idx in [(0, 0, 0, 0), (0, 0, 3, 2), (0, 0, 7, 3), (0, 0, 5, 1)]:
            xp, xm = x.clone(), x.clone()
            xp[idx] += eps
            xm[idx] -= eps
            args_p = {"q": q, "k": k, "v": v}
            args_m = dict(args_p)
            args_p[name], args_m[name] = xp, xm
            fd = (loss(args_p["q"], args_p["k"], args_p["v"]) - loss(args_m["q"], args_m["k"], args_m["v"])) / (2 * eps)
            assert abs(fd - float(g[idx])) < 1e-6, (name, idx, fd, float(g[idx]))


def test_delta_invariant():
    """delta_i = sum_c o*do equals sum_j P_ij dP_ij."""
    q, k, v, do = _inputs()
    o = O.mha_reference(q, k, v, sm_scale=0.3)
    p = torch.softmax(torch.einsum("bhqc,bhkc->bhqk", q, k) * 0.3, -1)
    dp = torch.einsum("bhqc,bhkc->bhqk", do, v)
    assert (O.delta(o, do) - (p * dp).sum(-1)).abs().max() < 1e-12


def test_gqa_reduces_to_mha():
    q, k, v, do = O.make_inputs(1, 4, 2, 32, 32, 8, dtype=torch.float64, seed=7)
    kw = dict(sm_scale=0.4, causal=True)
    o, l, m = O.mha_reference(q, k, v, save_residuals=True, **kw)
    dq, dk, dv = O.mha_bwd_reference(q, k, v, o, do, l, m, **kw)
    kr, vr = k.repeat_interleave(2, 1), v.repeat_interleave(2, 1)
    o2, l2, m2 = O.mha_reference(q, kr, vr, save_residuals=True, **kw)
    dq2, dk2, dv2 = O.mha_bwd_reference(q, kr, vr, o2, do, l2, m2, **kw)
    assert (o - o2).abs().max() < 1e-13 and (dq - dq2).abs().max() < 1e-13
    assert (dk - dk2.reshape(1, 2, 2, 32, 8).sum(2)).abs().max() < 1e-12
    assert (dv - dv2.reshape(1, 2, 2, 32, 8).sum(2)).abs().max() < 1e-12
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, scale=0.4, enable_gqa=True)
    assert (o - ref).abs().max() < 1e-12


def test_score_mod_paths_agree_with_autograd():
    """ALiBi and softcap backward (VJP path) against autograd of an independent dense softmax."""
    q, k, v, do = O.make_inputs(1, 2, 2, 16, 16, 8, dtype=torch.float64, seed=11)
    slopes = O.alibi_slopes(2)
    for mod in (O.score_mod_alibi_global(slopes), O.score_mod_softcap(3.0)):
        kw = dict(sm_scale=0.5, causal=True, score_mod=mod)
        o, l, m = O.mha_reference(q, k, v, save_residuals=True, **kw)
        dq, dk, dv = O.mha_bwd_reference(q, k, v, o, do, l, m, **kw)
        qd, kd, vd = [x.clone().requires_grad_() for x in (q, k, v)]
        outs = []
        for h in range(2):
            s = (qd[0, h] @ kd[0, h].T) * 0.5
            i = torch.arange(16)[:, None]
            j = torch.arange(16)[None, :]
            s = mod(s, 0, h, i, j)
            s = s.masked_fill(j > i, float("-inf"))
            outs.append(torch.softmax(s, -1) @ vd[0, h])
        r = torch.stack(outs)[None]
        assert (r - o).abs().max() < 1e-12
        gq, gk, gv = torch.autograd.grad(r, (qd, kd, vd), do)
        for a, b in ((dq, gq), (dk, gk), (dv, gv)):
            assert (a - b).abs().max() < 1e-11


def test_tile_score_fn_path_is_vjp_of_callable():
    """score_fn (tile callable, no sm_scale) path, as mha_reference.py:42-48 / :232-234."""
    q, k, v, do = O.make_inputs(1, 1, 1, 16, 16, 8, dtype=torch.float64, seed=2)
    fn = lambda qt, kt: 3.0 * torch.tanh((qt @ kt.T) / 3.0)
    o, l, m = O.mha_reference(q, k, v, save_residuals=True, score_fn=fn)
    dq, dk, dv = O.mha_bwd_reference(q, k, v, o, do, l, m, score_fn=fn)
    qd, kd, vd = [x.clone().requires_grad_() for x in (q, k, v)]
    r = torch.softmax(fn(qd[0, 0], kd[0, 0]), -1) @ vd[0, 0]
    gq, gk, gv = torch.autograd.grad(r, (qd, kd, vd), do[0, 0])
    assert (r - o[0, 0]).abs().max() < 1e-12
    for a, b in ((dq, gq), (dk, gk), (dv, gv)):
        assert (a - b).abs().max() < 1e-11


def test_mask_kwargs_match_bruteforce_loops():
    S = 24
    sid = O.doc_ids_from_lengths([5, 11, 8])
    for kw in (dict(causal=True), dict(window_size=7), dict(causal=True, window_size=4),
               dict(causal=True, segment_ids=sid), dict(window_size=6, s2_stride=4, causal=True)):
        keep = O._keep_rows(S, torch.arange(S), mask=None, b=0,
                            **{"causal": False, "window_size": None, "segment_ids": None, "s2_stride": None, **kw})
        for i in range(S):
            for j in range(S):
                e = True
                if kw.get("causal"):
                    e = e and j <= i
                if kw.get("segment_ids") is not None:
                    e = e and int(sid[i]) == int(sid[j])
                if kw.get("window_size") is not None:
                    too_old = (i - j) >= kw["window_size"]
                    if kw.get("s2_stride") is not None:
                        too_old = too_old and (j % kw["s2_stride"] != 0)
                    e = e and not too_old
                assert bool(keep[i, j]) == e, (kw, i, j)


def test_block_map_closed_form_vs_bruteforce():
    """Closed forms equal any(mask) for causal, window and (monotone ids) documents."""
    S, bq, bk = 256, 32, 16
    lens = [40, 100, 7, 109]
    sid = O.doc_ids_from_lengths(lens)
    for kw in (dict(causal=True), dict(window_size=50), dict(causal=True, window_size=33),
               dict(causal=True, segment_ids=sid)):
        keep = O.dense_mask(S, S, **kw)
        brute = O.block_map_bruteforce(keep, bq, bk)
        closed = O.block_map_closed_form(S // bq, S // bk, bq, bk, **kw)
        if "window_size" in kw and "causal" in kw:
            # the AND of two closures is conservative: it may run a tile with no kept element
            assert bool((closed | ~(brute != 0)).all())
        else:
            assert torch.equal(closed, brute != 0), kw


def test_row_subset_matches_full():
    q, k, v, do = O.make_inputs(1, 2, 1, 64, 64, 8, dtype=torch.float64, seed=9)
    kw = dict(sm_scale=0.3, causal=True, score_mod=O.score_mod_softcap(4.0))
    o, l, m = O.mha_reference(q, k, v, save_residuals=True, **kw)
    rows = torch.tensor([0, 5, 31, 63])
    o2, l2, m2 = O.mha_reference(q, k, v, save_residuals=True, q_rows=rows, **kw)
    assert torch.equal(o[:, :, rows], o2)
    do_s = torch.zeros_like(do)
    do_s[:, :, rows] = do[:, :, rows]
    dq, dk, dv = O.mha_bwd_reference(q, k, v, o, do_s, l, m, **kw)
    dq2, dk2, dv2 = O.mha_bwd_reference(q, k, v, o2, do[:, :, rows], l2, m2, q_rows=rows, **kw)
    assert (dq[:, :, rows] - dq2).abs().max() < 1e-14
    assert (dk - dk2).abs().max() < 1e-13 and (dv - dv2).abs().max() < 1e-13


def test_segment_lengths_properties():
    for seed in range(5):
        lens = O.make_segment_lengths(16384, seed=seed)
        assert sum(lens) == 16384 and min(lens) >= 512 and max(lens) <= 4096 + 511


def test_golden_vectors():
    """Regression of the oracle itself against committed float64 vectors (tests/golden)."""
    g = np.load(os.path.join(GOLDEN, "oracle_tiny.npz"))
    q, k, v, do = [torch.from_numpy(g[n]) for n in ("q", "k", "v", "do")]
    sid = torch.from_numpy(g["segment_ids"])
    kw = dict(sm_scale=float(g["sm_scale"]), causal=True, segment_ids=sid, score_mod=O.score_mod_softcap(float(g["cap"])))
    o, l, m = O.mha_reference(q, k, v, save_residuals=True, **kw)
    dq, dk, dv = O.mha_bwd_reference(q, k, v, o, do, l, m, **kw)
    for name, t in (("o", o), ("l", l), ("m", m), ("dq", dq), ("dk", dk), ("dv", dv)):
        assert np.allclose(t.numpy(), g[name], rtol=0, atol=1e-12), name


@pytest.mark.parametrize("causal", [False, True])
def test_additive_bias_branch_matches_sdpa_float_mask(causal):
    """`ab=` (mha_reference.py:50-51: added behind the score function, in front of the masks) against
    SDPA with a float ``attn_mask`` (added to the scaled logits), forward and autograd backward; under
    `causal` the float mask carries -inf above the diagonal.  A bias that was dropped, scaled by sm_scale
    or added behind the mask fails here."""
    q, k, v, do = O.make_inputs(2, 3, 3, 40, 56, 16, dtype=torch.float64, seed=13)
    g = torch.Generator().manual_seed(14)
    ab = torch.randn(2, 3, 40, 56, generator=g, dtype=torch.float64) * 2
    kw = dict(sm_scale=0.3, causal=causal)
    o, l, m = O.mha_reference(q, k, v, ab, save_residuals=True, **kw)
    dq, dk, dv = O.mha_bwd_reference(q, k, v, o, do, l, m, ab, **kw)
    bias = ab.clone()
    if causal:
        bias = bias.masked_fill(torch.arange(56)[None, :] > torch.arange(40)[:, None], float("-inf"))
    qd, kd, vd = [x.clone().requires_grad_() for x in (q, k, v)]
    r = torch.nn.functional.scaled_dot_product_attention(qd, kd, vd, attn_mask=bias, scale=0.3)
    assert (o - r).abs().max() < 1e-12
    s = torch.einsum("bhqc,bhkc->bhqk", q, k) * 0.3 + bias
    assert ((m + l.log()) - torch.logsumexp(s, -1)).abs().max() < 1e-12
    gq, gk, gv = torch.autograd.grad(r, (qd, kd, vd), do)
    for a, b in ((dq, gq), (dk, gk), (dv, gv)):
        assert (a - b).abs().max() < 1e-11


def test_additive_bias_with_score_mod_and_gqa_matches_autograd():
    """`ab=` next to a score function and grouped kv heads: the bias is added to the *modified* logits
    (softcap first, then + ab) -- against autograd of an independently written dense softmax."""
    q, k, v, do = O.make_inputs(1, 4, 2, 24, 24, 8, dtype=torch.float64, seed=15)
    ab = torch.randn(1, 4, 24, 24, generator=torch.Generator().manual_seed(16), dtype=torch.float64)
    kw = dict(sm_scale=0.6, causal=True, score_mod=O.score_mod_softcap(2.5))
    o, l, m = O.mha_reference(q, k, v, ab, save_residuals=True, **kw)
    dq, dk, dv = O.mha_bwd_reference(q, k, v, o, do, l, m, ab, **kw)
    qd, kd, vd = [x.clone().requires_grad_() for x in (q, k, v)]
    outs = []
    for h in range(4):
        s = 2.5 * torch.tanh((qd[0, h] @ kd[0, h // 2].T) * 0.6 / 2.5) + ab[0, h]
        s = s.masked_fill(torch.arange(24)[None, :] > torch.arange(24)[:, None], float("-inf"))
        outs.append(torch.softmax(s, -1) @ vd[0, h // 2])
    r = torch.stack(outs)[None]
    assert (r - o).abs().max() < 1e-12
    gq, gk, gv = torch.autograd.grad(r, (qd, kd, vd), do)
    for a, b in ((dq, gq), (dk, gk), (dv, gv)):
        assert (a - b).abs().max() < 1e-11


@pytest.mark.parametrize("per_batch", [False, True])
def test_dense_mask_branch_matches_sdpa_bool_mask(per_batch):
    """`mask=` (an arbitrary boolean keep mask, [Sq, Sk] or one per batch entry) against SDPA with a boolean
    ``attn_mask`` (True = attend), forward and autograd backward.  Every row keeps at least one key."""
    B, H, Sq, Sk = 2, 2, 32, 48
    q, k, v, do = O.make_inputs(B, H, H, Sq, Sk, 16, dtype=torch.float64, seed=17)
    g = torch.Generator().manual_seed(18)
    keep = torch.rand((B, Sq, Sk) if per_batch else (Sq, Sk), generator=g) < 0.4
    keep[..., 0] = True
    kw = dict(sm_scale=0.35, mask=keep)
    o, l, m = O.mha_reference(q, k, v, save_residuals=True, **kw)
    dq, dk, dv = O.mha_bwd_reference(q, k, v, o, do, l, m, **kw)
    qd, kd, vd = [x.clone().requires_grad_() for x in (q, k, v)]
    am = keep[:, None] if per_batch else keep
    r = torch.nn.functional.scaled_dot_product_attention(qd, kd, vd, attn_mask=am, scale=0.35)
    assert (o - r).abs().max() < 1e-12
    gq, gk, gv = torch.autograd.grad(r, (qd, kd, vd), do)
    for a, b in ((dq, gq), (dk, gk), (dv, gv)):
        assert (a - b).abs().max() < 1e-11
    # the mask composes with the keyword masks by AND
    o2 = O.mha_reference(q, k, v, causal=True, **kw)
    both = am & (torch.arange(Sk)[None, :] <= torch.arange(Sq)[:, None])
    r2 = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=both, scale=0.35)
    assert (o2 - r2).abs().max() < 1e-12


def test_legacy_alibi_slope_branch_matches_sdpa_float_mask():
    """`alibi_slope=` (the tile-local bias the reference's dense code mimics with `% 1024` / `% 512`,
    mha_reference.py:35-41): logits - slope |i % mod_q - j % mod_k|, here as a float attn_mask of SDPA."""
    S = 40
    q, k, v, do = O.make_inputs(1, 2, 2, S, S, 8, dtype=torch.float64, seed=19)
    kw = dict(sm_scale=0.5, alibi_slope=0.7, alibi_mods=(16, 8))
    o, l, m = O.mha_reference(q, k, v, save_residuals=True, **kw)
    dq, dk, dv = O.mha_bwd_reference(q, k, v, o, do, l, m, **kw)
    i, j = torch.arange(S)[:, None], torch.arange(S)[None, :]
    bias = -0.7 * ((i % 16) - (j % 8)).abs().to(torch.float64)
    qd, kd, vd = [x.clone().requires_grad_() for x in (q, k, v)]
    r = torch.nn.functional.scaled_dot_product_attention(qd, kd, vd, attn_mask=bias, scale=0.5)
    assert (o - r).abs().max() < 1e-12
    gq, gk, gv = torch.autograd.grad(r, (qd, kd, vd), do)
    for a, b in ((dq, gq), (dk, gk), (dv, gv)):
        assert (a - b).abs().max() < 1e-11


def test_bias_gradient_matches_autograd_of_sdpa():
    """`return_dab`: the gradient of the additive bias is ds = p (dp - delta), neither scaled by sm_scale nor by
    the score function's derivative -- against autograd through SDPA with a float ``attn_mask`` that requires
    grad (causal folded into the mask as -inf, whose entries receive no gradient), and with a softcap score
    through an independently written softmax."""
    B, H, Sq, Sk = 2, 2, 24, 40
    q, k, v, do = O.make_inputs(B, H, H, Sq, Sk, 8, dtype=torch.float64, seed=21)
    ab = torch.randn(B, H, Sq, Sk, generator=torch.Generator().manual_seed(22), dtype=torch.float64)
    kw = dict(sm_scale=0.37, causal=True)
    o, l, m = O.mha_reference(q, k, v, ab, save_residuals=True, **kw)
    dq, dk, dv, dab = O.mha_bwd_reference(q, k, v, o, do, l, m, ab, return_dab=True, **kw)
    above = torch.arange(Sk)[None, :] > torch.arange(Sq)[:, None]
    abd = ab.clone().requires_grad_()
    r = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=abd.masked_fill(above, float("-inf")), scale=0.37)
    (g,) = torch.autograd.grad(r, abd, do)
    assert (dab - g).abs().max() < 1e-12 and float(g.abs().max()) > 1e-3
    assert float(dab[..., above].abs().max()) == 0.0
    # softcap in front of the bias: d logits / d ab is still 1
    kw = dict(sm_scale=0.5, score_mod=O.score_mod_softcap(1.5))
    o, l, m = O.mha_reference(q, k, v, ab, save_residuals=True, **kw)
    dab = O.mha_bwd_reference(q, k, v, o, do, l, m, ab, return_dab=True, **kw)[3]
    abd = ab.clone().requires_grad_()
    s = 1.5 * torch.tanh(torch.einsum("bhqc,bhkc->bhqk", q, k) * 0.5 / 1.5) + abd
    (g,) = torch.autograd.grad(torch.softmax(s, -1) @ v, abd, do)
    assert (dab - g).abs().max() < 1e-12
