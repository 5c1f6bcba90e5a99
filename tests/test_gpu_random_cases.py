"""Seeded random cases that combine the features the other GPU tests take one at a time: dtype, head dimension
(the kernels' own and zero-padded ones), grouped heads, lengths that are no multiple of a tile and differ between
q and kv, the built-in masks and the `causal` flag, compiled closures, the score functions, segment ids in every
accepted form (one row or one per batch entry; common or separate for q and kv; sorted or not), the additive
bias in its broadcast shapes with its gradient, the compiled-loop kernels on request, the dS hand-over between
the backward passes and the autograd wrapper.  Every case goes through the three entry points and is compared
with the CPU oracle: the forward with the oracle's forward, the backward with the oracle's backward from the
kernels' own residuals (the reference's method for its backward kernels, flex_attention_dq_bwd.py:920-946).

The oracle masks through a dense [B, Sq, Sk] keep matrix assembled here from the parts of the case, scores through
the Python functions themselves.  Tile-form score functions are evaluated tile by tile at the call's block sizes
(128 x 128), as the reference's kernels hand them tiles (flex_attention_kernel.py:248-255), with sm_scale = 1."""
import math
import random
import types

import pytest
import torch

import custom_functors as cf
from helpers import assert_close
from oracle import mha_oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda"
N_CASES, N_LONG = 192, 32   # (the last N_LONG with 1400 to 2600 queries)
_CLOSURES = {"alibi_mod": cf.alibi_mod, "softcap_mod": cf.softcap_mod, "mixed_mod": cf.mixed_mod,
             "alibi_symmetric_mod": cf.alibi_symmetric_mod, "elementary_mod": cf.elementary_mod,
             "mixed_mod+prefix_lm": cf.mixed_mod}
_CLOSURE_MASKS = {"prefix_lm": cf.prefix_lm_mask, "checker": cf.checker_mask, "mixed_mod+prefix_lm": cf.prefix_lm_mask}
_TILE_FORMS = ("squared_tile", "tile_local_distance")


@pytest.fixture(scope="module")
def F():
    import flex_attention_tpu_amd as F
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return F


@pytest.fixture(scope="module")
def compiled():
    return cf.compiled()


def _draw(rng, closures, long):
    c = types.SimpleNamespace()
    c.dtype = torch.bfloat16 if rng.random() < 0.7 else torch.float32
    c.D = rng.choice([32, 64, 96, 128, 128, 128, 160, 256] if c.dtype == torch.bfloat16 else [32, 64, 64, 100, 128])
    c.B, c.Hkv, group = rng.choice([1, 2, 3]), rng.choice([1, 2]), rng.choice([1, 1, 2, 4])
    c.Hq = c.Hkv * group
    c.Sq = rng.choice([rng.randint(1, 127), rng.randint(128, 700), 128 * rng.randint(1, 5)])
    if long:   # (more work items than the persistent kernels have workgroups, tile lists beyond the unrolled length)
        c.Sq = rng.choice([rng.randint(1400, 2600), 128 * rng.randint(11, 20)])
    c.Sk = c.Sq if rng.random() < 0.7 else rng.choice([rng.randint(1, 700), 128 * rng.randint(1, 5)])
    # (float32 logits that a distance penalty takes to several hundred are spaced 6e-5 apart, and the probabilities
    #  inherit that: no float32 evaluation meets 1e-5 there, so the long float32 cases leave those penalties out)
    far = long and c.dtype == torch.float32
    closures = [x for x in closures if not (far and x.startswith("alibi"))]
    c.closure = rng.choice(closures) if c.Hq <= 4 and rng.random() < 0.4 else None   # (cf.SLOPES has four entries)
    c.mask = rng.choice(["none", "causal", "causal flag", "window", "causal window", "s2"])
    c.score = rng.choice(["none", "none", "softcap", "alibi tile" if far else "alibi", "alibi tile"])
    c.ids = rng.choice(["none", "none", "1d", "2d", "q/kv", "q/kv 2d"])
    c.ab = rng.choice(["none", "none", "11", "BH", "1H", "B1"])
    c.ab_dtype = rng.choice([torch.float32, torch.bfloat16])
    c.dab = c.ab != "none" and rng.random() < 0.5
    c.compiled_loop = rng.random() < 0.3
    c.scale = rng.choice([1.0, 1.0, 2.0, 0.5]) if c.dtype == torch.bfloat16 else rng.choice([1.0, 0.5])
    c.window, c.stride, c.cap = rng.randint(1, 300), rng.choice([16, 64, 100]), rng.choice([2.0, 10.0, 30.0])
    c.closure_causal, c.unsorted = rng.random() < 0.5, rng.random() < 0.6
    return c


def _segment_ids(c, rng, gen):
    """(segment_ids argument, ids of q [nb, Sq], ids of kv [nb, Sk]) or (None, None, None)."""
    if c.ids == "none" or (c.Sq != c.Sk and not c.ids.startswith("q/kv")):
        return None, None, None
    nb = c.B if c.ids.endswith("2d") else 1

    def documents(S):
        rows = []
        for _ in range(nb):
            lens, left = [], S
            while left > 0:
                lens.append(min(left, rng.randint(1, 300)))
                left -= lens[-1]
            rows.append(O.doc_ids_from_lengths(lens))
        return torch.stack(rows)

    def recurring(S):
        run = rng.choice([1, 8, 32])
        return torch.randint(0, 3, (nb, (S + run - 1) // run), generator=gen).repeat_interleave(run, dim=1)[:, :S]
    if c.ids in ("1d", "2d"):
        ids = documents(c.Sq)
        return (ids if c.ids == "2d" else ids[0]), ids, ids
    iq, ik = (recurring(c.Sq), recurring(c.Sk)) if c.unsorted else (documents(c.Sq), documents(c.Sk))
    return types.SimpleNamespace(q=iq if nb > 1 else iq[0], kv=ik if nb > 1 else ik[0]), iq, ik


def _build(c, rng, gen, compiled):
    """The package's closures and arguments of the case, the oracle's keywords, the dense keep matrix."""
    from flex_attention_tpu_amd import masks, scores
    qi, kj = torch.arange(c.Sq), torch.arange(c.Sk)
    keep = torch.ones(c.B, c.Sq, c.Sk, dtype=torch.bool)
    mf = bf = sfn = None
    okw, causal = {}, False
    if c.closure is not None:
        sfn, pair = compiled[c.closure]
        if pair is not None:
            mf, bf = pair
            keep &= _CLOSURE_MASKS[c.closure](qi, kj)[None]
        if c.closure in _CLOSURES:
            okw["score_mod"] = _CLOSURES[c.closure]
        if c.closure in _TILE_FORMS:
            fn = getattr(cf, c.closure)

            def tiled(qt, kt):
                return torch.cat([torch.cat([fn(qt[a:a + 128], kt[b:b + 128]) for b in range(0, kt.shape[0], 128)], dim=1)
                                  for a in range(0, qt.shape[0], 128)], dim=0)
            okw["score_fn"] = tiled
        causal = c.closure_causal
    else:
        if c.mask == "causal":
            mf, bf = masks.make_causal_mask_fns(128, 128)
        elif c.mask == "causal flag":
            causal = True
        elif c.mask == "window":
            mf, bf = masks.make_sliding_window_mask_fns(128, 128, c.window)
        elif c.mask == "causal window":
            mf, bf = masks.make_causal_sliding_window_mask_fns(128, 128, c.window)
        elif c.mask == "s2":
            mf, bf = masks.make_s2_mask_fns(128, 128, c.window, c.stride)
        if mf is not None:
            keep &= torch.as_tensor(mf(qi, kj)).bool()[None]
        if c.score == "softcap":
            sfn, okw["score_mod"] = scores.make_softcap_score_fn(c.cap), O.score_mod_softcap(c.cap)
        elif c.score == "alibi":
            sfn, okw["score_mod"] = scores.make_alibi_global_score_fn(c.Hq), O.score_mod_alibi_global(O.alibi_slopes(c.Hq))
        elif c.score == "alibi tile":   # (tile-local indices: the call's blocks are 128 x 128)
            sfn, okw["score_mod"] = scores.make_alibi_score_fn(0.5), O.score_mod_alibi_tile_local(0.5, 128, 128)
    if causal:
        keep &= (qi[:, None] >= kj[None, :])[None]
    sid, iq, ik = _segment_ids(c, rng, gen)
    if sid is not None:
        keep &= (iq[:, :, None] == ik[:, None, :]).expand(c.B, c.Sq, c.Sk)
    return mf, bf, sfn, okw, causal, sid, keep


def _case(index, compiled):
    """The index-th case whose every query keeps a key (others are drawn again: rows without a key have a test of
    their own, test_rows_that_keep_no_key)."""
    rng = random.Random(7919 * index + 13)
    gen = torch.Generator().manual_seed(index)
    while True:
        c = _draw(rng, list(compiled), long=index >= N_CASES - N_LONG)
        parts = _build(c, rng, gen, compiled)
        if bool(parts[-1].any(dim=-1).all()):
            return c, gen, parts


@pytest.mark.parametrize("index", range(N_CASES))
def test_random_case(F, compiled, index):
    c, gen, (mf, bf, sfn, okw, causal, sid, keep) = _case(index, compiled)
    dtype, tile_form = c.dtype, "score_fn" in okw
    print(f"case {index}: {str(dtype)[6:]} D={c.D} B={c.B} Hq={c.Hq} Hkv={c.Hkv} Sq={c.Sq} Sk={c.Sk} closure={c.closure} "
          f"mask={c.mask} window={c.window} stride={c.stride} score={c.score} ids={c.ids if sid is not None else 'none'} "
          f"causal={causal} ab={c.ab}/{str(c.ab_dtype)[6:]} dab={c.dab} compiled_loop={c.compiled_loop} scale={c.scale}", flush=True)
    sc = 1.0 if tile_form else c.scale / math.sqrt(c.D)
    q, k, v, do = O.make_inputs(c.B, c.Hq, c.Hkv, c.Sq, c.Sk, c.D, dtype=dtype, seed=1000 + index)
    if tile_form:   # (no sm_scale in front of a tile-form function: logits of order one through the inputs)
        q, k = (q.float() * 0.3).to(dtype), (k.float() * 0.3).to(dtype)
    ab = None
    if c.ab != "none":
        shape = {"11": (1, 1), "BH": (c.B, c.Hq), "1H": (1, c.Hq), "B1": (c.B, 1)}[c.ab]
        ab = torch.randn(*shape, c.Sq, c.Sk, generator=gen).to(c.ab_dtype)
    ab_dense = None if ab is None else ab.float().expand(c.B, c.Hq, c.Sq, c.Sk)
    okw = dict(okw, sm_scale=sc, mask=None if bool(keep.all()) else keep)
    ro, rl, rm = O.mha_reference(q, k, v, ab_dense, save_residuals=True, **okw)
    qg, kg, vg, dog = [x.to(DEV) for x in (q, k, v, do)]
    abg = None if ab is None else ab.to(DEV)
    o, l, m = F._flex_attention_impl(qg, kg, vg, abg, sid, True, causal, sc, 1, 128, 128, 128, False, bf, mf, sfn,
                                     compiled_loop=c.compiled_loop)
    assert o.shape == q.shape and l.shape == m.shape == (c.B, c.Hq, c.Sq)
    assert_close("o", o, ro, dtype)
    assert_close("lse", m + l.log(), rm + rl.log(), dtype, tensor_scale=dtype == torch.float32)   # (distance penalties reach 90)
    d = F.compute_delta(o, dog)
    kw = dict(block_b=1, block_q=128, block_k_major=128, block_k=128, sm_scale=sc, debug=False, score_fn=sfn, mask_fn=mf,
              block_mask_fn=bf, compiled_loop=c.compiled_loop, causal=causal)
    dq = F.flex_attention_bwd_dq(qg, kg, vg, abg, sid, l, m, o, dog, d, return_dab=c.dab, **kw)
    dq, dab = dq if c.dab else (dq, None)
    dk, dv, ds = F.flash_attention_bwd_dkv(kg, vg, qg, abg, sid, l, m, d, dog, block_q_major=128, return_ds=True, **kw)
    dk1, dv1 = F.flash_attention_bwd_dkv(kg, vg, qg, abg, sid, l, m, d, dog, block_q_major=128, **kw)
    assert torch.equal(dk, dk1) and torch.equal(dv, dv1), "dk, dv change when dS is exported"
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    same = O.mha_bwd_reference(q, k, v, o.float().cpu(), do, l.cpu(), m.cpu(), ab_dense, return_dab=c.dab, **okw)
    # (gradients summed over many keys, heads of a group and bias terms exceed 2.56 in places: the bound of the
    #  tensor's magnitude, see helpers.assert_close)
    for name, t, r in zip(("dq", "dk", "dv"), (dq, dk, dv), same):
        assert_close(name, t, r, dtype, tensor_scale=True)
    if c.dab:
        assert dab.shape == ab.shape and dab.dtype == ab.dtype
        rdab = same[3]
        summed = [i for i, n in enumerate(ab.shape[:2]) if n == 1 and (c.B, c.Hq)[i] != 1]
        if summed:
            rdab = rdab.sum(dim=summed, keepdim=True)
        assert_close("dab", dab, rdab, torch.bfloat16 if torch.bfloat16 in (dtype, c.ab_dtype) else dtype, tensor_scale=True)
    if ds is not None:
        dqx = F.flex_attention_bwd_dq(qg, kg, vg, abg, sid, l, m, o, dog, d, ds=ds, **kw)
        assert_close("dq from dS", dqx, same[0], dtype, tensor_scale=True)
    if index % 3 == 0:   # (the autograd wrapper chooses its kernels itself: the same bound, not the same bits)
        qa, ka, va = [x.clone().requires_grad_(True) for x in (qg, kg, vg)]
        oa = F.flex_attention(qa, ka, va, sfn, (mf, bf) if mf is not None else None, segment_ids=sid, causal=causal,
                              sm_scale=sc, ab=abg)
        assert_close("o (autograd)", oa, ro, dtype)
        ra = O.mha_bwd_reference(q, k, v, oa.detach().float().cpu(), do, l.cpu(), m.cpu(), ab_dense, **okw)
        for name, t, r in zip(("dq (autograd)", "dk (autograd)", "dv (autograd)"), torch.autograd.grad(oa, (qa, ka, va), dog), ra):
            assert_close(name, t, r, dtype, tensor_scale=True)
