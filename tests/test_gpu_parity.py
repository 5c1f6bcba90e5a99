"""GPU parity tests: the HIP kernels, called through the Python entry points (and therefore the
C ABI of libflexattn.so), against the CPU oracle on identical seeded inputs.

Tolerances (north star): block map bit-exact; bf16 max-abs <= 2e-2 and rel-L2 <= 1e-2 on
o, dq, dk, dv; fp32 <= 1e-5 for both (helpers.assert_close: the bf16 absolute bound is applied
element by element and widens to the spacing of bf16 values, 2^-7 |ref|, where that exceeds 2e-2).
The forward is compared with the oracle's forward; the backward kernels with the oracle's backward
from identical residuals (the reference's own method) and, in rel-L2, with the oracle's whole chain.
Full-size configurations are checked against the oracle on sampled q rows, on whole heads of the
dense launch and through size-independent invariants.

Cases that combine a score function with sm_scale != 1 (the position-bias and softcap cases here, configurations
4 and 5) are pinned to this build's definition, logits = score_mod(sm_scale <q, k>), which the oracle restates:
the reference does not agree with itself there (its forward ignores sm_scale next to a score function,
flex_attention_kernel.py:249-255, its backward kernels multiply the score function's result by it,
flex_attention_dq_bwd.py:340-345), and its drivers only ever pass sm_scale = 1 with score functions, where all
conventions coincide (those workloads: test_gpu_reference_drivers.py).
"""
import math
import os

import numpy as np
import pytest
import torch

from helpers import assert_close, oracle_kwargs, same_residual_grads
from oracle import mha_oracle as O

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
DEV = "cuda"


@pytest.fixture(scope="module")
def F():
    import flex_attention_tpu_amd as F
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return F


def _fwd(F, q, k, v, sc, mf, bf, score_fn, causal=False, blk=128):
    return F._flex_attention_impl(q, k, v, None, None, True, causal, sc, 1, blk, blk, blk, False, bf, mf, score_fn)


def _dq(F, q, k, v, l, m, o, do, d, sc, mf, bf, score_fn, causal=False, blk=128, ds=None, sid=None):
    return F.flex_attention_bwd_dq(q, k, v, None, sid, l, m, o, do, d, block_b=1, block_q=blk, block_k_major=blk,
                                   block_k=blk, sm_scale=sc, debug=False, score_fn=score_fn, mask_fn=mf,
                                   block_mask_fn=bf, causal=causal, ds=ds)


def _dkv(F, q, k, v, l, m, do, d, sc, mf, bf, score_fn, causal=False, blk=128, return_ds=False, sid=None):
    return F.flash_attention_bwd_dkv(k, v, q, None, sid, l, m, d, do, block_b=1, block_q=blk, block_q_major=blk,
                                     block_k_major=blk, block_k=blk, sm_scale=sc, causal=causal, debug=False,
                                     score_fn=score_fn, mask_fn=mf, block_mask_fn=bf, return_ds=return_ds)


def _exchanged_dq(F, q, k, v, l, m, o, do, d, sc, mf, bf, score_fn, dk, dv, expect, causal=False, sid=None):
    """The backward with dS handed from the dk/dv pass to the dq pass: dk, dv must be the bits of the pass
    without the export; returns that dq (None where the kernels of the call exchange nothing, which
    must be exactly where `expect` says so)."""
    dk2, dv2, ds = _dkv(F, q, k, v, l, m, do, d, sc, mf, bf, score_fn, causal=causal, return_ds=True, sid=sid)
    assert torch.equal(dk2, dk) and torch.equal(dv2, dv), "dk, dv change when dS is exported"
    assert (ds is not None) == expect, "dS exchange offered" if ds is not None else "no dS exchange offered"
    if ds is None:
        return None
    return _dq(F, q, k, v, l, m, o, do, d, sc, mf, bf, score_fn, causal=causal, ds=ds, sid=sid)


def _check_grads(got, chain_ref, q, k, v, do, o, l, m, dtype, okw, tag=""):
    """dq, dk, dv of the kernels against (1) the oracle's backward from the same residuals (o, l, m of
    the kernels' forward): the stated bound, element by element; (2) the oracle's backward from its own
    forward (the whole chain): rel-L2 asserted, max-abs reported (helpers.assert_close)."""
    same = same_residual_grads(q, k, v, do, o, l, m, **okw)
    for name, t, r, c in zip(("dq", "dk", "dv"), got, same, chain_ref):
        assert_close(tag + name, t, r, dtype)
        assert_close(tag + name + " chain", t, c, dtype, chain=True)


# ------------------------------------------------------------------------------------------------
# block-mask builder: bit-exact
# ------------------------------------------------------------------------------------------------
def _mask_cases(S, bq, bk):
    from flex_attention_tpu_amd import masks
    lens = O.make_segment_lengths(S, lo=max(8, S // 16), hi=max(16, S // 3), seed=4)
    return [
        ("none", masks.place_holder(bq, bk), {}),
        ("causal", masks.make_causal_mask_fns(bq, bk), dict(causal=True)),
        ("window", masks.make_sliding_window_mask_fns(bq, bk, S // 5 + 3), dict(window_size=S // 5 + 3)),
        ("causal_window", masks.make_causal_sliding_window_mask_fns(bq, bk, S // 7 + 1),
         dict(causal=True, window_size=S // 7 + 1)),
        ("jagged", masks.make_jagged_mask_fns(bq, bk, lens), dict(causal=True, segment_ids=O.doc_ids_from_lengths(lens))),
        ("s2", masks.make_s2_mask_fns(bq, bk, S // 9 + 2, 2 * bk), dict(window_size=S // 9 + 2, s2_stride=2 * bk)),
    ]


@pytest.mark.parametrize("S,bq,bk", [(1024, 128, 64), (1024, 64, 128), (2048, 128, 128), (768, 64, 64), (512, 32, 16)])
def test_block_mask_builder_bit_exact(F, S, bq, bk):
    from flex_attention_tpu_amd import block_mask
    for name, (mf, bf), kw in _mask_cases(S, bq, bk):
        bm = block_mask.create_block_mask((mf, bf), S, S, bq, bk, DEV)
        nq, nk = S // bq, S // bk
        state = bm.state.cpu()
        run = state != 0
        host = block_mask.host_block_map(bf, nq, nk)
        assert torch.equal(run, host), f"{name}: run-map differs from the block closure"
        keep = O.dense_mask(S, S, **kw) if kw else torch.ones(S, S, dtype=torch.bool)
        brute = O.block_map_bruteforce(keep, bq, bk)
        assert bool(((state == 2) <= (brute == 2)).all()), f"{name}: a tile marked full has masked elements"
        assert bool(((state == 0) <= (brute == 0)).all()), f"{name}: a skipped tile has kept elements"
        if name in ("none", "causal", "window", "jagged"):
            assert torch.equal(state, brute), f"{name}: state map differs from brute force"
        kv_cnt, kv_idx = bm.kv_cnt.cpu(), bm.kv_idx.cpu()
        q_cnt, q_idx = bm.q_cnt.cpu(), bm.q_idx.cpu()
        for qb in range(nq):
            assert kv_idx[qb, : kv_cnt[qb]].tolist() == torch.nonzero(run[qb]).flatten().tolist()
        for kb in range(nk):
            assert q_idx[kb, : q_cnt[kb]].tolist() == torch.nonzero(run[:, kb]).flatten().tolist()


def test_block_mask_builder_matches_config_fixtures(F):
    from flex_attention_tpu_amd import block_mask, configs
    g = np.load(os.path.join(GOLDEN, "block_maps.npz"))
    for name in ("cfg2", "cfg4", "cfg5"):
        cfg = configs.CONFIGS[name]
        n = int(g[name + "_n"])
        gold = torch.from_numpy(np.unpackbits(g[name], axis=1)[:, :n].astype(bool))
        bm = block_mask.create_block_mask(configs.mask_fns(cfg), cfg.S, cfg.S, 128, 128, DEV)
        run = bm.run_mask().cpu()
        if name == "cfg4":
            assert bool((run | ~gold).all()) and int(run.sum()) == 540
        else:
            assert torch.equal(run, gold), name


def test_ds_index_builder_bit_exact(F):
    """flexattn_build_ds_index: the blocks of the dS exchange buffer follow the kept tile pairs kv tile by kv tile
    and along each kv tile's q list; skipped pairs get -1 and take no room.  Against a host enumeration."""
    from flex_attention_tpu_amd import block_mask
    S = 2048
    for name, (mf, bf), _ in _mask_cases(S, 128, 128):
        bm = block_mask.create_block_mask((mf, bf), S, S, 128, 128, DEV)
        col, rank, pairs = bm.ds_index()
        run = bm.run_mask().cpu().numpy()
        nq, nk = run.shape
        want_col = np.concatenate([[0], np.cumsum(run.sum(axis=0))]).astype(np.int32)
        want_rank = np.full((nq, nk), -1, np.int32)
        for kb in range(nk):
            qs = np.nonzero(run[:, kb])[0]
            want_rank[qs, kb] = want_col[kb] + np.arange(len(qs))
        assert pairs == int(run.sum()), name
        assert np.array_equal(col.cpu().numpy(), want_col), name
        assert np.array_equal(rank.cpu().numpy(), want_rank), name


def test_ds_buffer_holds_the_kept_pairs_only(F):
    """The exchange buffer of a masked call is as large as the mask leaves it: 32 KB per query head and kept pair
    of 128 x 128 tiles (a causal window of 300 over 4096 tokens keeps 122 of 1024 pairs)."""
    from flex_attention_tpu_amd import masks
    S, W = 4096, 300
    sc = 1 / math.sqrt(128)
    g = torch.Generator().manual_seed(3)
    q, k, v, do = (torch.randn(1, 2, S, 128, generator=g).to(torch.bfloat16).to(DEV) for _ in range(4))
    mf, bf = masks.make_causal_sliding_window_mask_fns(128, 128, W)
    o, l, m = _fwd(F, q, k, v, sc, mf, bf, None)
    d = F.compute_delta(o, do)
    dk, dv, ds = _dkv(F, q, k, v, l, m, do, d, sc, mf, bf, None, return_ds=True)
    kept = sum(1 for qb in range(32) for kb in range(32) if kb <= qb and 128 * qb - (128 * kb + 127) < W)
    assert ds is not None and ds.buf.numel() == 2 * kept * 128 * 128 * 2 and kept == 122
    # a device without room for the buffer: the pass declines the exchange, the dq pass then recomputes
    from flex_attention_tpu_amd import flex_attention_dq_bwd as dqmod
    share, dqmod.DS_MEMORY_SHARE = dqmod.DS_MEMORY_SHARE, 0.0
    try:
        dk2, dv2, ds2 = _dkv(F, q, k, v, l, m, do, d, sc, mf, bf, None, return_ds=True)
    finally:
        dqmod.DS_MEMORY_SHARE = share
    assert ds2 is None and torch.equal(dk2, dk) and torch.equal(dv2, dv)


# ------------------------------------------------------------------------------------------------
# small-shape parity matrix (oracle runs whole tensors in float64)
# ------------------------------------------------------------------------------------------------
def _small_cases():
    from flex_attention_tpu_amd import masks, scores
    lens = [300, 212, 512]
    sc = 1 / math.sqrt(128)
    c = []
    c.append(("plain", (1, 2, 2, 512, 512), None, None, {}, sc))
    c.append(("causal", (2, 2, 2, 512, 512), masks.make_causal_mask_fns(128, 128), None, dict(causal=True), sc))
    c.append(("window", (1, 2, 2, 1024, 1024), masks.make_sliding_window_mask_fns(128, 128, 200), None, dict(window_size=200), sc))
    c.append(("causal_window", (1, 2, 2, 1024, 1024), masks.make_causal_sliding_window_mask_fns(128, 128, 257), None,
              dict(causal=True, window_size=257), sc))
    c.append(("jagged", (1, 2, 2, 1024, 1024), masks.make_jagged_mask_fns(128, 128, lens), None,
              dict(causal=True, segment_ids=O.doc_ids_from_lengths(lens)), sc))
    c.append(("s2", (1, 2, 2, 1024, 1024), masks.make_s2_mask_fns(128, 128, 128, 64), None,
              dict(mask=O.dense_mask(1024, 1024, window_size=128, s2_stride=64)), sc))
    c.append(("softcap", (1, 2, 2, 512, 512), masks.make_causal_mask_fns(128, 128), scores.make_softcap_score_fn(5.0),
              dict(causal=True, score_mod=O.score_mod_softcap(5.0)), sc))
    c.append(("alibi_global", (1, 4, 4, 512, 512), masks.make_causal_mask_fns(128, 128), scores.make_alibi_global_score_fn(4),
              dict(causal=True, score_mod=O.score_mod_alibi_global(O.alibi_slopes(4))), sc))
    c.append(("alibi_tile", (1, 2, 2, 512, 512), None, scores.make_alibi_score_fn(0.5),
              dict(score_mod=O.score_mod_alibi_tile_local(0.5, 128, 128)), sc))
    c.append(("gqa", (1, 8, 2, 512, 512), masks.make_causal_mask_fns(128, 128), None, dict(causal=True), sc))
    c.append(("cross", (1, 2, 2, 256, 768), None, None, {}, sc))
    return c


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "fp32"])
@pytest.mark.parametrize("case", _small_cases(), ids=lambda c: c[0])
def test_small_shapes_all_passes(F, case, dtype):
    name, (B, Hq, Hkv, Sq, Sk), mask_pair, score_fn, okw, sc = case
    D = 128
    q, k, v, do = O.make_inputs(B, Hq, Hkv, Sq, Sk, D, dtype=dtype, seed=17)
    ro, rl, rm = O.mha_reference(q, k, v, sm_scale=sc, save_residuals=True, **okw)
    rdq, rdk, rdv = O.mha_bwd_reference(q, k, v, ro, do, rl, rm, sm_scale=sc, **okw)
    qc, kc, vc, doc = q, k, v, do
    q, k, v, do = [x.to(DEV) for x in (q, k, v, do)]
    mf, bf = mask_pair if mask_pair else (None, None)
    o, l, m = _fwd(F, q, k, v, sc, mf, bf, score_fn)
    assert_close("o", o, ro, dtype)
    assert_close("lse", m + l.log(), rm + rl.log(), dtype)
    d = F.compute_delta(o, do)
    assert_close("delta", d, O.delta(o.cpu(), do.cpu()), torch.float32)
    dq = _dq(F, q, k, v, l, m, o, do, d, sc, mf, bf, score_fn)
    dk, dv = _dkv(F, q, k, v, l, m, do, d, sc, mf, bf, score_fn)
    _check_grads((dq, dk, dv), (rdq, rdk, rdv), qc, kc, vc, doc, o, l, m, dtype, dict(sm_scale=sc, **okw))
    # d=None: the dq pass takes delta itself (the bf16 stream kernels while they fetch an item's rows, the others
    # through the delta kernel): the same delta and the same dq, bit for bit
    dq_f, d_f = F.flex_attention_bwd_dq(q, k, v, None, None, l, m, o, do, None, block_b=1, block_q=128, block_k_major=128,
                                        block_k=128, sm_scale=sc, debug=False, score_fn=score_fn, mask_fn=mf,
                                        block_mask_fn=bf, return_delta=True)
    assert torch.equal(d_f, d) and torch.equal(dq_f, dq), "delta taken by the dq pass differs from the delta kernel's"
    # dS exchange: the bf16 stream kernels of plain and softcap scores offer it, and the dk/dv kernel with a compiled
    # main loop (the tile-local position bias); the global position bias's dk/dv stream does not
    dqx = _exchanged_dq(F, q, k, v, l, m, o, do, d, sc, mf, bf, score_fn, dk, dv,
                        expect=dtype == torch.bfloat16 and name != "alibi_global")
    if dqx is not None:
        _check_grads((dqx, dk, dv), (rdq, rdk, rdv), qc, kc, vc, doc, o, l, m, dtype, dict(sm_scale=sc, **okw), tag="exchange ")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "fp32"])
def test_whole_backward_from_one_call(F, dtype):
    """flex_attention_bwd (flexattn_bwd: delta, dq and dk/dv from one call) gives the bits of the three separate
    calls: a small problem (twice in a row), a larger one, and a ragged one (which falls back to the separate
    calls)."""
    from flex_attention_tpu_amd import masks, scores
    sc = 1 / math.sqrt(128)
    for (B, Hq, Hkv, S), repeat in (((1, 4, 2, 512), 2), ((2, 8, 8, 2048), 1), ((1, 2, 2, 300), 1)):
        q, k, v, do = (x.to(DEV) for x in O.make_inputs(B, Hq, Hkv, S, S, 128, dtype=dtype, seed=97))
        mf, bf = masks.make_causal_mask_fns(128, 128)
        sfn = scores.make_softcap_score_fn(20.0)
        o, l, m = _fwd(F, q, k, v, sc, mf, bf, sfn)
        d = F.compute_delta(o, do)
        dq = _dq(F, q, k, v, l, m, o, do, d, sc, mf, bf, sfn)
        dk, dv = _dkv(F, q, k, v, l, m, do, d, sc, mf, bf, sfn)
        for _ in range(repeat):
            dq2, dk2, dv2 = F.flex_attention_bwd(q, k, v, None, None, l, m, o, do, block_q=128, block_k=128, sm_scale=sc,
                                                 score_fn=sfn, mask_fn=mf, block_mask_fn=bf)
            assert torch.equal(dq2, dq) and torch.equal(dk2, dk) and torch.equal(dv2, dv), (B, Hq, S)


def test_causal_flag_and_segment_ids_arguments(F):
    """`causal=True` and `segment_ids=` are honoured by all three entry points."""
    sc = 0.1
    lens = [100, 156]
    sid = O.doc_ids_from_lengths(lens)
    q, k, v, do = O.make_inputs(1, 2, 2, 256, 256, 128, dtype=torch.bfloat16, seed=5)
    ro, rl, rm = O.mha_reference(q, k, v, sm_scale=sc, save_residuals=True, causal=True, segment_ids=sid)
    rdq, rdk, rdv = O.mha_bwd_reference(q, k, v, ro, do, rl, rm, sm_scale=sc, causal=True, segment_ids=sid)
    qc, kc, vc, doc = q, k, v, do
    q, k, v, do = [x.to(DEV) for x in (q, k, v, do)]
    o, l, m = F._flex_attention_impl(q, k, v, None, sid, True, True, sc, 1, 128, 128, 128, False, None, None, None)
    assert_close("o", o, ro, torch.bfloat16)
    d = F.compute_delta(o, do)
    dq = F.flex_attention_bwd_dq(q, k, v, None, sid, l, m, o, do, d, block_b=1, block_q=128, block_k_major=128,
                                 block_k=128, sm_scale=sc, debug=False, causal=True)
    dk, dv = F.flash_attention_bwd_dkv(k, v, q, None, sid, l, m, d, do, block_b=1, block_q=128, block_q_major=128,
                                       block_k_major=128, block_k=128, sm_scale=sc, causal=True, debug=False)
    _check_grads((dq, dk, dv), (rdq, rdk, rdv), qc, kc, vc, doc, o, l, m, torch.bfloat16,
                 dict(sm_scale=sc, causal=True, segment_ids=sid))
    # save_residuals=False returns the output only
    o2 = F._flex_attention_impl(q, k, v, None, sid, False, True, sc, 1, 128, 128, 128, False, None, None, None)
    assert torch.equal(o2, o)


def _all_passes_with(F, q, k, v, do, ab, sid, sc, mask_pair, score_fn, causal):
    mf, bf = mask_pair if mask_pair else (None, None)
    o, l, m = F._flex_attention_impl(q, k, v, ab, sid, True, causal, sc, 1, 128, 128, 128, False, bf, mf, score_fn)
    d = F.compute_delta(o, do)
    dq = F.flex_attention_bwd_dq(q, k, v, ab, sid, l, m, o, do, d, block_b=1, block_q=128, block_k_major=128,
                                 block_k=128, sm_scale=sc, debug=False, score_fn=score_fn, mask_fn=mf, block_mask_fn=bf,
                                 causal=causal)
    dk, dv = F.flash_attention_bwd_dkv(k, v, q, ab, sid, l, m, d, do, block_b=1, block_q=128, block_q_major=128,
                                       block_k_major=128, block_k=128, sm_scale=sc, causal=causal, debug=False,
                                       score_fn=score_fn, mask_fn=mf, block_mask_fn=bf)
    return o, l, m, dq, dk, dv


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "fp32"])
@pytest.mark.parametrize("case", ["plain", "softcap_causal_gqa", "ragged_bf16_bias"])
def test_additive_bias(F, case, dtype):
    """`ab` is added to the logits behind the score function and in front of the mask (mha_reference.py:50-51,
    flex_attention_kernel.py:262-266, flash_attention_dkv_bwd.py:261-263) in all three passes: full [B, H, Sq, Sk],
    broadcast over heads and batch, bfloat16 bias, ragged lengths."""
    from flex_attention_tpu_amd import masks, scores
    sc = 1 / math.sqrt(128)
    g = torch.Generator().manual_seed(3)
    if case == "plain":
        B, Hq, Hkv, Sq, Sk = 2, 2, 2, 256, 384
        ab = torch.randn(B, Hq, Sq, Sk, generator=g) * 2
        mask_pair, score_fn, okw, causal = None, None, {}, False
    elif case == "softcap_causal_gqa":
        B, Hq, Hkv, Sq, Sk = 2, 4, 2, 512, 512
        ab = torch.randn(B, 1, Sq, Sk, generator=g)            # one plane per batch entry, shared by the heads
        mask_pair, score_fn = masks.make_causal_mask_fns(128, 128), scores.make_softcap_score_fn(5.0)
        okw, causal = dict(causal=True, score_mod=O.score_mod_softcap(5.0)), False
    else:
        B, Hq, Hkv, Sq, Sk = 1, 2, 2, 200, 333
        ab = (torch.randn(1, 1, Sq, Sk, generator=g) * 3).to(torch.bfloat16)
        mask_pair, score_fn, okw, causal = None, None, dict(causal=True), True
    q, k, v, do = O.make_inputs(B, Hq, Hkv, Sq, Sk, 128, dtype=dtype, seed=61)
    ab_full = ab.float().expand(B, Hq, Sq, Sk)
    ro, rl, rm = O.mha_reference(q, k, v, ab_full, sm_scale=sc, save_residuals=True, **okw)
    rdq, rdk, rdv = O.mha_bwd_reference(q, k, v, ro, do, rl, rm, ab_full, sm_scale=sc, **okw)
    qg, kg, vg, dog = [x.to(DEV) for x in (q, k, v, do)]
    o, l, m, dq, dk, dv = _all_passes_with(F, qg, kg, vg, dog, ab.to(DEV), None, sc, mask_pair, score_fn, causal)
    assert_close("o", o, ro, dtype)
    assert_close("lse", m + l.log(), rm + rl.log(), dtype)
    tol = dict(sm_scale=sc, **okw)
    ma = O.mha_bwd_reference(q, k, v, o.float().cpu(), do, l.cpu(), m.cpu(), ab_full, return_dab=True, **tol)
    for name, t, r, chain in (("dq", dq, ma[0], rdq), ("dk", dk, ma[1], rdk), ("dv", dv, ma[2], rdv)):
        assert_close(name, t, r, dtype)
        assert_close(name + " chain", t, chain, dtype, chain=True)
    # the gradient of the bias (an output of the dq pass), in the bias's own shape and dtype: summed over the
    # dimensions it broadcasts
    mf_, bf_ = mask_pair if mask_pair else (None, None)
    d = F.compute_delta(o, dog)
    dq2, dab = F.flex_attention_bwd_dq(qg, kg, vg, ab.to(DEV), None, l, m, o, dog, d, block_b=1, block_q=128,
                                       block_k_major=128, block_k=128, sm_scale=sc, debug=False, score_fn=score_fn,
                                       mask_fn=mf_, block_mask_fn=bf_, causal=causal, return_dab=True)
    rdab = ma[3]
    for dim in (0, 1):
        if ab.shape[dim] == 1:
            rdab = rdab.sum(dim, keepdim=True)
    assert dab.shape == ab.shape and dab.dtype == ab.dtype
    assert_close("dq with dab", dq2, ma[0], dtype)
    if dtype == torch.bfloat16 or ab.dtype == torch.bfloat16:
        assert_close("dab", dab, rdab, torch.bfloat16)
    else:
        # float32: 1e-5 relative to the value where that exceeds 1 (dab is P (dP - delta), not normalised like the
        # other gradients: entries reach 8 here, where float32 round-off alone is 1e-6 per operation)
        err = (dab.cpu().double() - rdab).abs()
        assert O.rel_l2(dab, rdab) <= 1e-5 and bool((err <= 1e-5 * rdab.abs().clamp(min=1.0)).all()), float(err.max())
    assert float(rdab.abs().max()) > 1e-3
    # ... and through the differentiable op
    abg = ab.to(DEV).requires_grad_(True)
    qa = qg.clone().requires_grad_(True)
    og = F.flex_attention(qa, kg, vg, score_fn, mask_pair, causal=causal, sm_scale=sc, ab=abg)
    gq, gab = torch.autograd.grad(og, (qa, abg), dog)
    assert torch.equal(gab, dab) and gq.shape == q.shape
    # without the bias the result differs (the argument is not ignored)
    o0 = F._flex_attention_impl(qg, kg, vg, None, None, False, causal, sc, 1, 128, 128, 128, False,
                                mask_pair[1] if mask_pair else None, mask_pair[0] if mask_pair else None, score_fn)
    assert float((o0.float() - o.float()).abs().max()) > 0.05


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "fp32"])
def test_segment_ids_per_batch_entry(F, dtype):
    """Segment ids of shape [B, S] whose rows differ (mha_reference.py:65-73 takes them): every batch entry is
    masked by its own documents."""
    sc = 1 / math.sqrt(128)
    B, S = 3, 512
    sid = torch.stack([O.doc_ids_from_lengths(l) for l in ([100, 412], [256, 256], [512])])
    q, k, v, do = O.make_inputs(B, 4, 2, S, S, 128, dtype=dtype, seed=67)
    okw = dict(sm_scale=sc, causal=True, segment_ids=sid)
    ro, rl, rm = O.mha_reference(q, k, v, save_residuals=True, **okw)
    qg, kg, vg, dog = [x.to(DEV) for x in (q, k, v, do)]
    o, l, m, dq, dk, dv = _all_passes_with(F, qg, kg, vg, dog, None, sid, sc, None, None, True)
    assert o.shape == q.shape and l.shape == (B, 4, S) and dk.shape == k.shape
    assert_close("o", o, ro, dtype)
    assert_close("lse", m + l.log(), rm + rl.log(), dtype)
    ma = O.mha_bwd_reference(q, k, v, o.float().cpu(), do, l.cpu(), m.cpu(), **okw)
    for name, t, r in (("dq", dq, ma[0]), ("dk", dk, ma[1]), ("dv", dv, ma[2])):
        assert_close(name, t, r, dtype)
    # (the dS exchange works from the union map as well)
    d = F.compute_delta(o, dog)
    dqx = _exchanged_dq(F, qg, kg, vg, l, m, o, dog, d, sc, None, None, None, dk, dv, expect=dtype == torch.bfloat16,
                        causal=True, sid=sid)
    if dqx is not None:
        assert_close("exchange dq", dqx, ma[0], dtype)


@pytest.mark.parametrize("ids_kind", ["sorted", "one_entry_unsorted", "q_and_kv_differ"])
def test_segment_ids_per_batch_entry_on_the_persistent_schedule(F, ids_kind):
    """Rows of ids that differ between the batch entries at a size where the stream kernels run their persistent
    longest-first schedule (B=8, 16 q heads on 8 kv heads, S=1024: 512 forward items): one launch per pass, every
    entry masked by its own row (the kernels step through the id arrays with a batch stride), the block map the
    union over the entries.  Entry 0 is one document, entry 1 many short ones (most tiles it visits keep nothing
    of it), entry 2 documents that end inside tiles, entry 3 the first again, entries 4-7 the same in another order.  `one_entry_unsorted`: ids that
    recur, so the kernels compare staged ids instead of intervals; `q_and_kv_differ`: an object with .q / .kv.
    Against the oracle, the block map against the union of the entries' brute-force maps, and every entry against
    the same entry launched alone with its own row of ids and its own map: bit for bit (the tiles the union adds
    to an entry's lists keep nothing of it and add exact zeros)."""
    import types
    from flex_attention_tpu_amd import _common, block_mask
    sc = 1 / math.sqrt(128)
    B, Hq, Hkv, S = 8, 16, 8, 1024
    rows = [O.doc_ids_from_lengths(x) for x in ([1024], [60] * 17 + [4], [300, 212, 500, 12], [1024])]
    if ids_kind == "one_entry_unsorted":
        rows[2] = torch.arange(S) // 96 % 3            # ids 0, 1, 2, 0, 1, 2, ... in runs of 96
    rows = rows + [rows[2], rows[0], rows[1], rows[2]]
    sid = torch.stack([r.to(torch.int32) for r in rows])
    sid_arg = sid
    causal = ids_kind != "q_and_kv_differ"
    if not causal:   # (no causal term: the documents of the kv side begin elsewhere, every q id occurs among them;
        # one q head per kv head: without the causal term a key's gradient sums several times the terms)
        Hkv = Hq
        sid_kv = sid.clone()
        sid_kv[1] = sid_kv[6] = O.doc_ids_from_lengths([30] * 17 + [514])
        sid_kv[2] = sid_kv[4] = sid_kv[7] = O.doc_ids_from_lengths([500, 12, 212, 300])
        sid_arg = types.SimpleNamespace(q=sid, kv=sid_kv)
    q, k, v, do = O.make_inputs(B, Hq, Hkv, S, S, 128, dtype=torch.bfloat16, seed=139)
    if not causal:
        keep = sid[:, :, None] == sid_kv[:, None, :]
        okw = dict(sm_scale=sc, mask=keep)
    else:
        keep = (sid[:, :, None] == sid[:, None, :]) & (torch.arange(S)[:, None] >= torch.arange(S)[None, :])
        okw = dict(sm_scale=sc, causal=True, segment_ids=sid)
    ro, rl, rm = O.mha_reference(q, k, v, save_residuals=True, compute_dtype=torch.float32, **okw)
    qg, kg, vg, dog = [x.to(DEV) for x in (q, k, v, do)]
    o, l, m, dq, dk, dv = _all_passes_with(F, qg, kg, vg, dog, None, sid_arg, sc, None, None, causal)
    rows_kept = keep.any(-1)                              # (a query without a key has no defined output)
    rk = rows_kept[:, None, :, None]
    assert_close("o", torch.where(rk.to(DEV), o, torch.zeros_like(o)), torch.where(rk, ro, torch.zeros_like(ro)), torch.bfloat16)
    ma = O.mha_bwd_reference(q, k, v, o.float().cpu(), do, l.cpu(), m.cpu(), compute_dtype=torch.float32, **okw)
    for name, t, r in (("dq", dq, ma[0]), ("dk", dk, ma[1]), ("dv", dv, ma[2])):
        assert_close(name, t, r, torch.bfloat16)
    # the map: the union of the entries' maps
    spec = _common.resolve_mask(None, None, causal, sid_arg, S, S)
    bm = block_mask.build_block_map(spec, S, S, 128, 64, DEV)
    brute = torch.stack([O.block_map_bruteforce(keep[b], 128, 64) for b in range(B)])
    union = torch.where((brute == 0).all(0), 0, torch.where((brute == 2).all(0), 2, 1))
    st = bm.state.cpu()
    if ids_kind == "sorted":
        assert torch.equal(st.to(union.dtype), union)
    else:   # (ids that recur: the builder may keep a tile that holds no pair, never the other way round)
        assert bool(((st == 0) <= (union == 0)).all()) and bool(((st == 2) <= (union == 2)).all())
    # every entry alone (its own row of ids, its own map)
    for b in range(B):
        one = sid[b] if causal else types.SimpleNamespace(q=sid[b], kv=sid_kv[b])
        part = _all_passes_with(F, *[x[b:b + 1].contiguous() for x in (qg, kg, vg, dog)], None, one, sc, None, None, causal)
        for name, t, r in zip(("o", "l", "m", "dq", "dk", "dv"), part, (o, l, m, dq, dk, dv)):
            assert torch.equal(t[0], r[b]), f"{name} of entry {b} alone: {int((t[0] != r[b]).sum())} elements differ"


@pytest.mark.parametrize("D,dtype", [(64, torch.bfloat16), (96, torch.bfloat16), (32, torch.float32), (80, torch.float32)],
                         ids=["bf16-64", "bf16-96", "fp32-32", "fp32-80"])
def test_small_head_dimensions(F, D, dtype):
    """Head dimensions below the kernels' own (bf16 128, fp32 64 / 128) run zero-padded: all passes against the
    oracle at the caller's head dimension, causal, grouped kv heads."""
    from flex_attention_tpu_amd import masks
    sc = 1 / math.sqrt(D)
    q, k, v, do = O.make_inputs(1, 4, 2, 384, 384, D, dtype=dtype, seed=71)
    okw = dict(sm_scale=sc, causal=True)
    ro, rl, rm = O.mha_reference(q, k, v, save_residuals=True, **okw)
    qg, kg, vg, dog = [x.to(DEV) for x in (q, k, v, do)]
    o, l, m, dq, dk, dv = _all_passes_with(F, qg, kg, vg, dog, None, None, sc, masks.make_causal_mask_fns(128, 128), None, False)
    assert o.shape == q.shape and dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    assert_close("o", o, ro, dtype)
    assert_close("lse", m + l.log(), rm + rl.log(), dtype)
    ma = O.mha_bwd_reference(q, k, v, o.float().cpu(), do, l.cpu(), m.cpu(), **okw)
    for name, t, r in (("dq", dq, ma[0]), ("dk", dk, ma[1]), ("dv", dv, ma[2])):
        assert_close(name, t, r, dtype)


@pytest.mark.parametrize("case", _small_cases(), ids=lambda c: c[0])
def test_head_dimension_256(F, case):
    """bf16 at head dimension 256 (the reference takes any multiple of 128, flex_attention_kernel.py:302-306): rows
    of two 128-column panels through the kernels with a compiled main loop, every mask and score of the small
    matrix, all passes against the oracle.  These kernels exchange no dS."""
    name, (B, Hq, Hkv, Sq, Sk), mask_pair, score_fn, okw, _ = case
    D, dtype = 256, torch.bfloat16
    sc = 1 / math.sqrt(D)
    q, k, v, do = O.make_inputs(B, Hq, Hkv, Sq, Sk, D, dtype=dtype, seed=83)
    ro, rl, rm = O.mha_reference(q, k, v, sm_scale=sc, save_residuals=True, **okw)
    rdq, rdk, rdv = O.mha_bwd_reference(q, k, v, ro, do, rl, rm, sm_scale=sc, **okw)
    qc, kc, vc, doc = q, k, v, do
    q, k, v, do = [x.to(DEV) for x in (q, k, v, do)]
    mf, bf = mask_pair if mask_pair else (None, None)
    o, l, m = _fwd(F, q, k, v, sc, mf, bf, score_fn)
    assert o.shape == q.shape
    assert_close("o", o, ro, dtype)
    assert_close("lse", m + l.log(), rm + rl.log(), dtype)
    d = F.compute_delta(o, do)
    assert_close("delta", d, O.delta(o.cpu(), do.cpu()), torch.float32)
    dq = _dq(F, q, k, v, l, m, o, do, d, sc, mf, bf, score_fn)
    dk, dv = _dkv(F, q, k, v, l, m, do, d, sc, mf, bf, score_fn)
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    _check_grads((dq, dk, dv), (rdq, rdk, rdv), qc, kc, vc, doc, o, l, m, dtype, dict(sm_scale=sc, **okw))
    assert _exchanged_dq(F, q, k, v, l, m, o, do, d, sc, mf, bf, score_fn, dk, dv, expect=False) is None


def test_head_dimensions_between_128_and_256(F):
    """A bf16 head dimension of 192 runs zero-padded to 256; with an additive bias and its gradient, grouped kv
    heads, a ragged length and per-entry segment ids (the host-side paths around the kernels at the wider rows)."""
    D, dtype = 192, torch.bfloat16
    sc = 1 / math.sqrt(D)
    B, Hq, Hkv, S = 2, 4, 2, 300
    q, k, v, do = O.make_inputs(B, Hq, Hkv, S, S, D, dtype=dtype, seed=89)
    g = torch.Generator().manual_seed(97)
    ab = torch.randn(1, Hq, S, S, generator=g)
    sid = torch.stack([O.doc_ids_from_lengths(x) for x in ([100, 200], [300])])
    okw = dict(sm_scale=sc, causal=True, segment_ids=sid)
    ab_full = ab.expand(B, Hq, S, S)
    ro, rl, rm = O.mha_reference(q, k, v, ab_full, save_residuals=True, **okw)
    qg, kg, vg, dog, abg = [x.to(DEV) for x in (q, k, v, do, ab)]
    o, l, m, dq, dk, dv = _all_passes_with(F, qg, kg, vg, dog, abg, sid, sc, None, None, True)
    assert o.shape == q.shape and dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    assert_close("o", o, ro, dtype)
    assert_close("lse", m + l.log(), rm + rl.log(), dtype)
    ma = O.mha_bwd_reference(q, k, v, o.float().cpu(), do, l.cpu(), m.cpu(), ab_full, return_dab=True, **okw)
    for name, t, r in (("dq", dq, ma[0]), ("dk", dk, ma[1]), ("dv", dv, ma[2])):
        assert_close(name, t, r, dtype)
    dq2, dab = F.flex_attention_bwd_dq(qg, kg, vg, abg, sid, l, m, o, dog, F.compute_delta(o, dog), block_b=1, block_q=128,
                                       block_k_major=128, block_k=128, sm_scale=sc, debug=False, causal=True, return_dab=True)
    assert dab.shape == ab.shape and torch.equal(dq2, dq)
    assert_close("dab", dab, ma[3].sum(0, keepdim=True), dtype)   # (summed over the batch entries the bias is shared by)


@pytest.mark.parametrize("case", ["causal_gqa", "softcap_documents"])
def test_head_dimension_256_at_4096_tokens(F, case):
    """Head dimension 256 at the sequence length of the benchmark configurations (B=2, 8 q heads on 2 kv heads,
    S=4096): 64 kv tiles in a row's list, 32 q tiles times 4 heads in a column's.  Sampled rows of two whole kv
    groups against the oracle."""
    from flex_attention_tpu_amd import masks, scores
    D, S = 256, 4096
    sc = 1 / math.sqrt(D)
    q, k, v, do = O.make_inputs(2, 8, 2, S, S, D, dtype=torch.bfloat16, seed=137)
    if case == "causal_gqa":
        (mf, bf), sfn, okw = masks.make_causal_mask_fns(128, 128), None, dict(causal=True)
    else:
        lens = [1000, 24, 2000, 1072]
        (mf, bf), sfn = masks.make_jagged_mask_fns(128, 128, lens), scores.make_softcap_score_fn(30.0)
        okw = dict(causal=True, segment_ids=O.doc_ids_from_lengths(lens), score_mod=O.score_mod_softcap(30.0))
    heads = [(0, h) for h in range(4)] + [(1, h) for h in range(4, 8)]
    _sampled_oracle_check(F, q, k, v, do, sc, mf, bf, sfn, okw, 96, heads)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "fp32"])
def test_compiled_loop_kernels_on_request(F, dtype):
    """bf16 calls run the generated-stream kernels wherever one exists (covered by every other test
    here); `compiled_loop=True` (FLEXATTN_FLAG_COMPILED_LOOP) routes a call to the kernels with a
    compiled main loop, which must agree with the oracle as well, including rows whose tiles are
    partly or entirely masked, and the global ALiBi bias with several q heads per kv head.  For
    float32 the flag selects the FMA kernels instead of the ones on the fp32 matrix cores."""
    from flex_attention_tpu_amd import masks, scores
    cases = [c for c in _small_cases() if c[3] is None or dtype == torch.float32]
    cases.append(("alibi_gqa", (1, 4, 2, 512, 512), masks.make_causal_mask_fns(128, 128), scores.make_alibi_global_score_fn(4),
                  dict(causal=True, score_mod=O.score_mod_alibi_global(O.alibi_slopes(4))), 1 / math.sqrt(128)))
    for name, shape, mask_pair, score_fn, okw, sc in cases:
        B, Hq, Hkv, Sq, Sk = shape
        q, k, v, do = O.make_inputs(B, Hq, Hkv, Sq, Sk, 128, dtype=dtype, seed=23)
        ro, rl, rm = O.mha_reference(q, k, v, sm_scale=sc, save_residuals=True, **okw)
        rdq, rdk, rdv = O.mha_bwd_reference(q, k, v, ro, do, rl, rm, sm_scale=sc, **okw)
        qc, kc, vc, doc = q, k, v, do
        q, k, v, do = [x.to(DEV) for x in (q, k, v, do)]
        mf, bf = mask_pair if mask_pair else (None, None)
        o, l, m = F._flex_attention_impl(q, k, v, None, None, True, False, sc, 1, 128, 128, 128, False, bf, mf, score_fn,
                                         compiled_loop=True)
        assert_close(name + " o", o, ro, dtype)
        assert_close(name + " lse", m + l.log(), rm + rl.log(), dtype)
        d = F.compute_delta(o, do)
        dq = F.flex_attention_bwd_dq(q, k, v, None, None, l, m, o, do, d, block_b=1, block_q=128, block_k_major=128,
                                     block_k=128, sm_scale=sc, debug=False, score_fn=score_fn, mask_fn=mf,
                                     block_mask_fn=bf, compiled_loop=True)
        dk, dv = F.flash_attention_bwd_dkv(k, v, q, None, None, l, m, d, do, block_b=1, block_q=128, block_q_major=128,
                                           block_k_major=128, block_k=128, sm_scale=sc, causal=False, debug=False,
                                           score_fn=score_fn, mask_fn=mf, block_mask_fn=bf, compiled_loop=True)
        _check_grads((dq, dk, dv), (rdq, rdk, rdv), qc, kc, vc, doc, o, l, m, dtype, dict(sm_scale=sc, **okw), name + " ")
        # the default (generated-stream) kernels on the same inputs: GQA with the bias takes the
        # stream forward and dq and the compiled dk/dv
        if name == "alibi_gqa":
            o2, l2, m2 = _fwd(F, q, k, v, sc, mf, bf, score_fn)
            assert_close(name + " o", o2, ro, dtype)
            d2 = F.compute_delta(o2, do)
            dq2 = _dq(F, q, k, v, l2, m2, o2, do, d2, sc, mf, bf, score_fn)
            dk2, dv2 = _dkv(F, q, k, v, l2, m2, do, d2, sc, mf, bf, score_fn)
            _check_grads((dq2, dk2, dv2), (rdq, rdk, rdv), qc, kc, vc, doc, o2, l2, m2, dtype,
                         dict(sm_scale=sc, **okw), name + " ")


def test_single_key_rows(F):
    """Under a causal mask query 0 keeps one key: o[0] is v[0] up to the rounding of the one probability
    to bf16 (p is rounded for the PV product, l sums the unrounded p: at most one bf16 step) and its
    dq, P (dP - delta) with dP ~ delta, all but vanishes."""
    from flex_attention_tpu_amd import masks
    sc = 1 / math.sqrt(128)
    q, k, v, do = O.make_inputs(2, 4, 4, 512, 512, 128, dtype=torch.bfloat16, seed=29)
    q, k, v, do = [x.to(DEV) for x in (q, k, v, do)]
    mf, bf = masks.make_causal_mask_fns(128, 128)
    o, l, m = _fwd(F, q, k, v, sc, mf, bf, None)
    o0, v0 = o[:, :, 0, :].float(), v[:, :, 0, :].float()
    assert bool(((o0 - v0).abs() <= v0.abs() * 2.0 ** -7).all())
    assert float((l[:, :, 0] - 1).abs().max()) < 1e-6
    d = F.compute_delta(o, do)
    dq = _dq(F, q, k, v, l, m, o, do, d, sc, mf, bf, None)
    assert float(dq[:, :, 0, :].float().abs().max()) <= 2e-2


@pytest.mark.parametrize("mask", ["none", "causal"])
def test_growing_scores_move_the_reference_maximum(F, mask):
    """Keys whose norm grows along the sequence and a large logit scale: the running row maximum keeps
    rising by tens of log2 units, so the forward stream's reference maximum moves many times per row (the
    blocks it normally skips, and the correction of the chain in flight).  Forward against the oracle."""
    from flex_attention_tpu_amd import masks
    B, H, S, D = 2, 4, 2048, 128
    q, k, v, _ = O.make_inputs(B, H, H, S, S, D, dtype=torch.bfloat16, seed=41)
    k = (k.float() * torch.linspace(0.1, 3.0, S).view(1, 1, S, 1)).to(torch.bfloat16)
    # (sm_scale * log2(e) = 0.5 exactly: the streams fold that factor into their bf16 copy of Q, which
    # then rounds nothing; with logits this large any other scale would test that rounding instead)
    sc = 0.5 * math.log(2.0)
    causal = mask == "causal"
    mf, bf = masks.make_causal_mask_fns(128, 128) if causal else (None, None)
    ro, rl, rm = O.mha_reference(q, k, v, save_residuals=True, sm_scale=sc, causal=causal)
    o, l, m = _fwd(F, q.to(DEV), k.to(DEV), v.to(DEV), sc, mf, bf, None)
    assert_close(f"o[{mask}]", o, ro, torch.bfloat16)
    lse, rlse = m + torch.log(l), rm + torch.log(rl)
    assert float((lse.cpu().double() - rlse.double()).abs().max()) <= 2e-2 + 2.0 ** -8 * float(rlse.abs().max())
    assert float((m.cpu().double() - rm.double()).abs().max()) <= 2.0 ** -7 * float(rm.abs().max())


@pytest.mark.parametrize("shape", [(1, 1, 1, 128, 128), (1, 2, 1, 384, 384), (2, 3, 3, 640, 640), (1, 4, 2, 1152, 1152),
                                   (2, 16, 16, 2048, 2048), (3, 16, 4, 2048, 2048), (8, 32, 32, 1024, 1024),
                                   (1, 2, 2, 256, 1280), (1, 2, 2, 1280, 256)], ids=lambda s: "x".join(map(str, s)))
def test_odd_shapes_against_the_fp32_kernels(F, shape):
    """Shapes around the edges of the work schedules (one tile, odd tile counts, a missing second q tile
    of a forward pair, grids below, at and above one work-group per CU, GQA, Sq != Sk): the bf16
    generated-stream kernels against the fp32 kernels (exact arithmetic, independent code) on the
    same bf16-rounded inputs, plain and with masks that leave partial and empty tiles."""
    from flex_attention_tpu_amd import masks
    B, Hq, Hkv, Sq, Sk = shape
    sc = 1 / math.sqrt(128)
    g = torch.Generator().manual_seed(Sq + 7 * Sk + Hq)
    q, do = (torch.randn(B, Hq, Sq, 128, generator=g).to(torch.bfloat16).to(DEV) for _ in range(2))
    k, v = (torch.randn(B, Hkv, Sk, 128, generator=g).to(torch.bfloat16).to(DEV) for _ in range(2))
    pairs = [(None, None)]
    if Sq == Sk:
        lens, left = [], Sq
        while left > 0:
            lens.append(min(left, 128 + (len(lens) * 97) % 300))
            left -= lens[-1]
        pairs += [masks.make_causal_mask_fns(128, 128), masks.make_causal_sliding_window_mask_fns(128, 128, 300),
                  masks.make_jagged_mask_fns(128, 128, lens)]
    for mf, bf in pairs:
        def all_passes(q_, k_, v_, do_):
            o, l, m = _fwd(F, q_, k_, v_, sc, mf, bf, None)
            d = F.compute_delta(o, do_)
            return (o, m + l.log(), _dq(F, q_, k_, v_, l, m, o, do_, d, sc, mf, bf, None)) + tuple(
                _dkv(F, q_, k_, v_, l, m, do_, d, sc, mf, bf, None))
        got = all_passes(q, k, v, do)
        ref = all_passes(q.float(), k.float(), v.float(), do.float())
        for name, a, b in zip(("o", "lse", "dq", "dk", "dv"), got, ref):
            assert O.rel_l2(a.float().cpu(), b.cpu()) <= 1e-2, (name, shape)


@pytest.mark.parametrize("shape", [(1, 2, 128, 128), (2, 3, 640, 640), (2, 16, 2048, 2048), (8, 32, 1024, 1024), (1, 2, 256, 1280),
                                   (1, 2, 1280, 256)], ids=lambda s: "x".join(map(str, s)))
def test_position_bias_against_the_fp32_kernels(F, shape):
    """slopes[h] (j - i) added to the scores (one query head per kv head: the generated-stream kernels
    take it in) against the fp32 kernels, without a mask (the bias grows towards later keys), under
    the causal mask and under a causal window, on grids below and above one work-group per CU."""
    from flex_attention_tpu_amd import masks, scores
    B, H, Sq, Sk = shape
    sc = 1 / math.sqrt(128)
    g = torch.Generator().manual_seed(Sq + 7 * Sk + H)
    q, do = (torch.randn(B, H, Sq, 128, generator=g).to(torch.bfloat16).to(DEV) for _ in range(2))
    k, v = (torch.randn(B, H, Sk, 128, generator=g).to(torch.bfloat16).to(DEV) for _ in range(2))
    sfn = scores.make_alibi_global_score_fn(H)
    pairs = [(None, None)]
    if Sq == Sk:
        pairs += [masks.make_causal_mask_fns(128, 128), masks.make_causal_sliding_window_mask_fns(128, 128, 300)]
    for mf, bf in pairs:
        def all_passes(q_, k_, v_, do_):
            o, l, m = _fwd(F, q_, k_, v_, sc, mf, bf, sfn)
            d = F.compute_delta(o, do_)
            return (o, m + l.log(), _dq(F, q_, k_, v_, l, m, o, do_, d, sc, mf, bf, sfn)) + tuple(
                _dkv(F, q_, k_, v_, l, m, do_, d, sc, mf, bf, sfn))
        got = all_passes(q, k, v, do)
        ref = all_passes(q.float(), k.float(), v.float(), do.float())
        for name, a, b in zip(("o", "lse", "dq", "dk", "dv"), got, ref):
            assert O.rel_l2(a.float().cpu(), b.cpu()) <= 1e-2, (name, shape, mf is None)


@pytest.mark.parametrize("shape", [(1, 2, 2, 128, 128), (2, 4, 2, 640, 640), (1, 16, 4, 2048, 2048), (4, 32, 32, 1024, 1024),
                                   (1, 2, 2, 256, 1280)], ids=lambda s: "x".join(map(str, s)))
def test_softcap_against_the_fp32_kernels(F, shape):
    """cap tanh(s / cap) (the generated-stream kernels take it in where they can) against the fp32 kernels:
    a small and the benchmark's cap, no mask, causal and document masks, GQA, grids below and above one
    work-group per CU."""
    from flex_attention_tpu_amd import masks, scores
    B, Hq, Hkv, Sq, Sk = shape
    sc = 1 / math.sqrt(128)
    g = torch.Generator().manual_seed(Sq + 7 * Sk + Hq)
    q, do = (torch.randn(B, Hq, Sq, 128, generator=g).to(torch.bfloat16).to(DEV) for _ in range(2))
    k, v = (torch.randn(B, Hkv, Sk, 128, generator=g).to(torch.bfloat16).to(DEV) for _ in range(2))
    q = q * 3  # (scores of several caps: the tanh saturates)
    pairs = [(None, None)]
    if Sq == Sk:
        lens, left = [], Sq
        while left > 0:
            lens.append(min(left, 128 + (len(lens) * 97) % 300))
            left -= lens[-1]
        pairs += [masks.make_causal_mask_fns(128, 128), masks.make_jagged_mask_fns(128, 128, lens)]
    for cap in (2.0, 30.0):
        sfn = scores.make_softcap_score_fn(cap)
        for mf, bf in pairs:
            def all_passes(q_, k_, v_, do_):
                o, l, m = _fwd(F, q_, k_, v_, sc, mf, bf, sfn)
                d = F.compute_delta(o, do_)
                return (o, m + l.log(), _dq(F, q_, k_, v_, l, m, o, do_, d, sc, mf, bf, sfn)) + tuple(
                    _dkv(F, q_, k_, v_, l, m, do_, d, sc, mf, bf, sfn))
            got = all_passes(q, k, v, do)
            ref = all_passes(q.float(), k.float(), v.float(), do.float())
            for name, a, b in zip(("o", "lse", "dq", "dk", "dv"), got, ref):
                assert O.rel_l2(a.float().cpu(), b.cpu()) <= 1e-2, (name, shape, cap, mf is None)


def test_document_masks_longest_first_schedule(F):
    """Enough (batch, head, tile) items that the persistent work-groups of all three generated-stream kernels
    take the longest-first schedule that document masks get (eight items each), with documents of very
    different lengths: against the fp32 kernels."""
    from flex_attention_tpu_amd import masks
    B, H, S = 16, 32, 1024
    sc = 1 / math.sqrt(128)
    g = torch.Generator().manual_seed(91)
    q, do = (torch.randn(B, H, S, 128, generator=g).to(torch.bfloat16).to(DEV) for _ in range(2))
    k, v = (torch.randn(B, H, S, 128, generator=g).to(torch.bfloat16).to(DEV) for _ in range(2))
    mf, bf = masks.make_jagged_mask_fns(128, 128, [100, 412, 212, 300])

    def all_passes(q_, k_, v_, do_):
        o, l, m = _fwd(F, q_, k_, v_, sc, mf, bf, None)
        d = F.compute_delta(o, do_)
        return (o, m + l.log(), _dq(F, q_, k_, v_, l, m, o, do_, d, sc, mf, bf, None)) + tuple(
            _dkv(F, q_, k_, v_, l, m, do_, d, sc, mf, bf, None))
    got = all_passes(q, k, v, do)
    ref = all_passes(q.float(), k.float(), v.float(), do.float())
    for name, a, b in zip(("o", "lse", "dq", "dk", "dv"), got, ref):
        assert O.rel_l2(a.float().cpu(), b.cpu()) <= 1e-2, name


def _sampled_oracle_check(F, q, k, v, do, sc, mf, bf, sfn, okw, n_rows, heads, dtype=torch.bfloat16, tag="", **call_kw):
    """All passes of one call on the GPU against the oracle on `n_rows` sampled q rows of the (batch, q head)
    pairs `heads` (whole kv groups): o, lse and dq on those rows; dk, dv with dO zeroed outside the sampled rows
    (the gradients are linear in dO, so every kv position is exercised at full length).  The backward against the
    oracle's backward from the kernels' own residuals.  `call_kw` goes to the three entry points (compiled_loop)."""
    B, Hq, Sq, _ = q.shape
    Hkv = k.shape[1]
    g = torch.Generator().manual_seed(7)
    rows = torch.sort(torch.randperm(Sq, generator=g)[:n_rows]).values
    rows[0], rows[-1] = 0, Sq - 1
    ro, rl, rm = O.mha_reference(q, k, v, sm_scale=sc, save_residuals=True, q_rows=rows, heads=heads,
                                 compute_dtype=torch.float32, **okw)
    do_s = torch.zeros_like(do)
    do_s[:, :, rows] = do[:, :, rows]
    qg, kg, vg, dog = [x.to(DEV) for x in (q, k, v, do_s)]
    o, l, m = F._flex_attention_impl(qg, kg, vg, None, None, True, False, sc, 1, 128, 128, 128, False, bf, mf, sfn, **call_kw)
    d = F.compute_delta(o, dog)
    dq = F.flex_attention_bwd_dq(qg, kg, vg, None, None, l, m, o, dog, d, block_b=1, block_q=128, block_k_major=128,
                                 block_k=128, sm_scale=sc, debug=False, score_fn=sfn, mask_fn=mf, block_mask_fn=bf, **call_kw)
    dk, dv = F.flash_attention_bwd_dkv(kg, vg, qg, None, None, l, m, d, dog, block_b=1, block_q=128, block_q_major=128,
                                       block_k_major=128, block_k=128, sm_scale=sc, causal=False, debug=False,
                                       score_fn=sfn, mask_fn=mf, block_mask_fn=bf, **call_kw)
    torch.cuda.synchronize()
    sdq, sdk, sdv = same_residual_grads(q, k, v, do_s, o, l, m, sm_scale=sc, q_rows=rows, heads=heads,
                                        compute_dtype=torch.float32, **okw)
    dr = rows.to(DEV)
    group = Hq // Hkv
    for (b, h) in heads:
        assert_close(f"{tag}o[{b},{h}]", o[b, h, dr], ro[b, h], dtype)
        assert_close(f"{tag}lse[{b},{h}]", (m + l.log())[b, h, dr], (rm + rl.log())[b, h], dtype)
        assert_close(f"{tag}dq[{b},{h}]", dq[b, h, dr], sdq[b, h], dtype)
    for (b, hk) in sorted({(b, h // group) for (b, h) in heads}):
        assert all((b, hk * group + gq) in heads for gq in range(group)), "sample whole KV groups"
        assert_close(f"{tag}dk[{b},{hk}]", dk[b, hk], sdk[b, hk], dtype)
        assert_close(f"{tag}dv[{b},{hk}]", dv[b, hk], sdv[b, hk], dtype)


@pytest.mark.parametrize("S,compiled_loop", [(131072, False), (131072, True), (262144, False)],
                         ids=["131072-default", "131072-compiled_loop", "262144-default"])
def test_long_tile_lists(F, S, compiled_loop):
    """One head of 131072 and of 262144 tokens under the causal mask (the reference's own sweep goes to 262144,
    roofline_data_flex.csv:10): up to 4096 kv tiles of 64 rows in a row's list and 2048 q tiles of 128 rows in a
    column's.  The generated-stream kernels prefetch the first 1024 (dq: 2048) list entries of an item in
    registers and read the rest of a longer list when the item starts; and the same with every pass on its
    compiled-loop kernel.  Sampled rows against the oracle."""
    from flex_attention_tpu_amd import masks
    sc = 1 / math.sqrt(128)
    q, k, v, do = O.make_inputs(1, 1, 1, S, S, 128, dtype=torch.bfloat16, seed=131)
    mf, bf = masks.make_causal_mask_fns(128, 128)
    _sampled_oracle_check(F, q, k, v, do, sc, mf, bf, None, dict(causal=True), 160, [(0, 0)], compiled_loop=compiled_loop)


def test_long_tile_lists_position_bias_and_window(F):
    """Lists beyond the prefetched part under the other stream variants: the position bias (whose forward walks
    the list from its end) with a causal window at 131072 tokens (rows of 2048 kv tiles, of which a window of 5000
    tokens keeps about 80), two heads."""
    from flex_attention_tpu_amd import masks, scores
    S = 131072
    sc = 1 / math.sqrt(128)
    q, k, v, do = O.make_inputs(1, 2, 2, S, S, 128, dtype=torch.bfloat16, seed=133)
    mf, bf = masks.make_causal_sliding_window_mask_fns(128, 128, 5000)
    sfn = scores.make_alibi_global_score_fn(2)
    okw = dict(causal=True, window_size=5000, score_mod=O.score_mod_alibi_global(O.alibi_slopes(2)))
    _sampled_oracle_check(F, q, k, v, do, sc, mf, bf, sfn, okw, 128, [(0, 0), (0, 1)])


@pytest.mark.parametrize("case", ["persistent_mha_b8_h32_s1024", "gqa_4to1_s2048", "documents_longest_first",
                                  "alibi_b8_h32_s1024", "softcap_gqa_s2048"])
def test_schedule_edges_against_the_oracle(F, case):
    """Shapes at the edges of the work schedules (the persistent grid of one work-group per CU with several heads
    per work-group, grouped kv heads at 2048 tokens, the longest-first schedule that document masks get with
    eight items per work-group) and the position-bias and softcap streams on such grids: sampled rows of a few
    heads of the full launch against the oracle."""
    from flex_attention_tpu_amd import masks, scores
    sc = 1 / math.sqrt(128)
    mf, bf, sfn = None, None, None
    if case == "persistent_mha_b8_h32_s1024":
        B, Hq, Hkv, S, heads = 8, 32, 32, 1024, [(0, 0), (5, 17), (7, 31)]
        (mf, bf), okw = masks.make_causal_mask_fns(128, 128), dict(causal=True)
    elif case == "gqa_4to1_s2048":
        B, Hq, Hkv, S, heads = 3, 16, 4, 2048, [(0, 0), (0, 1), (0, 2), (0, 3), (2, 12), (2, 13), (2, 14), (2, 15)]
        (mf, bf), okw = masks.make_causal_sliding_window_mask_fns(128, 128, 300), dict(causal=True, window_size=300)
    elif case == "documents_longest_first":
        B, Hq, Hkv, S, heads = 16, 32, 32, 1024, [(0, 0), (9, 30), (15, 31)]
        lens = [100, 412, 212, 300]
        (mf, bf), okw = masks.make_jagged_mask_fns(128, 128, lens), dict(causal=True, segment_ids=O.doc_ids_from_lengths(lens))
    elif case == "alibi_b8_h32_s1024":
        B, Hq, Hkv, S, heads = 8, 32, 32, 1024, [(0, 0), (3, 8), (7, 31)]
        (mf, bf), sfn = masks.make_causal_mask_fns(128, 128), scores.make_alibi_global_score_fn(32)
        okw = dict(causal=True, score_mod=O.score_mod_alibi_global(O.alibi_slopes(32)))
    else:
        B, Hq, Hkv, S, heads = 1, 16, 4, 2048, [(0, 4), (0, 5), (0, 6), (0, 7)]
        lens = [700, 900, 448]
        (mf, bf), sfn = masks.make_jagged_mask_fns(128, 128, lens), scores.make_softcap_score_fn(2.0)
        okw = dict(causal=True, segment_ids=O.doc_ids_from_lengths(lens), score_mod=O.score_mod_softcap(2.0))
    q, k, v, do = O.make_inputs(B, Hq, Hkv, S, S, 128, dtype=torch.bfloat16, seed=137)
    if case == "softcap_gqa_s2048":
        q = (q.float() * 3).to(torch.bfloat16)   # (scores of several caps: the tanh saturates)
    _sampled_oracle_check(F, q, k, v, do, sc, mf, bf, sfn, okw, 160, heads)


def test_integration_doc_binding_runs_verbatim(F):
    """The ctypes binding printed in the integration notes at the repository root, executed as it stands (only the
    library path is filled in), against the oracle: the struct layouts of the document and of the header agree."""
    import re
    from flex_attention_tpu_amd import _lib
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "INTEGRATION.md")).read()
    code = re.search(r"```python\n(.*?)```", text, flags=re.S).group(1)
    assert "def causal_forward" in code
    ns = {}
    exec(compile(code.replace('"libflexattn.so"', repr(_lib.LIB_PATH)), "INTEGRATION.md", "exec"), ns)
    sc = 1 / math.sqrt(128)
    q, k, v = O.make_inputs(2, 3, 3, 512, 512, 128, dtype=torch.bfloat16, seed=41, with_do=False)
    ro, rl, rm = O.mha_reference(q, k, v, sm_scale=sc, save_residuals=True, causal=True)
    o, l, m = ns["causal_forward"](q.to(DEV), k.to(DEV), v.to(DEV), sc)
    torch.cuda.synchronize()
    assert_close("o", o, ro, torch.bfloat16)
    assert_close("lse", m + l.log(), rm + rl.log(), torch.bfloat16)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "fp32"])
def test_rows_that_keep_no_key(F, dtype):
    """Sq > Sk under a window: q rows i >= Sk - 1 + window keep no key.  They return o = 0, l = 0,
    m = -inf and contribute nothing to any gradient (no NaN anywhere); the other rows match the
    oracle.  (The reference replaces masked logits by -1e9 and would return a uniform softmax for
    such rows; they are outside its contract.)"""
    from flex_attention_tpu_amd import masks
    Sq, Sk, W = 512, 256, 100
    sc = 1 / math.sqrt(128)
    first_empty = Sk - 1 + W
    q, k, v, do = O.make_inputs(1, 2, 2, Sq, Sk, 128, dtype=dtype, seed=3)
    live = torch.arange(first_empty)
    okw = dict(sm_scale=sc, window_size=W, q_rows=live)
    ro, rl, rm = O.mha_reference(q, k, v, save_residuals=True, **okw)
    rdq, rdk, rdv = O.mha_bwd_reference(q, k, v, ro, do[:, :, live], rl, rm, **okw)
    mf, bf = masks.make_sliding_window_mask_fns(128, 128, W)
    qc, kc, vc, doc = q, k, v, do
    q, k, v, do = [x.to(DEV) for x in (q, k, v, do)]
    o, l, m = _fwd(F, q, k, v, sc, mf, bf, None)
    assert float(o[:, :, first_empty:].float().abs().max()) == 0.0
    assert float(l[:, :, first_empty:].abs().max()) == 0.0 and bool(torch.isinf(m[:, :, first_empty:]).all())
    assert_close("o", o[:, :, :first_empty], ro, dtype)
    d = F.compute_delta(o, do)
    dq = _dq(F, q, k, v, l, m, o, do, d, sc, mf, bf, None)
    dk, dv = _dkv(F, q, k, v, l, m, do, d, sc, mf, bf, None)
    for t in (dq, dk, dv):
        assert bool(torch.isfinite(t.float()).all())
    assert float(dq[:, :, first_empty:].float().abs().max()) == 0.0
    _check_grads((dq[:, :, :first_empty], dk, dv), (rdq, rdk, rdv), qc, kc, vc, doc, o, l, m, dtype, okw)
    # dq from the dk/dv pass's dS: the last q tile's list of kv tiles is empty (its rows are written as zeros)
    dqx = _exchanged_dq(F, q, k, v, l, m, o, do, d, sc, mf, bf, None, dk, dv, expect=dtype == torch.bfloat16)
    if dqx is not None:
        assert float(dqx[:, :, first_empty:].float().abs().max()) == 0.0
        _check_grads((dqx[:, :, :first_empty], dk, dv), (rdq, rdk, rdv), qc, kc, vc, doc, o, l, m, dtype, okw, tag="exchange ")


@pytest.mark.parametrize("case", ["causal", "gqa_softcap_docs", "alibi_window", "fp32_plain"])
def test_autograd_function_end_to_end(F, case):
    """torch.autograd.grad through flex_attention (forward saves o, l, m; backward runs delta, dq and
    dk/dv: the wiring of jax_exp.py:207-321) against the oracle's gradients."""
    from flex_attention_tpu_amd import masks, scores
    sc = 1 / math.sqrt(128)
    dtype = torch.bfloat16
    if case == "causal":
        shape, mf, sfn, okw = (2, 4, 4, 512, 512), masks.make_causal_mask_fns(128, 128), None, dict(causal=True)
    elif case == "gqa_softcap_docs":
        lens = [200, 312, 512]
        shape, mf, sfn = (1, 8, 2, 1024, 1024), masks.make_jagged_mask_fns(128, 128, lens), scores.make_softcap_score_fn(30.0)
        okw = dict(causal=True, segment_ids=O.doc_ids_from_lengths(lens), score_mod=O.score_mod_softcap(30.0))
    elif case == "alibi_window":
        shape, mf = (1, 4, 4, 1024, 1024), masks.make_causal_sliding_window_mask_fns(128, 128, 257)
        sfn = scores.make_alibi_global_score_fn(4)
        okw = dict(causal=True, window_size=257, score_mod=O.score_mod_alibi_global(O.alibi_slopes(4)))
    else:
        shape, mf, sfn, okw, dtype = (1, 4, 4, 512, 512), None, None, {}, torch.float32
    B, Hq, Hkv, Sq, Sk = shape
    q, k, v, do = O.make_inputs(B, Hq, Hkv, Sq, Sk, 128, dtype=dtype, seed=53)
    ro, rl, rm = O.mha_reference(q, k, v, sm_scale=sc, save_residuals=True, **okw)
    rdq, rdk, rdv = O.mha_bwd_reference(q, k, v, ro, do, rl, rm, sm_scale=sc, **okw)
    qg, kg, vg = [x.to(DEV).requires_grad_(True) for x in (q, k, v)]
    o = F.flex_attention(qg, kg, vg, sfn, mf, sm_scale=sc)
    assert o.requires_grad and o.dtype == dtype
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), do.to(DEV))
    assert_close("o", o, ro, dtype)
    # (the saved statistics are not returned by the differentiable op: the same forward once more for them)
    mfn, bfn = mf if mf is not None else (None, None)
    o_, l_, m_ = _fwd(F, qg.detach(), kg.detach(), vg.detach(), sc, mfn, bfn, sfn)
    assert torch.equal(o_, o.detach())
    _check_grads((dq, dk, dv), (rdq, rdk, rdv), q, k, v, do, o_, l_, m_, dtype, dict(sm_scale=sc, **okw))
    # .backward() accumulates into .grad; gradients only where asked for
    o2 = F.flex_attention(qg, kg.detach(), vg.detach(), sfn, mf, sm_scale=sc)
    o2.backward(do.to(DEV))
    assert kg.grad is None
    # (dq alone is recomputed by the dq kernel; with dk / dv wanted as well it comes from the dk/dv pass's dS where
    # the backward hands it over, softcap scores: not the same bits, the same bound)
    sdq = same_residual_grads(q, k, v, do, o_, l_, m_, sm_scale=sc, **okw)[0]
    assert_close("dq alone", qg.grad, sdq, dtype)
    if case != "gqa_softcap_docs":
        assert torch.equal(qg.grad, dq)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "fp32"])
@pytest.mark.parametrize("case", ["plain_200x300", "causal_1000", "softcap_causal_window_700", "alibi_causal_333",
                                  "documents_900", "gqa_causal_130"])
def test_ragged_sequence_lengths(F, case, dtype):
    """Lengths that are no multiple of the kernels' tiles (the reference's drivers use Sk = 25600 with
    1024-blocks, bwd_dq.py:389-390): the entry points pad to the tile, padded keys get no probability, and
    every output has the caller's lengths."""
    from flex_attention_tpu_amd import masks, scores
    sc = 1 / math.sqrt(128)
    B, Hq, Hkv, mf, sfn, okw, sid = 1, 2, 2, (None, None), None, {}, None
    if case == "plain_200x300":
        Sq, Sk = 200, 300
    elif case == "causal_1000":
        Sq = Sk = 1000
        mf, okw = masks.make_causal_mask_fns(128, 128), dict(causal=True)
    elif case == "softcap_causal_window_700":
        Sq = Sk = 700
        mf, sfn = masks.make_causal_sliding_window_mask_fns(128, 128, 200), scores.make_softcap_score_fn(10.0)
        okw = dict(causal=True, window_size=200, score_mod=O.score_mod_softcap(10.0))
    elif case == "alibi_causal_333":
        Sq = Sk = 333
        mf, sfn = masks.make_causal_mask_fns(128, 128), scores.make_alibi_global_score_fn(2)
        okw = dict(causal=True, score_mod=O.score_mod_alibi_global(O.alibi_slopes(2)))
    elif case == "documents_900":
        Sq = Sk = 900
        sid = O.doc_ids_from_lengths([250, 130, 400, 120])
        okw = dict(causal=True, segment_ids=sid)
    else:
        B, Hq, Hkv, Sq, Sk = 2, 4, 2, 130, 130
        mf, okw = masks.make_causal_mask_fns(128, 128), dict(causal=True)
    q, k, v, do = O.make_inputs(B, Hq, Hkv, Sq, Sk, 128, dtype=dtype, seed=83)
    ro, rl, rm = O.mha_reference(q, k, v, sm_scale=sc, save_residuals=True, **okw)
    rdq, rdk, rdv = O.mha_bwd_reference(q, k, v, ro, do, rl, rm, sm_scale=sc, **okw)
    qg, kg, vg, dog = [x.to(DEV) for x in (q, k, v, do)]
    causal_flag = case == "documents_900"
    o, l, m = F._flex_attention_impl(qg, kg, vg, None, sid, True, causal_flag, sc, 1, 128, 128, 128, False, mf[1], mf[0], sfn)
    assert o.shape == q.shape and l.shape == (B, Hq, Sq) and o.is_contiguous()
    assert_close("o", o, ro, dtype)
    assert_close("lse", m + l.log(), rm + rl.log(), dtype)
    d = F.compute_delta(o, dog)
    dq = F.flex_attention_bwd_dq(qg, kg, vg, None, sid, l, m, o, dog, d, block_b=1, block_q=128, block_k_major=128,
                                 block_k=128, sm_scale=sc, debug=False, score_fn=sfn, mask_fn=mf[0], block_mask_fn=mf[1],
                                 causal=causal_flag)
    dk, dv = F.flash_attention_bwd_dkv(kg, vg, qg, None, sid, l, m, d, dog, block_b=1, block_q=128, block_q_major=128,
                                       block_k_major=128, block_k=128, sm_scale=sc, causal=causal_flag, debug=False,
                                       score_fn=sfn, mask_fn=mf[0], block_mask_fn=mf[1])
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    _check_grads((dq, dk, dv), (rdq, rdk, rdv), q, k, v, do, o, l, m, dtype, dict(sm_scale=sc, **okw))
    dqx = _exchanged_dq(F, qg, kg, vg, l, m, o, dog, d, sc, mf[0], mf[1], sfn, dk, dv,
                        expect=dtype == torch.bfloat16 and not case.startswith("alibi"), causal=causal_flag, sid=sid)
    if dqx is not None:
        assert dqx.shape == q.shape
        _check_grads((dqx, dk, dv), (rdq, rdk, rdv), q, k, v, do, o, l, m, dtype, dict(sm_scale=sc, **okw), tag="exchange ")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "fp32"])
def test_distinct_unsorted_segment_ids(F, dtype):
    """q and kv positions with ids of their own (the reference's SegmentIds with .q / .kv, jax_exp.py:37-51),
    not sorted along the sequence, different lengths on the two sides: keep = same id (and causal)."""
    import types
    sc = 1 / math.sqrt(128)
    Sq, Sk = 384, 640
    g = torch.Generator().manual_seed(5)
    ids_q = torch.randint(0, 3, (Sq // 32,), generator=g).repeat_interleave(32)    # runs of 32, ids recur
    ids_k = torch.randint(0, 3, (Sk // 16,), generator=g).repeat_interleave(16)
    ids_k[:16] = ids_q[0]                                                            # (every query keeps a key)
    for v_ in range(3):
        ids_k[16 * (v_ + 1): 16 * (v_ + 2)] = v_
    keep = ids_q[:, None] == ids_k[None, :]
    q, k, v, do = O.make_inputs(1, 2, 2, Sq, Sk, 128, dtype=dtype, seed=89)
    okw = dict(sm_scale=sc, mask=keep)
    ro, rl, rm = O.mha_reference(q, k, v, save_residuals=True, **okw)
    rdq, rdk, rdv = O.mha_bwd_reference(q, k, v, ro, do, rl, rm, **okw)
    sid = types.SimpleNamespace(q=ids_q, kv=ids_k)
    qg, kg, vg, dog = [x.to(DEV) for x in (q, k, v, do)]
    o, l, m = F._flex_attention_impl(qg, kg, vg, None, sid, True, False, sc, 1, 128, 128, 128, False, None, None, None)
    assert_close("o", o, ro, dtype)
    d = F.compute_delta(o, dog)
    dq = F.flex_attention_bwd_dq(qg, kg, vg, None, sid, l, m, o, dog, d, block_b=1, block_q=128, block_k_major=128,
                                 block_k=128, sm_scale=sc, debug=False)
    dk, dv = F.flash_attention_bwd_dkv(kg, vg, qg, None, sid, l, m, d, dog, block_b=1, block_q=128, block_q_major=128,
                                       block_k_major=128, block_k=128, sm_scale=sc, causal=False, debug=False)
    _check_grads((dq, dk, dv), (rdq, rdk, rdv), q, k, v, do, o, l, m, dtype, okw)
    # the builder's map for unsorted ids: never skips a tile with a kept element, never calls a tile full that is not
    from flex_attention_tpu_amd import _common, block_mask
    spec = _common.resolve_mask(None, None, False, sid, Sq, Sk)
    bm = block_mask.build_block_map(spec, Sq, Sk, 128, 64, DEV)
    brute = O.block_map_bruteforce(keep, 128, 64)
    st = bm.state.cpu()
    assert bool(((st == 0) <= (brute == 0)).all()) and bool(((st == 2) <= (brute == 2)).all())


def test_entry_points_reject_bad_arguments_on_gpu(F):
    q = torch.zeros(1, 2, 256, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError):  # block_q must divide the sequence length
        F._flex_attention_impl(q, q, q, None, None, False, False, 1.0, 1, 96, 64, 64, False, None, None, None)
    q = torch.zeros(1, 2, 256, 384, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(NotImplementedError):  # bf16 head dimensions above 256 have no kernel (others are padded to 128 or 256)
        F._flex_attention_impl(q, q, q, None, None, False, False, 1.0, 1, 128, 128, 128, False, None, None, None)
    q = torch.zeros(1, 2, 256, 192, dtype=torch.float32, device=DEV)
    with pytest.raises(NotImplementedError):  # float32: above 128
        F._flex_attention_impl(q, q, q, None, None, False, False, 1.0, 1, 128, 128, 128, False, None, None, None)
    q = torch.zeros(1, 2, 256, 128, dtype=torch.float16, device=DEV)
    with pytest.raises(NotImplementedError):
        F._flex_attention_impl(q, q, q, None, None, False, False, 1.0, 1, 128, 128, 128, False, None, None, None)
    q = torch.zeros(2, 2, 256, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError, match="rows"):  # ids per batch entry: one row for every entry of the call
        F._flex_attention_impl(q, q, q, None, torch.arange(3)[:, None].expand(3, 256), False, False, 1.0, 1, 128, 128, 128,
                               False, None, None, None)


# ------------------------------------------------------------------------------------------------
# the five benchmark configurations at full size
# ------------------------------------------------------------------------------------------------
def test_cfg1_fp32_full(F):
    from flex_attention_tpu_amd import configs
    cfg = configs.CONFIGS["cfg1"]
    q, k, v, do = configs.make_inputs(cfg)
    sc = cfg.sm_scale
    ro, rl, rm = O.mha_reference(q, k, v, sm_scale=sc, save_residuals=True)
    rdq, rdk, rdv = O.mha_bwd_reference(q, k, v, ro, do, rl, rm, sm_scale=sc)
    qc, kc, vc, doc = q, k, v, do
    q, k, v, do = [x.to(DEV) for x in (q, k, v, do)]
    o, l, m = _fwd(F, q, k, v, sc, None, None, None)
    d = F.compute_delta(o, do)
    dq = _dq(F, q, k, v, l, m, o, do, d, sc, None, None, None)
    dk, dv = _dkv(F, q, k, v, l, m, do, d, sc, None, None, None)
    for name, t, r in (("o", o, ro), ("m", m, rm), ("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv)):
        assert_close(name, t, r, torch.float32)   # (fp32: the whole chain meets 1e-5 as it stands)
    assert O.rel_l2(l, rl) <= 1e-5
    _check_grads((dq, dk, dv), (rdq, rdk, rdv), qc, kc, vc, doc, o, l, m, torch.float32, dict(sm_scale=sc))


def _full_config_check(F, name, n_rows, heads_q, dense_group):
    """Runs forward, delta, dq and dk/dv of a full-size configuration and checks
    (1) o, l, m and dq on `n_rows` sampled q rows of the heads `heads_q` against the oracle,
    (2) dk, dv against the oracle with dO zeroed outside the sampled rows (the gradients are linear
        in dO, so this exercises every kv position at full sequence length),
        (gradients: against the oracle's backward from the kernels' own residuals at the stated bound, and
        against the oracle's whole chain in rel-L2, see _check_grads)
    (3) invariants of the dense-dO run: sum_i q_i.dq_i == sum_j k_j.dk_j per kv head, and
        row-stochastic P (v = 1 gives o = 1),
    (4) o, lse, dq of every row of the q heads of the kv group `dense_group` = (b, kv head) and that
        kv head's dk, dv, taken from the same dense full-size launch (persistent work-groups, several
        items each, cross-item prefetch), against the dense oracle."""
    from flex_attention_tpu_amd import configs
    cfg = configs.CONFIGS[name]
    sc = cfg.sm_scale
    okw = oracle_kwargs(cfg)
    q, k, v, do = configs.make_inputs(cfg)
    mf, bf = configs.mask_fns(cfg)
    sfn = configs.score_fn(cfg)
    g = torch.Generator().manual_seed(1)
    rows = torch.sort(torch.randperm(cfg.S, generator=g)[:n_rows]).values
    rows[0], rows[-1] = 0, cfg.S - 1
    heads = [(b, h) for (b, h) in heads_q]
    ro, rl, rm = O.mha_reference(q, k, v, sm_scale=sc, save_residuals=True, q_rows=rows, heads=heads, **okw)
    rdq, rdk_s, rdv_s = O.mha_bwd_reference(q, k, v, ro, do[:, :, rows], rl, rm, sm_scale=sc, q_rows=rows, heads=heads, **okw)
    do_sparse = torch.zeros_like(do)
    do_sparse[:, :, rows] = do[:, :, rows]

    qg, kg, vg, dog, dosg = [x.to(DEV) for x in (q, k, v, do, do_sparse)]
    o, l, m = _fwd(F, qg, kg, vg, sc, mf, bf, sfn)
    d = F.compute_delta(o, dog)
    dq = _dq(F, qg, kg, vg, l, m, o, dog, d, sc, mf, bf, sfn)
    dk, dv = _dkv(F, qg, kg, vg, l, m, dog, d, sc, mf, bf, sfn)
    # (the same dq pass taking delta itself, as the package's backward runs it: the same bits)
    dq_f, d_f = F.flex_attention_bwd_dq(qg, kg, vg, None, None, l, m, o, dog, None, block_b=1, block_q=128, block_k_major=128,
                                        block_k=128, sm_scale=sc, debug=False, score_fn=sfn, mask_fn=mf, block_mask_fn=bf,
                                        return_delta=True)
    assert torch.equal(d_f, d) and torch.equal(dq_f, dq), "delta taken by the dq pass differs from the delta kernel's"
    d_s = F.compute_delta(o, dosg)
    dk_s, dv_s = _dkv(F, qg, kg, vg, l, m, dosg, d_s, sc, mf, bf, sfn)
    # the same backward with dS handed from the dk/dv pass to the dq pass (plain and softcap scores)
    dqx = _exchanged_dq(F, qg, kg, vg, l, m, o, dog, d, sc, mf, bf, sfn, dk, dv, expect=cfg.score in ("none", "softcap"))
    torch.cuda.synchronize()
    # the oracle's backward from the kernels' own residuals on the sampled rows (identical inputs)
    sdq, sdk_s, sdv_s = same_residual_grads(q, k, v, do, o, l, m, sm_scale=sc, q_rows=rows, heads=heads, **okw)

    group = cfg.Hq // cfg.Hkv
    for (b, h) in heads:
        assert_close(f"o[{b},{h}]", o[b, h, rows.to(DEV)], ro[b, h], cfg.dtype)
        assert_close(f"lse[{b},{h}]", (m + l.log())[b, h, rows.to(DEV)], (rm + rl.log())[b, h], cfg.dtype)
        assert_close(f"dq[{b},{h}]", dq[b, h, rows.to(DEV)], sdq[b, h], cfg.dtype)
        assert_close(f"dq[{b},{h}] chain", dq[b, h, rows.to(DEV)], rdq[b, h], cfg.dtype, chain=True)
        if dqx is not None:
            assert_close(f"exchange dq[{b},{h}]", dqx[b, h, rows.to(DEV)], sdq[b, h], cfg.dtype)
    kv_heads = sorted({(b, h // group) for (b, h) in heads})
    for (b, hk) in kv_heads:
        assert all((b, hk * group + gq) in heads for gq in range(group)), "sample whole KV groups"
        assert_close(f"dk[{b},{hk}]", dk_s[b, hk], sdk_s[b, hk], cfg.dtype)
        assert_close(f"dv[{b},{hk}]", dv_s[b, hk], sdv_s[b, hk], cfg.dtype)
        assert_close(f"dk[{b},{hk}] chain", dk_s[b, hk], rdk_s[b, hk], cfg.dtype, chain=True)
        assert_close(f"dv[{b},{hk}] chain", dv_s[b, hk], rdv_s[b, hk], cfg.dtype, chain=True)

    # invariants of the dense run (float64 sums of the bf16 results)
    qd = (qg.double() * dq.double()).sum(dim=(2, 3)).reshape(cfg.B, cfg.Hkv, group).sum(-1)
    kd = (kg.double() * dk.double()).sum(dim=(2, 3))
    scale = (qg.double().abs() * dq.double().abs()).sum(dim=(2, 3)).reshape(cfg.B, cfg.Hkv, group).sum(-1)
    assert float(((qd - kd).abs() / scale).max()) < 2e-3, "sum q.dq != sum k.dk"
    o1 = _fwd(F, qg, kg, torch.ones_like(vg), sc, mf, bf, sfn)[0]
    assert float((o1.float() - 1).abs().max()) < 1e-2, "P rows do not sum to 1"

    # (4) whole heads of the same dense full-size launch (every row, dense dO) against the dense oracle
    #     (float32 CPU math): the q heads of one kv group, so that dk, dv of its kv head are complete.
    b, hk = dense_group
    dheads = [(b, hk * group + gq) for gq in range(group)]
    wo, wl, wm = O.mha_reference(q, k, v, sm_scale=sc, save_residuals=True, heads=dheads, compute_dtype=torch.float32, **okw)
    wdq, wdk, wdv = same_residual_grads(q, k, v, do, o, l, m, sm_scale=sc, heads=dheads, compute_dtype=torch.float32, **okw)
    lse, wlse = m + l.log(), wm + wl.log()
    for (_, h) in dheads:
        assert_close(f"o[{b},{h}] whole", o[b, h], wo[b, h], cfg.dtype)
        assert_close(f"lse[{b},{h}] whole", lse[b, h], wlse[b, h], cfg.dtype)
        assert_close(f"dq[{b},{h}] whole", dq[b, h], wdq[b, h], cfg.dtype)
        if dqx is not None:
            assert_close(f"exchange dq[{b},{h}] whole", dqx[b, h], wdq[b, h], cfg.dtype)
    assert_close(f"dk[{b},{hk}] whole", dk[b, hk], wdk[b, hk], cfg.dtype)
    assert_close(f"dv[{b},{hk}] whole", dv[b, hk], wdv[b, hk], cfg.dtype)
    return dict(o=o, l=l, m=m, dq=dq, dk=dk, dv=dv)


def test_cfg2_cfg3_causal_bf16_full(F):
    _full_config_check(F, "cfg2", n_rows=384, heads_q=[(0, 0), (3, 31)], dense_group=(2, 13))


def test_cfg4_alibi_window_bf16_full(F):
    _full_config_check(F, "cfg4", n_rows=384, heads_q=[(0, 0), (1, 15)], dense_group=(1, 0))


def test_cfg5_gqa_softcap_document_bf16_full(F):
    _full_config_check(F, "cfg5", n_rows=384, heads_q=[(0, 4), (0, 5), (0, 6), (0, 7)], dense_group=(0, 5))


def test_whole_head_oracle_at_s4096(F):
    """Configuration 2/3 shape: two whole heads against the dense oracle (float32 CPU math)."""
    from flex_attention_tpu_amd import configs, masks
    cfg = configs.CONFIGS["cfg2"]
    sc = cfg.sm_scale
    q, k, v, do = O.make_inputs(1, 2, 2, cfg.S, cfg.S, cfg.D, dtype=cfg.dtype, seed=0)
    ro, rl, rm = O.mha_reference(q, k, v, sm_scale=sc, save_residuals=True, causal=True, compute_dtype=torch.float32)
    rdq, rdk, rdv = O.mha_bwd_reference(q, k, v, ro, do, rl, rm, sm_scale=sc, causal=True, compute_dtype=torch.float32)
    mf, bf = masks.make_causal_mask_fns(128, 128)
    qc, kc, vc, doc = q, k, v, do
    q, k, v, do = [x.to(DEV) for x in (q, k, v, do)]
    o, l, m = _fwd(F, q, k, v, sc, mf, bf, None)
    d = F.compute_delta(o, do)
    dq = _dq(F, q, k, v, l, m, o, do, d, sc, mf, bf, None)
    dk, dv = _dkv(F, q, k, v, l, m, do, d, sc, mf, bf, None)
    assert_close("o", o, ro, torch.bfloat16)
    _check_grads((dq, dk, dv), (rdq, rdk, rdv), qc, kc, vc, doc, o, l, m, torch.bfloat16,
                 dict(sm_scale=sc, causal=True, compute_dtype=torch.float32))
