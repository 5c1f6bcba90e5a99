"""CPU tests of the host-side mirror of the reference's Python surface: mask / score factories,
MaskSpec composition, argument validation."""
import json
import os

import numpy as np
import pytest
import torch

from flex_attention_tpu_amd import _lib, block_mask, configs, masks, scores
from oracle import mha_oracle as O

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _dense(mask_fn, S):
    idx = torch.arange(S)
    return mask_fn(idx, idx)


def test_mask_closures_match_oracle_dense_masks():
    S = 96
    lens = [20, 41, 35]
    cases = [
        (masks.make_causal_mask_fns(16, 16), dict(causal=True)),
        (masks.make_sliding_window_mask_fns(16, 16, 23), dict(window_size=23)),
        (masks.make_causal_sliding_window_mask_fns(16, 16, 10), dict(causal=True, window_size=10)),
        (masks.make_jagged_mask_fns(16, 16, lens), dict(causal=True, segment_ids=O.doc_ids_from_lengths(lens))),
        (masks.make_s2_mask_fns(16, 16, 9, 8), dict(window_size=9, s2_stride=8)),
    ]
    for (mf, bf), kw in cases:
        assert torch.equal(_dense(mf, S), O.dense_mask(S, S, **kw)), kw
        # closures also accept numpy index arrays, as the reference's accept jnp arrays
        idx = np.arange(S)
        assert np.array_equal(np.asarray(mf(idx, idx)), O.dense_mask(S, S, **kw).numpy())


def test_block_closures_match_closed_form_and_bruteforce():
    S, bq, bk = 256, 32, 16
    lens = [40, 100, 7, 109]
    sid = O.doc_ids_from_lengths(lens)
    cases = [
        (masks.make_causal_mask_fns(bq, bk), dict(causal=True), True),
        (masks.make_sliding_window_mask_fns(bq, bk, 50), dict(window_size=50), True),
        (masks.make_jagged_mask_fns(bq, bk, lens), dict(causal=True, segment_ids=sid), True),
        (masks.make_causal_sliding_window_mask_fns(bq, bk, 33), dict(causal=True, window_size=33), False),
        (masks.make_s2_mask_fns(bq, bk, 40, 16), dict(window_size=40, s2_stride=16), False),
    ]
    for (mf, bf), kw, exact in cases:
        host = block_mask.host_block_map(bf, S // bq, S // bk)
        closed = O.block_map_closed_form(S // bq, S // bk, bq, bk, **kw)
        assert torch.equal(host, closed), kw
        brute = O.block_map_bruteforce(_dense(mf, S), bq, bk) != 0
        if exact:
            assert torch.equal(host, brute), kw
        else:
            assert bool((host | ~brute).all()), kw  # conservative: never skips a tile with kept elements


def test_place_holder_and_spec_composition():
    p, pb = masks.place_holder(128, 128)
    assert p(3, 4) is True and p.spec.flags == 0
    c = masks.make_causal_mask_fns(8, 8)[0].spec
    w = masks.make_sliding_window_mask_fns(8, 8, 5)[0].spec
    cw = c.combine(w)
    assert cw.flags == (_lib.MASK_CAUSAL | _lib.MASK_WINDOW) and cw.window == 5
    assert w.combine(masks.MaskSpec(flags=_lib.MASK_WINDOW, window=3)).window == 3
    s2 = masks.make_s2_mask_fns(8, 8, 4, 2)[0].spec
    assert s2.combine(c) == s2
    with pytest.raises(NotImplementedError):
        s2.combine(w)
    j1 = masks.make_jagged_mask_fns(8, 8, [8, 8])[0].spec
    j2 = masks.make_jagged_mask_fns(8, 8, [4, 12])[0].spec
    assert j1.combine(c) == j1
    with pytest.raises(NotImplementedError):
        j1.combine(j2)


def test_document_mask_from_segment_ids():
    ids = torch.tensor([0, 0, 0, 1, 1, 2, 2, 2])
    mf, bf = masks.make_document_mask_fns(4, 4, ids)
    assert torch.equal(_dense(mf, 8), O.dense_mask(8, 8, causal=True, segment_ids=ids))
    mf2, _ = masks.make_document_mask_fns(4, 4, ids, causal=False)
    assert torch.equal(_dense(mf2, 8), O.dense_mask(8, 8, segment_ids=ids))
    with pytest.raises(NotImplementedError):
        masks.make_document_mask_fns(4, 4, torch.tensor([1, 0, 0, 1]))


def test_score_closures_match_oracle_mods():
    g = torch.Generator().manual_seed(0)
    q = torch.randn(16, 8, generator=g, dtype=torch.float64)
    k = torch.randn(16, 8, generator=g, dtype=torch.float64)
    i = torch.arange(16)[:, None]
    j = torch.arange(16)[None, :]
    s = q @ k.T
    assert torch.allclose(scores.make_softcap_score_fn(3.0)(q, k), O.score_mod_softcap(3.0)(s, 0, 0, i, j))
    assert torch.allclose(scores.make_alibi_score_fn(0.5)(q, k), O.score_mod_alibi_tile_local(0.5, 16, 16)(s, 0, 0, i, j))
    fn = scores.make_alibi_global_score_fn(4)
    ref = O.score_mod_alibi_global(O.alibi_slopes(4))(s, 0, 2, i + 32, j + 16)
    assert torch.allclose(fn(q, k, head=2, q_start=32, k_start=16), ref)
    assert fn.spec.kind == _lib.SCORE_ALIBI and len(fn.spec.slopes) == 4
    assert abs(fn.spec.slopes[0] - 2 ** (-8 / 4)) < 1e-15


def test_config_helpers_match_oracle_and_fixtures():
    with open(os.path.join(GOLDEN, "cfg5_doc_lengths.json")) as f:
        gold = json.load(f)
    for seed in range(4):
        assert configs.segment_lengths(16384, seed=seed) == gold[str(seed)] == O.make_segment_lengths(16384, seed=seed)
    c2, c4 = configs.CONFIGS["cfg2"], configs.CONFIGS["cfg4"]
    assert configs.n_pairs_per_head(c2) == 4096 * 4096 / 2
    assert configs.n_pairs_per_head(c4) == 7_872_000  # 524800 + 7168*1025
    assert abs(configs.flops_fwd(c2) - 5.498e11) / 5.498e11 < 1e-3
    a = configs.make_inputs(configs.CONFIGS["cfg1"])
    b = O.make_inputs(1, 4, 4, 512, 512, 64, dtype=torch.float32, seed=0)
    assert all(torch.equal(x, y) for x, y in zip(a, b))


def test_block_map_fixtures_match_closures():
    """Committed brute-force run-maps of the benchmark configurations == the block closures."""
    g = np.load(os.path.join(GOLDEN, "block_maps.npz"))
    for name in ("cfg2", "cfg4", "cfg5"):
        cfg = configs.CONFIGS[name]
        n = int(g[name + "_n"])
        gold = torch.from_numpy(np.unpackbits(g[name], axis=1)[:, :n].astype(bool))
        _, bf = configs.mask_fns(cfg)
        host = block_mask.host_block_map(bf, n, n)
        if name == "cfg4":  # AND of two closures is conservative
            assert bool((host | ~gold).all()) and int(host.sum()) == 540
        else:
            assert torch.equal(host, gold), name
    assert int(torch.from_numpy(np.unpackbits(g["cfg2"], axis=1)[:, :32]).sum()) == 528


def test_entry_points_validate_arguments_without_gpu():
    import flex_attention_tpu_amd as F
    q = torch.zeros(1, 2, 128, 128, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="GPU"):
        F._flex_attention_impl(q, q, q, None, None, False, False, 1.0, 1, 128, 128, 128, False, None, None, None)
    # the additive bias is checked against the shapes of q and k before anything is launched
    from flex_attention_tpu_amd._common import bias_c, check_doc_batches, resolve_mask, segment_doc_ids
    for bad in (torch.zeros(1, 2, 128, 64), torch.zeros(3, 2, 128, 128), torch.zeros(2, 128, 128)):
        with pytest.raises(ValueError, match="ab"):
            bias_c(bad, 1, 2, 128, 128, 128, 128, torch.device("cpu"))
    with pytest.raises(NotImplementedError, match="dtype"):
        bias_c(torch.zeros(1, 2, 128, 128, dtype=torch.float16), 1, 2, 128, 128, 128, 128, torch.device("cpu"))
    c, keep = bias_c(torch.zeros(1, 1, 100, 120), 2, 2, 100, 120, 128, 128, torch.device("cpu"))
    assert tuple(keep.shape) == (1, 1, 128, 128) and c.stride_b == 0 and c.stride_h == 0 and c.ptr == keep.data_ptr()
    # segment ids per batch entry: equal rows collapse into one, rows that differ stay rows of the specification
    # (the kernels take them with a batch stride), ragged lengths pad every row, and the rows must match the batch
    same = torch.zeros(2, 128, dtype=torch.int32)
    assert segment_doc_ids(same)[0].batches == 1
    ids = torch.stack([torch.zeros(100), torch.cat([torch.zeros(40), torch.ones(60)])]).to(torch.int32)
    dq, dk = segment_doc_ids(ids)
    assert dq.batches == 2 and dk is None and len(dq) == 100 and dq.is_sorted()
    r = dq.ranges_in(dq)
    assert r.shape == (2, 100, 2) and r[0, 5].tolist() == [0, 99] and r[1, 5].tolist() == [0, 39] and r[1, 50].tolist() == [40, 99]
    spec = resolve_mask(None, None, True, ids, 100, 100, 128, 128)
    assert spec.doc_ids.array.shape == (2, 128) and spec.doc_ids_k.array.shape == (2, 128)
    assert spec.doc_ids.array[1, -1] == 1 and (spec.doc_ids_k.array[:, 100:] == 2).all()   # padded keys: an id of their own
    check_doc_batches(spec, 2)
    with pytest.raises(ValueError, match="rows"):
        check_doc_batches(spec, 3)
    with pytest.raises(NotImplementedError):
        block_mask.spec_of(lambda a, b: a[:, None] >= b[None, :], None)
    from flex_attention_tpu_amd._common import check_blocks, score_spec_c
    with pytest.raises(ValueError):
        check_blocks(512, 512, block_q=100)
    with pytest.raises(ValueError):
        check_blocks(512, 512, block_k_major=256, block_k=96)
    with pytest.raises(NotImplementedError):
        score_spec_c(lambda a, b: a @ b.T, 2, "cpu", 1, 1)


def test_make_jax_score_fn_recognises_functors():
    from flex_attention_tpu_amd.util import make_jax_score_fn
    cap = 30.0
    slope = 0.25

    def softcap(q_tile, k_tile):
        logits = torch.matmul(q_tile, k_tile.T)
        return cap * torch.tanh(logits / cap)

    def alibi(q_tile, k_tile):
        mm, nn = q_tile.shape[0], k_tile.shape[0]
        dist = torch.abs(torch.arange(mm)[:, None] - torch.arange(nn)[None, :])
        return q_tile @ k_tile.T - slope * dist

    def plain(q_tile, k_tile):
        return torch.einsum("qd,kd->qk", q_tile, k_tile)

    def unsupported(q_tile, k_tile):
        return torch.softmax(q_tile @ k_tile.T, -1)

    s = make_jax_score_fn(softcap).spec
    assert s.kind == _lib.SCORE_SOFTCAP and abs(s.cap - cap) < 1e-6
    s = make_jax_score_fn(alibi).spec
    assert s.kind == _lib.SCORE_ALIBI_TILE and abs(s.slope - slope) < 1e-9
    assert make_jax_score_fn(plain).spec.kind == _lib.SCORE_NONE
    tagged = scores.make_softcap_score_fn(5.0)
    assert make_jax_score_fn(tagged) is tagged
    with pytest.raises(NotImplementedError):
        make_jax_score_fn(unsupported)


def test_tile_callable_convention_equals_score_mod_at_unit_scale():
    """The reference hands `score_fn(q_tile, k_tile)` the raw tiles and applies no sm_scale in its
    forward (flex_attention_kernel.py:249-255) nor in its dense reference (mha_reference.py:44-48);
    the kernels here compute score_mod(sm_scale * <q, k>).  At sm_scale = 1 the two coincide: the
    oracle's tile-callable path on this package's closures equals its score_mod path, forward and
    backward, for the soft-cap and the tile-local ALiBi."""
    q, k, v, do = O.make_inputs(1, 2, 2, 32, 32, 8, dtype=torch.float64, seed=5)
    for fn, mod in ((scores.make_softcap_score_fn(3.0), O.score_mod_softcap(3.0)),
                    (scores.make_alibi_score_fn(0.5), O.score_mod_alibi_tile_local(0.5, 32, 32))):
        o1, l1, m1 = O.mha_reference(q, k, v, save_residuals=True, score_fn=fn, sm_scale=0.3)  # (sm_scale is ignored here)
        o2, l2, m2 = O.mha_reference(q, k, v, save_residuals=True, score_mod=mod, sm_scale=1.0)
        assert (o1 - o2).abs().max() < 1e-12 and (l1 - l2).abs().max() < 1e-12 and (m1 - m2).abs().max() < 1e-12
        g1 = O.mha_bwd_reference(q, k, v, o1, do, l1, m1, score_fn=fn, sm_scale=1.0)
        g2 = O.mha_bwd_reference(q, k, v, o2, do, l2, m2, score_mod=mod, sm_scale=1.0)
        for a, b in zip(g1, g2):
            assert (a - b).abs().max() < 1e-11


def test_score_fn_with_non_unit_scale_warns():
    from flex_attention_tpu_amd import _common
    with pytest.warns(UserWarning, match="sm_scale"):
        _common.score_spec_c(scores.make_softcap_score_fn(3.0), 2, "cpu", 128, 128, 0.5)
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        _common.score_spec_c(scores.make_softcap_score_fn(3.0), 2, "cpu", 128, 128, 1.0)
        _common.score_spec_c(None, 2, "cpu", 128, 128, 0.5)


def test_host_caches_are_bounded():
    from flex_attention_tpu_amd import _common, block_mask
    lru = block_mask.LRU(3)
    for i in range(10):
        lru.put(i, str(i))
    assert len(lru) == 3 and lru.get(9) == "9" and lru.get(0) is None
    lru.get(7)          # 7 becomes the most recent
    lru.put(10, "10")   # drops 8
    assert lru.get(8) is None and lru.get(7) == "7"
    assert block_mask._map_cache.maxsize == block_mask.MAP_CACHE_SIZE
    # a segment-id tensor is turned into host ids once per tensor object and version
    ids = torch.tensor([0, 0, 1, 1, 2, 2, 2, 2], dtype=torch.int32)
    d1, none = _common.segment_doc_ids(ids)
    assert none is None and _common.segment_doc_ids(ids)[0] is d1
    ids[4] = 1
    d2 = _common.segment_doc_ids(ids)[0]
    assert d2 is not d1 and d2.array.tolist() == [0, 0, 1, 1, 1, 2, 2, 2]
    assert _common.segment_doc_ids(d2)[0] is d2
    # distinct, unsorted q / kv ids (the reference's SegmentIds) come back as a pair
    import types
    pair = types.SimpleNamespace(q=torch.tensor([3, 1, 1, 2]), kv=torch.tensor([1, 1, 2, 3, 3, 0]))
    dq, dk = _common.segment_doc_ids(pair)
    assert dq.array.tolist() == [3, 1, 1, 2] and dk.array.tolist() == [1, 1, 2, 3, 3, 0]
    # ragged lengths: padded keys get an id no query carries
    spec = _common.resolve_mask(None, None, True, None, 200, 300, 256, 384)
    assert spec.flags == _lib.MASK_CAUSAL | _lib.MASK_DOC
    assert spec.doc_ids.array.tolist() == [0] * 256 and spec.doc_ids_k.array.tolist() == [0] * 300 + [1] * 84


def test_ds_exchange_policy():
    """The backward hands dS from the dk/dv pass to the dq pass for softcap scores and for masks that leave many
    partial tiles, not for plain scores under no mask or a plain causal one."""
    from flex_attention_tpu_amd import masks, scores
    from flex_attention_tpu_amd.flex_attention_dq_bwd import ds_exchange_pays
    causal = masks.make_causal_mask_fns(128, 128)[0]
    assert not ds_exchange_pays(None) and not ds_exchange_pays(None, causal)
    assert not ds_exchange_pays(scores.make_alibi_global_score_fn(4), causal)
    assert ds_exchange_pays(scores.make_softcap_score_fn(30.0), causal)
    assert ds_exchange_pays(None, masks.make_causal_sliding_window_mask_fns(128, 128, 300)[0])
    assert ds_exchange_pays(None, masks.make_jagged_mask_fns(128, 128, [100, 156])[0])
    assert ds_exchange_pays(None, None, segment_ids=[0] * 128 + [1] * 128)



def test_no_compute_path_without_the_library(monkeypatch, tmp_path):
    """Without libflexattn.so the loader raises, naming the build step: nothing falls back to the CPU, and the
    package never imports the oracle (checked in a fresh interpreter, where no test has imported it)."""
    import subprocess
    import sys
    from flex_attention_tpu_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libflexattn.so"))
    with pytest.raises(ImportError, match="no other compute path"):
        _lib.load()
    code = ("import sys, flex_attention_tpu_amd as F; from flex_attention_tpu_amd import flex_attention, compiler, util, roofline; "
            "bad = [m for m in sys.modules if m == 'oracle' or m.startswith('oracle.')]; print(bad); sys.exit(1 if bad else 0)")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", code], cwd=root, capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
