"""GPU parity of closures compiled into the kernels (compiler.py): arbitrary Python score and mask
functions, transpiled to HIP functors, against the CPU oracle evaluating the same Python functions.
The functor libraries are built ahead of the run (custom_functors.prebuild, called by the build step)."""
import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import custom_functors as cf  # noqa: E402
from helpers import assert_close, same_residual_grads  # noqa: E402
from oracle import mha_oracle as O  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def F():
    import flex_attention_tpu_amd as F
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return F


@pytest.fixture(scope="module")
def compiled():
    return cf.compiled()


def _oracle_kwargs(name, Sq, Sk):
    """Oracle keywords: the Python functions themselves (score_mod on tensors, dense mask from mask_fn)."""
    kw = {}
    parts = name.split("+")
    mods = {"alibi_mod": cf.alibi_mod, "softcap_mod": cf.softcap_mod, "mixed_mod": cf.mixed_mod,
            "alibi_symmetric_mod": cf.alibi_symmetric_mod, "elementary_mod": cf.elementary_mod}
    masks = {"prefix_lm": cf.prefix_lm_mask, "checker": cf.checker_mask}
    for p in parts:
        if p in mods:
            kw["score_mod"] = mods[p]
        if p in masks:
            kw["mask"] = masks[p](torch.arange(Sq), torch.arange(Sk))
    return kw


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "fp32"])
@pytest.mark.parametrize("name", ["alibi_mod", "softcap_mod", "mixed_mod", "alibi_symmetric_mod", "elementary_mod", "prefix_lm",
                                  "checker", "mixed_mod+prefix_lm"])
def test_compiled_closures_all_passes(F, compiled, name, dtype):
    _closures_all_passes(F, compiled, name, dtype, 128)


@pytest.mark.parametrize("name", ["alibi_mod", "mixed_mod+prefix_lm"])
def test_compiled_closures_head_dimension_256(F, compiled, name):
    """The functor libraries hold the bf16 kernels of head dimension 256 as well."""
    _closures_all_passes(F, compiled, name, torch.bfloat16, 256)


def test_closures_that_equal_a_builtin_functor_run_its_kernels(F):
    """Closures the compiler recognises (a soft-cap, global ALiBi with slopes computed from the head's index, a
    causal window) carry the specifications of this package's own factories: the calls give the bits of the
    factories' closures (the generated-stream kernels on a closed-form block map) and need no functor library."""
    from flex_attention_tpu_amd import compiler, masks, scores
    B, Hq, Hkv, S = 2, 4, 4, 1024
    sc = 1 / math.sqrt(128)
    q, k, v, do = [x.to(DEV) for x in O.make_inputs(B, Hq, Hkv, S, S, 128, dtype=torch.bfloat16, seed=73)]
    mask_c = compiler.compile_mask_fn(cf.causal_window_mask, 128, 128)
    mask_b = masks.make_causal_sliding_window_mask_fns(128, 128, 200)
    assert mask_c[0].spec == mask_b[0].spec
    for closure, factory in ((cf.softcap30_mod, scores.make_softcap_score_fn(30.0)),
                             (cf.alibi_formula_mod, scores.make_alibi_global_score_fn(Hq))):
        sfn = compiler.compile_score_mod(closure)
        assert sfn.spec.custom is None and sfn.spec.kind == factory.spec.kind
        results = []
        for score_fn, (mf, bf) in ((sfn, mask_c), (factory, mask_b)):
            o, l, m = F._flex_attention_impl(q, k, v, None, None, True, False, sc, 1, 128, 128, 128, False, bf, mf, score_fn)
            grads = F.flex_attention_bwd(q, k, v, None, None, l, m, o, do, block_q=128, block_k=128, sm_scale=sc,
                                         score_fn=score_fn, mask_fn=mf, block_mask_fn=bf)
            results.append((o, l, m, *grads))
        for name, a, b in zip(("o", "l", "m", "dq", "dk", "dv"), *results):
            assert torch.equal(a, b), f"{closure.__name__}: {name} differs from the factory's"
        ro = O.mha_reference(q.cpu(), k.cpu(), v.cpu(), sm_scale=sc, causal=True, window_size=200,
                             score_mod=lambda s, b, h, i, j, f=closure: f(s, b, h, i, j))
        assert_close(closure.__name__ + " o", results[0][0], ro, torch.bfloat16)


def test_autograd_through_a_compiled_closure(F, compiled):
    """torch.autograd.grad through flex_attention with a compiled score function and a compiled mask: the backward
    hands dS from the dk/dv pass to the dq pass by itself (the score function is evaluated in one backward pass)."""
    name = "mixed_mod+prefix_lm"
    score_fn, mask_pair = compiled[name]
    B, Hq, Hkv, S = 2, 4, 2, 512
    sc = 1 / math.sqrt(128)
    q, k, v, do = O.make_inputs(B, Hq, Hkv, S, S, 128, dtype=torch.bfloat16, seed=67)
    okw = dict(sm_scale=sc, **_oracle_kwargs(name, S, S))
    ro, rl, rm = O.mha_reference(q, k, v, save_residuals=True, **okw)
    rdq, rdk, rdv = O.mha_bwd_reference(q, k, v, ro, do, rl, rm, **okw)
    qg, kg, vg = [x.to(DEV).requires_grad_(True) for x in (q, k, v)]
    o = F.flex_attention(qg, kg, vg, score_fn, mask_pair, sm_scale=sc)
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), do.to(DEV))
    assert_close("o", o, ro, torch.bfloat16)
    for nm, t, c in zip(("dq", "dk", "dv"), (dq, dk, dv), (rdq, rdk, rdv)):
        assert_close(nm + " chain", t, c, torch.bfloat16, chain=True)
    from flex_attention_tpu_amd.flex_attention_dq_bwd import ds_exchange_pays
    assert ds_exchange_pays(score_fn, mask_pair[0])


def test_plain_python_closures_through_the_entry_points(F):
    """Plain Python functions handed to the entry points and to flex_attention themselves (no factory, no explicit
    compile step), as the reference's callers hand theirs to its kernels: these two are recognised, so the calls
    give the bits of the factories' closures."""
    from flex_attention_tpu_amd import masks, scores
    B, Hq, Hkv, S = 1, 4, 2, 768
    sc = 1 / math.sqrt(128)
    q, k, v, do = [x.to(DEV) for x in O.make_inputs(B, Hq, Hkv, S, S, 128, dtype=torch.bfloat16, seed=79)]
    fm, fs = masks.make_causal_sliding_window_mask_fns(128, 128, 200), scores.make_softcap_score_fn(30.0)
    want = F._flex_attention_impl(q, k, v, None, None, True, False, sc, 1, 128, 128, 128, False, fm[1], fm[0], fs)
    got = F._flex_attention_impl(q, k, v, None, None, True, False, sc, 1, 128, 128, 128, False, None, cf.causal_window_mask,
                                 cf.softcap30_mod)
    for name, a, b in zip(("o", "l", "m"), got, want):
        assert torch.equal(a, b), name
    o, l, m = want
    d = F.compute_delta(o, do)
    kw = dict(block_b=1, block_q=128, block_k_major=128, block_k=128, sm_scale=sc, debug=False)
    dq = F.flex_attention_bwd_dq(q, k, v, None, None, l, m, o, do, d, score_fn=cf.softcap30_mod, mask_fn=cf.causal_window_mask, **kw)
    dk, dv = F.flash_attention_bwd_dkv(k, v, q, None, None, l, m, d, do, block_q_major=128, causal=False,
                                       score_fn=cf.softcap30_mod, mask_fn=cf.causal_window_mask, **kw)
    assert torch.equal(dq, F.flex_attention_bwd_dq(q, k, v, None, None, l, m, o, do, d, score_fn=fs, mask_fn=fm[0],
                                                   block_mask_fn=fm[1], **kw))
    wk, wv = F.flash_attention_bwd_dkv(k, v, q, None, None, l, m, d, do, block_q_major=128, causal=False, score_fn=fs,
                                       mask_fn=fm[0], block_mask_fn=fm[1], **kw)
    assert torch.equal(dk, wk) and torch.equal(dv, wv)
    qa = q.clone().requires_grad_(True)
    oa = F.flex_attention(qa, k, v, cf.softcap30_mod, cf.causal_window_mask, sm_scale=sc)
    assert torch.equal(oa.detach(), o)
    (ga,) = torch.autograd.grad(oa, (qa,), do)
    assert torch.equal(ga, dq)


def _closures_all_passes(F, compiled, name, dtype, D):
    score_fn, mask_pair = compiled[name]
    B, Hq, Hkv, S = 2, 4, 2, 512
    sc = 1 / math.sqrt(D)
    q, k, v, do = O.make_inputs(B, Hq, Hkv, S, S, D, dtype=dtype, seed=61)
    from flex_attention_tpu_amd import masks
    okw = dict(sm_scale=sc, causal=(name == "alibi_mod"), **_oracle_kwargs(name, S, S))
    ro, rl, rm = O.mha_reference(q, k, v, save_residuals=True, **okw)
    rdq, rdk, rdv = O.mha_bwd_reference(q, k, v, ro, do, rl, rm, **okw)
    mf, bf = mask_pair if mask_pair else (None, None)
    if name == "alibi_mod":   # (a compiled score under a built-in mask)
        mf, bf = masks.make_causal_mask_fns(128, 128)
    qg, kg, vg, dog = [x.to(DEV) for x in (q, k, v, do)]
    o, l, m = F._flex_attention_impl(qg, kg, vg, None, None, True, False, sc, 1, 128, 128, 128, False, bf, mf, score_fn)
    assert_close("o", o, ro, dtype)
    assert_close("lse", m + l.log(), rm + rl.log(), dtype)
    d = F.compute_delta(o, dog)
    dq = F.flex_attention_bwd_dq(qg, kg, vg, None, None, l, m, o, dog, d, block_b=1, block_q=128, block_k_major=128,
                                 block_k=128, sm_scale=sc, debug=False, score_fn=score_fn, mask_fn=mf, block_mask_fn=bf)
    dk, dv = F.flash_attention_bwd_dkv(kg, vg, qg, None, None, l, m, d, dog, block_b=1, block_q=128, block_q_major=128,
                                       block_k_major=128, block_k=128, sm_scale=sc, causal=False, debug=False,
                                       score_fn=score_fn, mask_fn=mf, block_mask_fn=bf)
    same = same_residual_grads(q, k, v, do, o, l, m, **okw)
    for nm, t, r, c in zip(("dq", "dk", "dv"), (dq, dk, dv), same, (rdq, rdk, rdv)):
        assert_close(nm, t, r, dtype)
        assert_close(nm + " chain", t, c, dtype, chain=True)
    # the backward that hands dS from the dk/dv pass to the dq pass (bf16 at head dimension 128): the same dk, dv,
    # and a dq for which no score function is evaluated a second time; a compiled mask alone runs the streams
    kw = dict(block_b=1, block_q=128, block_k_major=128, block_k=128, sm_scale=sc, debug=False, score_fn=score_fn,
              mask_fn=mf, block_mask_fn=bf)
    dk2, dv2, ds = F.flash_attention_bwd_dkv(kg, vg, qg, None, None, l, m, d, dog, block_q_major=128, causal=False,
                                             return_ds=True, **kw)
    assert torch.equal(dk2, dk) and torch.equal(dv2, dv), "dk, dv change when dS is exported"
    assert (ds is not None) == (dtype == torch.bfloat16 and D == 128)
    if ds is not None:
        dqx = F.flex_attention_bwd_dq(qg, kg, vg, None, None, l, m, o, dog, d, ds=ds, **kw)
        assert_close("dq from dS", dqx, same[0], dtype)
        assert_close("dq from dS chain", dqx, rdq, dtype, chain=True)


def test_compiled_alibi_equals_the_builtin_functor(F, compiled):
    """The hand-written global ALiBi, compiled, against the built-in functor (generated-stream kernels)."""
    from flex_attention_tpu_amd import masks, scores
    sc = 1 / math.sqrt(128)
    q, k, v, _ = O.make_inputs(1, 4, 4, 512, 512, 128, dtype=torch.bfloat16, seed=67)
    q, k, v = [x.to(DEV) for x in (q, k, v)]
    mf, bf = masks.make_causal_mask_fns(128, 128)
    a = F._flex_attention_impl(q, k, v, None, None, True, False, sc, 1, 128, 128, 128, False, bf, mf, compiled["alibi_mod"][0])
    b = F._flex_attention_impl(q, k, v, None, None, True, False, sc, 1, 128, 128, 128, False, bf, mf,
                               scores.make_alibi_global_score_fn(4, cf.SLOPES))
    assert O.rel_l2(a[0], b[0].float().cpu()) <= 5e-3
    assert float(((a[2] + a[1].log()) - (b[2] + b[1].log())).abs().max()) <= 1e-2


@pytest.mark.parametrize("name", ["prefix_lm", "checker"])
def test_compiled_mask_block_map_bit_exact(F, compiled, name):
    """state != 0 of the GPU builder equals the block closure (any(mask_fn over the tile)) bit for bit, state
    equals the brute-force map, at the kernels' granularities."""
    from flex_attention_tpu_amd import block_mask, compiler
    fn = {"prefix_lm": cf.prefix_lm_mask, "checker": cf.checker_mask}[name]
    S = 1024
    dense = fn(torch.arange(S), torch.arange(S))
    for bq, bk in ((128, 64), (64, 128), (64, 64)):
        mf, bf = compiler.compile_mask_fn(fn, bq, bk)
        bm = block_mask.create_block_mask((mf, bf), S, S, bq, bk, DEV)
        state = bm.state.cpu()
        assert torch.equal(state, O.block_map_bruteforce(dense, bq, bk))
        assert torch.equal(state != 0, block_mask.host_block_map(bf, S // bq, S // bk))


@pytest.mark.parametrize("name", ["squared_tile", "tile_local_distance"])
def test_tile_form_functions_through_make_jax_score_fn(F, compiled, name):
    """The reference's tile form f(q_tile, k_tile) through util.make_jax_score_fn (sm_scale = 1, where the
    reference's conventions agree): forward and gradients against the oracle's tile-callable path."""
    fn = {"squared_tile": cf.squared_tile, "tile_local_distance": cf.tile_local_distance}[name]
    score_fn = compiled[name][0]
    S = 256
    q, k, v, do = O.make_inputs(1, 2, 2, S, S, 128, dtype=torch.float32, seed=71)
    q, do = q * 0.1, do * 0.1   # (sm_scale is 1 here: keeps logits and gradients of order one)
    # the oracle calls the function on whole [S, 128] x [S, 128] tiles: tile-local indices then span 128 rows /
    # columns only if the function is evaluated tile by tile, as the kernels do (block_q = block_k = 128)
    def tiled(qt, kt):
        rows = [torch.cat([fn(qt[a:a + 128], kt[b:b + 128]) for b in range(0, kt.shape[0], 128)], dim=1)
                for a in range(0, qt.shape[0], 128)]
        return torch.cat(rows, dim=0)
    ro, rl, rm = O.mha_reference(q, k, v, save_residuals=True, score_fn=tiled)
    rdq, rdk, rdv = O.mha_bwd_reference(q, k, v, ro, do, rl, rm, score_fn=tiled)
    qg, kg, vg, dog = [x.to(DEV) for x in (q, k, v, do)]
    o, l, m = F._flex_attention_impl(qg, kg, vg, None, None, True, False, 1.0, 1, 128, 128, 128, False, None, None, score_fn)
    d = F.compute_delta(o, dog)
    dq = F.flex_attention_bwd_dq(qg, kg, vg, None, None, l, m, o, dog, d, block_b=1, block_q=128, block_k_major=128,
                                 block_k=128, sm_scale=1.0, debug=False, score_fn=score_fn)
    dk, dv = F.flash_attention_bwd_dkv(kg, vg, qg, None, None, l, m, d, dog, block_b=1, block_q=128, block_q_major=128,
                                       block_k_major=128, block_k=128, sm_scale=1.0, causal=False, debug=False, score_fn=score_fn)
    for nm, t, r in (("o", o, ro), ("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv)):
        assert_close(nm, t, r, torch.float32)


def test_plain_library_refuses_compiled_closures(F):
    """libflexattn.so itself holds no compiled closure: a CUSTOM kind handed to it is ENOTSUP."""
    import ctypes as C
    from flex_attention_tpu_amd import _lib
    lib = _lib.load()
    m = _lib.MaskSpecC(_lib.MASK_CUSTOM, 0, 0, 0, None, None)
    st = torch.empty(4, 4, dtype=torch.uint8, device=DEV)
    rc = lib.flexattn_build_block_mask(C.byref(m), 512, 512, 128, 128, st.data_ptr(), None, None, None, None, None)
    assert rc == _lib.ENOTSUP and b"compiled mask" in lib.flexattn_last_error_string()
