"""GPU parity on the workloads of the reference's own driver scripts, with their arguments.

The reference has no test suite: each of its drivers builds one workload, runs the kernels and the dense
reference and prints a relative L2 error (main.py:44-177 forward; flex_attention_dq_bwd.py:788-946 dq;
flash_attention_dkv_bwd.py:772-940 dk/dv; the early float32 drivers reference_bwd_test.py:744-812 and
bwd_dq.py:385-478, at the end of this file, run at 1/sqrt(D)).  These tests run the same workloads through this package's entry
points with the drivers' keyword arguments -- sm_scale = 1.0 on unit-variance bf16 inputs of head dimension
128 (logits of standard deviation 11: softmax rows dominated by one or two keys, a harder regime than the
1/sqrt(D) of the benchmark configurations), blocks of 1024, batch 1 -- and compare with the oracle on sampled
rows at the stated tolerances (helpers.assert_close): rel-L2 <= 1e-2 for every tensor; o, lse and dv element by
element; dq and dk, which reach magnitudes of 25 to 40 here, against the bound of the tensor's largest magnitude
(`tensor_scale`).  Inputs come from this build's seeded generator (the reference's JAX PRNG streams are not
reproducible without JAX).

At this scale the library runs the forward and dq on kernels that scale the fp32 product (dq with plain scores: the
exact-scale variant of its generated stream; the forward, and dq under the position bias and softcap: the kernels
with a compiled main loop):
the ordinary streams fold the scale into their bf16 copy of Q, which costs logits of this size their accuracy (o off
by 0.06, dq by 2 % in relative L2 when measured), so these tests also pin that choice: they fail on those.

Differences from the drivers, on purpose: the backward takes the residuals of the forward under the same mask
(the drivers feed the residuals of an unmasked forward to masked backward kernels; the one test of that habit
below is test_backward_from_the_residuals_of_an_unmasked_forward), and the position-bias case is compared with
the oracle's tile-local bias, which is what the reference's score function computes on a tile
(scores.py:3-11), not with the global bias of its dense reference.
"""
import numpy as np
import pytest
import torch

from helpers import assert_close, same_residual_grads
from oracle import mha_oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda"
BLOCK = 1024      # block_q = block_k_major = block_k of the drivers
SM_SCALE = 1.0


@pytest.fixture(scope="module")
def F():
    import flex_attention_tpu_amd as F
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return F


def driver_doc_lengths(total_len, num_docs, seed):
    """Document lengths as the dk/dv driver draws them (flash_attention_dkv_bwd.py:747-770): num_docs - 1 distinct
    cut points from numpy's legacy generator."""
    np.random.seed(seed)
    cuts = np.sort(np.random.choice(range(1, total_len), num_docs - 1, replace=False))
    return [int(n) for n in np.diff(np.concatenate(([0], cuts, [total_len])))]


def _driver_cases(S):
    """(name, (mask_fn, block_mask_fn), score_fn, oracle keywords) of the drivers' case lists."""
    from flex_attention_tpu_amd import masks, scores
    lens = driver_doc_lengths(S, 5, 42)
    return {
        "causal": (masks.make_causal_mask_fns(BLOCK, BLOCK), None, dict(causal=True)),
        "sliding_window_1024": (masks.make_sliding_window_mask_fns(BLOCK, BLOCK, 1024), None, dict(window_size=1024)),
        "jagged_5_docs": (masks.make_jagged_mask_fns(BLOCK, BLOCK, lens), None,
                          dict(causal=True, segment_ids=O.doc_ids_from_lengths(lens))),
        "alibi_0.5": ((None, None), scores.make_alibi_score_fn(slope=0.5),
                      dict(score_mod=O.score_mod_alibi_tile_local(0.5, BLOCK, BLOCK))),
        "tanh_30": ((None, None), scores.make_softcap_score_fn(cap=30.0), dict(score_mod=O.score_mod_softcap(30.0))),
    }


def _run_all(F, q, k, v, do, mf, bf, sfn, fwd_masks=None, BLOCK=BLOCK):
    """Forward, delta, dq and dk/dv with the drivers' keyword arguments.  `fwd_masks`: another mask pair for the
    forward than for the backward."""
    fm, fb = (mf, bf) if fwd_masks is None else fwd_masks
    o, l, m = F._flex_attention_impl(q, k, v, None, None, True, False, SM_SCALE, 1, BLOCK, BLOCK, BLOCK, False, fb, fm, sfn)
    d = F.compute_delta(o, do)
    dq = F.flex_attention_bwd_dq(q, k, v, None, None, l, m, o, do, d, block_b=1, block_q=BLOCK, block_k_major=BLOCK,
                                 block_k=BLOCK, sm_scale=SM_SCALE, debug=False, score_fn=sfn, mask_fn=mf, block_mask_fn=bf)
    dk, dv = F.flash_attention_bwd_dkv(k, v, q, None, None, l, m, d, do, block_b=1, block_q=BLOCK, block_q_major=BLOCK,
                                       block_k_major=BLOCK, block_k=BLOCK, sm_scale=SM_SCALE, causal=False, debug=False,
                                       score_fn=sfn, mask_fn=mf, block_mask_fn=bf)
    torch.cuda.synchronize()
    return o, l, m, dq, dk, dv


def _sample_rows(S, n):
    g = torch.Generator().manual_seed(11)
    rows = torch.sort(torch.randperm(S, generator=g)[:n]).values
    rows[0], rows[-1] = 0, S - 1
    return rows


@pytest.mark.parametrize("case", ["causal", "jagged_5_docs"])
def test_unit_scale_small_shapes(F, case):
    """sm_scale = 1.0 at a size where every element is compared: B = 2, H = 2, S = 512 (the exact-scale variant of the
    dq stream kernel, which serves plain scores at this scale, on single- and multi-step items with partial
    tiles)."""
    from flex_attention_tpu_amd import masks
    S = 512
    if case == "causal":
        (mf, bf), okw = masks.make_causal_mask_fns(128, 128), dict(causal=True)
    else:
        lens = driver_doc_lengths(S, 5, 42)
        (mf, bf), okw = masks.make_jagged_mask_fns(128, 128, lens), dict(causal=True, segment_ids=O.doc_ids_from_lengths(lens))
    q, k, v, do = O.make_inputs(2, 2, 2, S, S, 128, dtype=torch.bfloat16, seed=3)
    ro, rl, rm = O.mha_reference(q, k, v, sm_scale=SM_SCALE, save_residuals=True, **okw)
    o, l, m, dq, dk, dv = _run_all(F, q.to(DEV), k.to(DEV), v.to(DEV), do.to(DEV), mf, bf, None, BLOCK=128)
    sdq, sdk, sdv = same_residual_grads(q, k, v, do, o, l, m, sm_scale=SM_SCALE, **okw)
    assert_close("o", o, ro, torch.bfloat16)
    assert_close("lse", m + l.log(), rm + rl.log(), torch.bfloat16)
    assert_close("dq", dq, sdq, torch.bfloat16, tensor_scale=True)
    assert_close("dk", dk, sdk, torch.bfloat16, tensor_scale=True)
    assert_close("dv", dv, sdv, torch.bfloat16)


def test_forward_driver_workload(F):
    """main.py:44-177: bf16, B = 1, H = 1, S = 16384, D = 128, blocks 1024, the place-holder mask (the only live
    case of the list), sm_scale = 1.0 (main.py:155)."""
    from flex_attention_tpu_amd import masks
    S = 16384
    q, k, v, _ = O.make_inputs(1, 1, 1, S, S, 128, dtype=torch.bfloat16, seed=0)
    mf, bf = masks.place_holder(BLOCK, BLOCK)
    rows = _sample_rows(S, 256)
    ro, rl, rm = O.mha_reference(q, k, v, sm_scale=SM_SCALE, save_residuals=True, q_rows=rows, compute_dtype=torch.float32)
    o, l, m = F._flex_attention_impl(q.to(DEV), k.to(DEV), v.to(DEV), None, None, True, False, SM_SCALE, 1, BLOCK, BLOCK,
                                     BLOCK, False, bf, mf, None)
    dr = rows.to(DEV)
    assert_close("o", o[:, :, dr], ro, torch.bfloat16)
    assert_close("lse", (m + l.log())[:, :, dr], rm + rl.log(), torch.bfloat16)


@pytest.mark.parametrize("case", ["causal", "sliding_window_1024", "jagged_5_docs", "alibi_0.5", "tanh_30"])
def test_backward_driver_workloads(F, case):
    """flex_attention_dq_bwd.py:788-946 and flash_attention_dkv_bwd.py:772-940: bf16, B = 1, H = 8, S = 4096,
    D = 128, blocks 1024, sm_scale = 1.0; cases causal, sliding window 1024 (one-sided, no causal bound), five
    documents drawn with seed 42 (the dk/dv driver's), the tile-local position bias of slope 0.5 and softcap 30,
    the last two without a mask.  All passes on two heads' sampled rows against the oracle."""
    S, H = 4096, 8
    (mf, bf), sfn, okw = _driver_cases(S)[case]
    q, k, v, do = O.make_inputs(1, H, H, S, S, 128, dtype=torch.bfloat16, seed=0)
    rows = _sample_rows(S, 192)
    heads = [(0, 0), (0, 7)]
    ro, rl, rm = O.mha_reference(q, k, v, sm_scale=SM_SCALE, save_residuals=True, q_rows=rows, heads=heads,
                                 compute_dtype=torch.float32, **okw)
    do_s = torch.zeros_like(do)   # (dk, dv are linear in dO: rows outside the sample contribute nothing)
    do_s[:, :, rows] = do[:, :, rows]
    o, l, m, dq, dk, dv = _run_all(F, q.to(DEV), k.to(DEV), v.to(DEV), do_s.to(DEV), mf, bf, sfn)
    sdq, sdk, sdv = same_residual_grads(q, k, v, do_s, o, l, m, sm_scale=SM_SCALE, q_rows=rows, heads=heads,
                                        compute_dtype=torch.float32, **okw)
    dr = rows.to(DEV)
    for (b, h) in heads:
        assert_close(f"o[{h}]", o[b, h, dr], ro[b, h], torch.bfloat16)
        assert_close(f"lse[{h}]", (m + l.log())[b, h, dr], (rm + rl.log())[b, h], torch.bfloat16)
        assert_close(f"dq[{h}]", dq[b, h, dr], sdq[b, h], torch.bfloat16, tensor_scale=True)
        assert_close(f"dk[{h}]", dk[b, h], sdk[b, h], torch.bfloat16, tensor_scale=True)
        assert_close(f"dv[{h}]", dv[b, h], sdv[b, h], torch.bfloat16)


def test_backward_from_the_residuals_of_an_unmasked_forward(F):
    """The drivers hand (o, l, m) of an unmasked forward to backward kernels that run under the causal mask
    (flex_attention_dq_bwd.py:920-926, flash_attention_dkv_bwd.py:913-919): P is then no softmax, but the
    backward kernels are functions of (l, m, delta) as given, and the dense reference gets the same ones."""
    from flex_attention_tpu_amd import masks
    S, H = 4096, 8
    (mf, bf), _, okw = _driver_cases(S)["causal"]
    q, k, v, do = O.make_inputs(1, H, H, S, S, 128, dtype=torch.bfloat16, seed=0)
    rows = _sample_rows(S, 192)
    heads = [(0, 3)]
    do_s = torch.zeros_like(do)
    do_s[:, :, rows] = do[:, :, rows]
    o, l, m, dq, dk, dv = _run_all(F, q.to(DEV), k.to(DEV), v.to(DEV), do_s.to(DEV), mf, bf, None,
                                   fwd_masks=masks.place_holder(BLOCK, BLOCK))
    sdq, sdk, sdv = same_residual_grads(q, k, v, do_s, o, l, m, sm_scale=SM_SCALE, q_rows=rows, heads=heads,
                                        compute_dtype=torch.float32, **okw)
    dr = rows.to(DEV)
    assert_close("dq", dq[0, 3, dr], sdq[0, 3], torch.bfloat16, tensor_scale=True)
    assert_close("dk", dk[0, 3], sdk[0, 3], torch.bfloat16, tensor_scale=True)
    assert_close("dv", dv[0, 3], sdv[0, 3], torch.bfloat16)


def _fp32_all(F, q, k, v, do, bq, bkm, bk):
    sc = 1.0 / float(np.sqrt(np.float32(128)))
    o, l, m = F._flex_attention_impl(q, k, v, None, None, True, False, sc, 1, bq, bkm, bk, False, None, None, None)
    d = F.compute_delta(o, do)
    dq = F.flex_attention_bwd_dq(q, k, v, None, None, l, m, o, do, d, block_b=1, block_q=bq, block_k_major=bkm,
                                 block_k=bk, sm_scale=sc, debug=False)
    dk, dv = F.flash_attention_bwd_dkv(k, v, q, None, None, l, m, d, do, block_b=1, block_q=bq, block_q_major=bq,
                                       block_k_major=bkm, block_k=bk, sm_scale=sc, causal=False, debug=False)
    torch.cuda.synchronize()
    return sc, o, l, m, dq, dk, dv


def test_fp32_cross_attention_driver_workload(F):
    """bwd_dq.py:385-478: float32, B = H = 1, 128 queries against 25600 keys, D = 128, sm_scale = 1/sqrt(D), no mask,
    block_q 128, block_k 256.  Every element against the float64 oracle at 1e-5."""
    q, k, v, do = O.make_inputs(1, 1, 1, 128, 25600, 128, dtype=torch.float32, seed=0)
    sc, o, l, m, dq, dk, dv = _fp32_all(F, q.to(DEV), k.to(DEV), v.to(DEV), do.to(DEV), 128, 256, 256)
    ro, rl, rm = O.mha_reference(q, k, v, sm_scale=sc, save_residuals=True)
    rdq, rdk, rdv = O.mha_bwd_reference(q, k, v, ro, do, rl, rm, sm_scale=sc)
    assert_close("o", o, ro, torch.float32)
    assert_close("lse", m + l.log(), rm + rl.log(), torch.float32)
    for name, t, r in (("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv)):
        assert_close(name, t, r, torch.float32, chain=True)


def test_fp32_long_sequence_driver_workload(F):
    """reference_bwd_test.py:744-812: float32, B = H = 1, S = 16384, D = 128, sm_scale = 1/sqrt(D), no mask, block_q
    128, block_k 128.  Sampled rows against the float64 oracle at 1e-5 (dk, dv with dO zeroed outside the sample)."""
    S = 16384
    q, k, v, do = O.make_inputs(1, 1, 1, S, S, 128, dtype=torch.float32, seed=0)
    rows = _sample_rows(S, 192)
    do_s = torch.zeros_like(do)
    do_s[:, :, rows] = do[:, :, rows]
    sc, o, l, m, dq, dk, dv = _fp32_all(F, q.to(DEV), k.to(DEV), v.to(DEV), do_s.to(DEV), 128, 128, 128)
    ro, rl, rm = O.mha_reference(q, k, v, sm_scale=sc, save_residuals=True, q_rows=rows)
    rdq, rdk, rdv = O.mha_bwd_reference(q, k, v, ro, do_s[:, :, rows], rl, rm, sm_scale=sc, q_rows=rows)
    dr = rows.to(DEV)
    assert_close("o", o[:, :, dr], ro, torch.float32)
    assert_close("lse", (m + l.log())[:, :, dr], rm + rl.log(), torch.float32)
    assert_close("dq", dq[:, :, dr], rdq, torch.float32, chain=True)
    assert_close("dk", dk, rdk, torch.float32, chain=True)
    assert_close("dv", dv, rdv, torch.float32, chain=True)
