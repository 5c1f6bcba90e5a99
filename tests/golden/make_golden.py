"""Writes the committed fixtures of tests/golden (run from the repository root):

    python tests/golden/make_golden.py

* oracle_tiny.npz   float64 inputs and oracle outputs/gradients of a tiny GQA + softcap + document
                    + causal case: a regression vector for the oracle itself.  Its values were
                    cross-checked at generation time against torch.autograd of an independent
                    dense softmax (asserted below), not merely produced by the oracle.
* block_maps.npz    run-maps (bit-packed) of the five benchmark configurations at 128x128 blocks,
                    computed by brute force ``any(mask over tile)`` from the element masks.
* cfg5_doc_lengths.json  document lengths of configuration 5 for seeds 0..3.

The reference repository holds no golden vectors for this path and cannot be executed (JAX is
not installed), so these fixtures are produced by this build's oracle and pinned by the
independent checks in tests/test_oracle.py.
"""
import json
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import mha_oracle as O  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def tiny():
    B, Hq, Hkv, S, D = 1, 4, 2, 24, 8
    q, k, v, do = O.make_inputs(B, Hq, Hkv, S, S, D, dtype=torch.float64, seed=123)
    lens = [7, 9, 8]
    sid = O.doc_ids_from_lengths(lens)
    cap, sc = 2.5, 0.6
    kw = dict(sm_scale=sc, causal=True, segment_ids=sid, score_mod=O.score_mod_softcap(cap))
    o, l, m = O.mha_reference(q, k, v, save_residuals=True, **kw)
    dq, dk, dv = O.mha_bwd_reference(q, k, v, o, do, l, m, **kw)
    # independent cross-check before committing the numbers
    qd, kd, vd = [x.clone().requires_grad_() for x in (q, k, v)]
    i = torch.arange(S)[:, None]
    j = torch.arange(S)[None, :]
    keep = (j <= i) & (sid[:, None] == sid[None, :])
    outs = []
    for h in range(Hq):
        s = cap * torch.tanh((qd[0, h] @ kd[0, h // 2].T) * sc / cap)
        outs.append(torch.softmax(s.masked_fill(~keep, float("-inf")), -1) @ vd[0, h // 2])
    r = torch.stack(outs)[None]
    gq, gk, gv = torch.autograd.grad(r, (qd, kd, vd), do)
    assert (r - o).abs().max() < 1e-12
    for a, b in ((dq, gq), (dk, gk), (dv, gv)):
        assert (a - b).abs().max() < 1e-11
    np.savez(os.path.join(HERE, "oracle_tiny.npz"), q=q.numpy(), k=k.numpy(), v=v.numpy(), do=do.numpy(),
             segment_ids=sid.numpy(), sm_scale=sc, cap=cap, o=o.numpy(), l=l.numpy(), m=m.numpy(),
             dq=dq.numpy(), dk=dk.numpy(), dv=dv.numpy())


def block_maps():
    out = {}
    blk = 128
    cases = {
        "cfg1": (512, {}),
        "cfg2": (4096, dict(causal=True)),
        "cfg4": (8192, dict(causal=True, window_size=1025)),
        "cfg5": (16384, dict(causal=True, segment_ids=O.doc_ids_from_lengths(O.make_segment_lengths(16384, seed=0)))),
    }
    for name, (S, kw) in cases.items():
        n = S // blk
        run = torch.zeros(n, n, dtype=torch.bool)
        for qb in range(n):
            keep = O.dense_mask(S, S, q_offset=qb * blk, q_len=blk, **kw)
            run[qb] = keep.reshape(blk, n, blk).any(dim=2).any(dim=0)
        out[name] = np.packbits(run.numpy(), axis=1)
        out[name + "_n"] = np.int64(n)
    np.savez(os.path.join(HERE, "block_maps.npz"), **out)


def doc_lengths():
    with open(os.path.join(HERE, "cfg5_doc_lengths.json"), "w") as f:
        json.dump({str(s): O.make_segment_lengths(16384, seed=s) for s in range(4)}, f)


if __name__ == "__main__":
    tiny()
    block_maps()
    doc_lengths()
    print("wrote fixtures to", HERE)
