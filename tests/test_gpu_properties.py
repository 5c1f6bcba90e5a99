"""Size-independent properties of the kernels at the full sizes of the benchmark configurations, where the oracle
only reaches sampled rows and single heads: every output element of the full launch takes part, bit for bit.

* Determinism: the same call twice gives the same bits (every output tile has one writer and a fixed order of
  accumulation; nothing depends on which work-group runs an item, or when).
* Equivariance: permuting the batch entries (and, where the score function does not depend on the head, the kv
  groups of heads) permutes the outputs and changes no bit.  The persistent work-groups then run the same items in
  another order, next to other items and with other prefetched neighbours: state that leaks from one item into
  the next, or a schedule that visits an item twice or not at all, shows here on every element.
* Homogeneity: scaling dO (or v) by two doubles dq, dk, dv (or o) exactly: delta, dP and dS double without rounding
  (powers of two), so the bf16 results are the doubled bf16 results.
* No gradient without dO: dO = 0 gives dq = dk = dv = 0.
* Locality: a (batch entry, kv group) launched alone gives its bits of the full launch (one item per work-group
  against the persistent schedule); under a causal mask the first half of the tokens alone gives the first half of
  o, l, m and dq.
* Grouped kv heads give, per query head, the bits of the same call with the kv heads repeated.
* Segment ids with a row per batch entry: permuting the entries together with their rows permutes the outputs, and
  an entry launched alone with its row gives its bits of the batch.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda"


@pytest.fixture(scope="module")
def F():
    import flex_attention_tpu_amd as F
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return F


def _calls(F, cfg):
    from flex_attention_tpu_amd import configs
    import warnings
    warnings.filterwarnings("ignore", message="score_fn with sm_scale")
    mf, bf = configs.mask_fns(cfg)
    sfn = configs.score_fn(cfg)
    sc = cfg.sm_scale

    def fwd(q, k, v):
        return F._flex_attention_impl(q, k, v, None, None, True, False, sc, 1, 128, 128, 128, False, bf, mf, sfn)

    def bwd(q, k, v, o, l, m, do):
        return F.flex_attention_bwd(q, k, v, None, None, l, m, o, do, block_q=128, block_k=128, sm_scale=sc, score_fn=sfn,
                                    mask_fn=mf, block_mask_fn=bf)

    def bwd_exchanging(q, k, v, o, l, m, do):
        """The backward with dS handed from the dk/dv pass to the dq pass (None where nothing is exchanged)."""
        d = F.compute_delta(o, do)
        dk, dv, ds = F.flash_attention_bwd_dkv(k, v, q, None, None, l, m, d, do, block_b=1, block_q=128, block_q_major=128,
                                               block_k_major=128, block_k=128, sm_scale=sc, causal=False, debug=False,
                                               score_fn=sfn, mask_fn=mf, block_mask_fn=bf, return_ds=True)
        if ds is None:
            return None
        dq = F.flex_attention_bwd_dq(q, k, v, None, None, l, m, o, do, d, block_b=1, block_q=128, block_k_major=128,
                                     block_k=128, sm_scale=sc, debug=False, score_fn=sfn, mask_fn=mf, block_mask_fn=bf, ds=ds)
        return dq, dk, dv
    return fwd, bwd, bwd_exchanging


def _same(name, a, b):
    assert torch.equal(a, b), f"{name}: {int((a != b).sum())} of {a.numel()} elements differ"


@pytest.mark.parametrize("name", ["cfg1", "cfg2", "cfg4", "cfg5"])
def test_full_size_properties(F, name):
    from flex_attention_tpu_amd import configs
    cfg = configs.CONFIGS[name]
    fwd, bwd, bwd_x = _calls(F, cfg)
    q, k, v, do = [x.to(DEV) for x in configs.make_inputs(cfg)]
    group = cfg.Hq // cfg.Hkv

    o, l, m = fwd(q, k, v)
    grads = bwd(q, k, v, o, l, m, do)

    # determinism
    o2, l2, m2 = fwd(q, k, v)
    for n, a, b in zip(("o", "l", "m"), (o, l, m), (o2, l2, m2)):
        _same(f"{n} of a second run", a, b)
    for n, a, b in zip(("dq", "dk", "dv"), grads, bwd(q, k, v, o, l, m, do)):
        _same(f"{n} of a second run", a, b)

    # equivariance under a permutation of the batch entries and, unless the score depends on the head, of the kv groups
    g = torch.Generator().manual_seed(5)
    pb = torch.randperm(cfg.B, generator=g).to(DEV)
    pk = (torch.randperm(cfg.Hkv, generator=g) if cfg.score != "alibi" else torch.arange(cfg.Hkv)).to(DEV)
    pq = (pk[:, None] * group + torch.arange(group, device=DEV)[None, :]).reshape(-1)   # q heads follow their kv head

    def perm_q(x):
        return x[pb][:, pq].contiguous()

    def perm_k(x):
        return x[pb][:, pk].contiguous()
    op, lp, mp = fwd(perm_q(q), perm_k(k), perm_k(v))
    _same("o under a permutation of batch entries and kv groups", op, perm_q(o))
    _same("l under a permutation", lp, perm_q(l))
    _same("m under a permutation", mp, perm_q(m))
    dqp, dkp, dvp = bwd(perm_q(q), perm_k(k), perm_k(v), op, lp, mp, perm_q(do))
    _same("dq under a permutation", dqp, perm_q(grads[0]))
    _same("dk under a permutation", dkp, perm_k(grads[1]))
    _same("dv under a permutation", dvp, perm_k(grads[2]))

    # homogeneity: powers of two go through every product and sum without rounding
    o_v2 = fwd(q, k, v * 2)[0]
    _same("o of 2 v", o_v2, o * 2)
    for n, a, b in zip(("dq", "dk", "dv"), bwd(q, k, v, o, l, m, do * 2), grads):
        _same(f"{n} of 2 dO", a, b * 2)
    for n, a in zip(("dq", "dk", "dv"), bwd(q, k, v, o, l, m, torch.zeros_like(do))):
        assert not a.any(), f"{n} of dO = 0 is not zero"

    # the backward that hands dS over: the same dk, dv; dq deterministic, equivariant and homogeneous as well
    gx = bwd_x(q, k, v, o, l, m, do)
    if gx is not None:
        _same("dk with the dS hand-over", gx[1], grads[1])
        _same("dv with the dS hand-over", gx[2], grads[2])
        _same("dq from dS, second run", bwd_x(q, k, v, o, l, m, do)[0], gx[0])
        _same("dq from dS under a permutation", bwd_x(perm_q(q), perm_k(k), perm_k(v), op, lp, mp, perm_q(do))[0], perm_q(gx[0]))
        _same("dq from dS of 2 dO", bwd_x(q, k, v, o, l, m, do * 2)[0], gx[0] * 2)


@pytest.mark.parametrize("name", ["cfg1", "cfg2", "cfg4", "cfg5"])
def test_a_part_launched_alone_equals_its_part_of_the_full_launch(F, name):
    """One (batch entry, kv group) launched on its own gives the bits it has in the full launch: the small launch
    runs one work item per work-group, handed out by the hardware, the full one the persistent schedule with
    several items per work-group and the next item's first step copied during the last step of the one before.
    (The position bias takes its slopes from the head's index and the number of heads of the call: that
    configuration launches a whole batch entry instead.)"""
    from flex_attention_tpu_amd import configs
    cfg = configs.CONFIGS[name]
    fwd, bwd, bwd_x = _calls(F, cfg)
    q, k, v, do = [x.to(DEV) for x in configs.make_inputs(cfg)]
    group = cfg.Hq // cfg.Hkv
    b = cfg.B - 1
    kv_heads = slice(0, cfg.Hkv) if cfg.score == "alibi" else slice(cfg.Hkv - 1, cfg.Hkv)
    q_heads = slice(kv_heads.start * group, kv_heads.stop * group)

    def part_q(x):
        return x[b:b + 1, q_heads].contiguous()

    def part_k(x):
        return x[b:b + 1, kv_heads].contiguous()
    o, l, m = fwd(q, k, v)
    grads = bwd(q, k, v, o, l, m, do)
    os_, ls_, ms_ = fwd(part_q(q), part_k(k), part_k(v))
    _same("o", os_, part_q(o))
    _same("l", ls_, part_q(l))
    _same("m", ms_, part_q(m))
    dqs, dks, dvs = bwd(part_q(q), part_k(k), part_k(v), os_, ls_, ms_, part_q(do))
    _same("dq", dqs, part_q(grads[0]))
    _same("dk", dks, part_k(grads[1]))
    _same("dv", dvs, part_k(grads[2]))
    gx = bwd_x(q, k, v, o, l, m, do)
    if gx is not None:
        _same("dq from dS", bwd_x(part_q(q), part_k(k), part_k(v), os_, ls_, ms_, part_q(do))[0], part_q(gx[0]))


@pytest.mark.parametrize("name", ["cfg2", "cfg4"])
def test_causal_prefix(F, name):
    """Under a causal mask the first half of the rows does not see the second: the forward and dq of the first
    S / 2 tokens alone give the bits of the first S / 2 rows of the full launch (another number of tiles, other lists,
    another schedule; the same arithmetic per row)."""
    from flex_attention_tpu_amd import configs
    cfg = configs.CONFIGS[name]
    fwd, bwd, _ = _calls(F, cfg)
    q, k, v, do = [x.to(DEV) for x in configs.make_inputs(cfg)]
    n = cfg.S // 2
    o, l, m = fwd(q, k, v)
    dq = bwd(q, k, v, o, l, m, do)[0]

    def head(x):
        return x[:, :, :n].contiguous()
    oh, lh, mh = fwd(head(q), head(k), head(v))
    _same("o of the first half", oh, head(o))
    _same("l of the first half", lh, head(l))
    _same("m of the first half", mh, head(m))
    _same("dq of the first half", bwd(head(q), head(k), head(v), oh, lh, mh, head(do))[0], head(dq))


def _random_case(rng, it, D=128):
    """A random shape, mask, score function, dtype and kernel family (seeded): (tag, tensors, call arguments).
    Head dimension D; 256 is bf16 only."""
    import math
    from flex_attention_tpu_amd import masks, scores
    B, Hkv, g = rng.choice([2, 3, 4, 8]), rng.choice([2, 4, 8, 16]), rng.choice([1, 1, 2, 4])
    S = 128 * rng.choice([2, 4, 7, 8, 13, 16, 24, 32])
    mk = rng.choice(["none", "causal", "window", "causal_window", "documents"])
    sk = rng.choice(["none", "none", "alibi", "softcap"])
    dt = rng.choice([torch.bfloat16, torch.bfloat16, torch.bfloat16, torch.float32])
    compiled_loop = rng.random() < 0.2
    if D > 128:
        dt = torch.bfloat16
    if dt == torch.float32 and S > 2048:
        S = 1024
    if mk == "none":
        mf, bf = None, None
    elif mk == "causal":
        mf, bf = masks.make_causal_mask_fns(128, 128)
    elif mk == "window":
        mf, bf = masks.make_sliding_window_mask_fns(128, 128, rng.randint(100, 900))
    elif mk == "causal_window":
        mf, bf = masks.make_causal_sliding_window_mask_fns(128, 128, rng.randint(1, 700))
    else:
        lens, left = [], S
        while left > 0:
            lens.append(min(left, rng.randint(1, 700)))
            left -= lens[-1]
        mf, bf = masks.make_jagged_mask_fns(128, 128, lens)
    sfn = {"none": None, "alibi": scores.make_alibi_global_score_fn(Hkv * g),
           "softcap": scores.make_softcap_score_fn(rng.choice([2.0, 30.0]))}[sk]
    sc = rng.choice([1.0, 1.0, 3.0]) / math.sqrt(D)
    gen = torch.Generator().manual_seed(7000 + it)
    q, k, v, do = [torch.randn(B, h, S, D, generator=gen).to(dt).to(DEV) for h in (Hkv * g, Hkv, Hkv, Hkv * g)]
    tag = f"B={B} Hq={Hkv * g} Hkv={Hkv} S={S} D={D} mask={mk} score={sk} scale={sc:.3f} {str(dt)[6:]} compiled_loop={compiled_loop}"
    return tag, (q, k, v, do), (sc, mf, bf, sfn, compiled_loop), mk


def _all_passes(F, q, k, v, do, sc, mf, bf, sfn, compiled_loop):
    o, l, m = F._flex_attention_impl(q, k, v, None, None, True, False, sc, 1, 128, 128, 128, False, bf, mf, sfn,
                                     compiled_loop=compiled_loop)
    d = F.compute_delta(o, do)
    kw = dict(sm_scale=sc, debug=False, score_fn=sfn, mask_fn=mf, block_mask_fn=bf, compiled_loop=compiled_loop)
    dq = F.flex_attention_bwd_dq(q, k, v, None, None, l, m, o, do, d, block_b=1, block_q=128, block_k_major=128, block_k=128, **kw)
    dk, dv, ds = F.flash_attention_bwd_dkv(k, v, q, None, None, l, m, d, do, block_b=1, block_q=128, block_q_major=128,
                                           block_k_major=128, block_k=128, causal=False, return_ds=True, **kw)
    dqx = dq if ds is None else F.flex_attention_bwd_dq(q, k, v, None, None, l, m, o, do, d, block_b=1, block_q=128,
                                                        block_k_major=128, block_k=128, ds=ds, **kw)
    return o, l, m, dq, dk, dv, dqx


@pytest.mark.parametrize("D,n_cases,seed", [(128, 24, 20), (256, 10, 22)], ids=["d128", "d256"])
def test_random_shapes_locality(F, D, n_cases, seed):
    """The locality properties above on random shapes (2 to 32 tiles, 2 to 64 heads, grouped kv heads), masks,
    score functions, scales, both dtypes and both kernel families (24 cases at head dimension 128, 10 at 256): one
    batch entry alone against its part of the full launch, every output and the dq from handed-over dS, and under
    causal masks a prefix of the tokens against the prefix of o, l, m, dq.  Bit for bit."""
    import random
    import warnings
    warnings.filterwarnings("ignore", message="score_fn with sm_scale")
    rng = random.Random(seed)
    for it in range(n_cases):
        tag, (q, k, v, do), args, mk = _random_case(rng, it, D)
        full = _all_passes(F, q, k, v, do, *args)
        b = rng.randrange(q.shape[0])
        part = _all_passes(F, *[x[b:b + 1].contiguous() for x in (q, k, v, do)], *args)
        for name, a, r in zip(("o", "l", "m", "dq", "dk", "dv", "dq from dS"), part, full):
            _same(f"{tag}: {name} of batch entry {b} alone", a, r[b:b + 1])
        if mk in ("causal", "causal_window") and q.shape[2] >= 512:
            n = 128 * rng.randrange(1, q.shape[2] // 128)
            pre = _all_passes(F, *[x[:, :, :n].contiguous() for x in (q, k, v, do)], *args)
            for name, a, r in zip(("o", "l", "m", "dq"), pre[:4], full[:4]):
                _same(f"{tag}: {name} of the first {n} tokens alone", a, r[:, :, :n])


@pytest.mark.parametrize("D,n_cases,seed", [(128, 12, 21), (256, 6, 23)], ids=["d128", "d256"])
def test_grouped_kv_heads_equal_repeated_kv_heads(F, D, n_cases, seed):
    """Grouped kv heads against the same call with every kv head repeated for its query heads (on 12 seeded random
    shapes, masks and score functions at head dimension 128, 6 at 256): o, l, m and dq bit for bit (a query head's rows do not care how the kv heads
    are stored; the schedules differ); dk, dv, which the grouped kernels sum over the group in fp32 inside one work
    item, against the sum of the repeated heads' bf16 results in relative L2."""
    import random
    import warnings
    warnings.filterwarnings("ignore", message="score_fn with sm_scale")
    rng = random.Random(seed)
    done = 0
    it = 0
    while done < n_cases:
        it += 1
        tag, (q, k, v, do), args, _ = _random_case(rng, 100 + it, D)
        g = q.shape[1] // k.shape[1]
        if g == 1:
            continue
        done += 1
        a = _all_passes(F, q, k, v, do, *args)
        ke, ve = k.repeat_interleave(g, 1).contiguous(), v.repeat_interleave(g, 1).contiguous()
        e = _all_passes(F, q, ke, ve, do, *args)
        for name, x, y in zip(("o", "l", "m", "dq"), a[:4], e[:4]):
            _same(f"{tag}: {name} with repeated kv heads", y, x)
        B, Hkv, S, _ = k.shape
        for name, x, y in zip(("dk", "dv"), a[4:6], e[4:6]):
            ys = y.float().view(B, Hkv, g, S, D).sum(2)
            rel = float((x.float() - ys).norm() / (ys.norm() + 1e-9))
            assert rel <= 6e-3, f"{tag}: {name} of the group against the sum over repeated heads: rel-L2 {rel:.2e}"


def test_segment_ids_per_batch_entry_properties(F):
    """Rows of segment ids that differ between the batch entries, at 4096 tokens (B=4, 16 q heads on 4 kv heads,
    softcap scores, random documents per entry, one entry with ids that recur): one launch per pass on the union
    map.  Determinism, equivariance under a permutation of the entries with their rows, and every entry alone
    with its own row and its own map: bit for bit, all outputs and the dq from handed-over dS."""
    import math
    import random
    import warnings
    from flex_attention_tpu_amd import scores
    warnings.filterwarnings("ignore", message="score_fn with sm_scale")
    B, Hq, Hkv, S, D = 4, 16, 4, 4096, 128
    rng = random.Random(31)
    rows = []
    for b in range(B):
        lens, left = [], S
        while left > 0:
            lens.append(min(left, rng.randint(1, 1500)))
            left -= lens[-1]
        ids = torch.repeat_interleave(torch.arange(len(lens)), torch.tensor(lens))
        rows.append(ids % 3 if b == 2 else ids)      # (entry 2: ids recur, no intervals)
    sid = torch.stack(rows).to(torch.int32)
    gen = torch.Generator().manual_seed(9000)
    q, k, v, do = [torch.randn(B, h, S, D, generator=gen).to(torch.bfloat16).to(DEV) for h in (Hq, Hkv, Hkv, Hq)]
    sc, sfn = 1 / math.sqrt(D), scores.make_softcap_score_fn(30.0)

    def passes(q, k, v, do, sid):
        o, l, m = F._flex_attention_impl(q, k, v, None, sid, True, True, sc, 1, 128, 128, 128, False, None, None, sfn)
        d = F.compute_delta(o, do)
        kw = dict(sm_scale=sc, debug=False, score_fn=sfn, causal=True)
        dq = F.flex_attention_bwd_dq(q, k, v, None, sid, l, m, o, do, d, block_b=1, block_q=128, block_k_major=128, block_k=128, **kw)
        dk, dv, ds = F.flash_attention_bwd_dkv(k, v, q, None, sid, l, m, d, do, block_b=1, block_q=128, block_q_major=128,
                                               block_k_major=128, block_k=128, return_ds=True, **kw)
        assert ds is not None
        dqx = F.flex_attention_bwd_dq(q, k, v, None, sid, l, m, o, do, d, block_b=1, block_q=128, block_k_major=128,
                                      block_k=128, ds=ds, **kw)
        return o, l, m, dq, dk, dv, dqx
    names = ("o", "l", "m", "dq", "dk", "dv", "dq from dS")
    full = passes(q, k, v, do, sid)
    for n, a, b_ in zip(names, passes(q, k, v, do, sid), full):
        _same(f"{n} of a second run", a, b_)
    pb = torch.tensor([2, 0, 3, 1])
    perm = passes(*[x[pb.to(DEV)].contiguous() for x in (q, k, v, do)], sid[pb])
    for n, a, b_ in zip(names, perm, full):
        _same(f"{n} under a permutation of the batch entries and their rows of ids", a, b_[pb.to(DEV)])
    for b in range(B):
        part = passes(*[x[b:b + 1].contiguous() for x in (q, k, v, do)], sid[b])
        for n, a, b_ in zip(names, part, full):
            _same(f"{n} of entry {b} alone", a, b_[b:b + 1])


def test_tensors_beyond_2_31_elements(F):
    """q, o, dO, dq of 2.3 * 2^30 elements each (B=16, Hq=136, S=8192, D=128; 36 GiB on the device for the eight
    tensors): element offsets do not fit 32 bits from the thirteenth batch entry on.  The last entry of the launch
    must equal that entry launched alone, bit for bit, in every pass; under a causal mask and under a causal window
    with a softcap (stream kernels of two kinds, grouped kv heads, the persistent schedules)."""
    import math
    import warnings
    from flex_attention_tpu_amd import masks, scores
    warnings.filterwarnings("ignore", message="score_fn with sm_scale")
    B, Hq, Hkv, S, D = 16, 136, 34, 8192, 128
    assert B * Hq * S * D > 2 ** 31
    free, _ = torch.cuda.mem_get_info()
    if free < 60 * 2 ** 30:
        pytest.skip("needs 60 GiB of free device memory")
    gen = torch.Generator(device=DEV).manual_seed(1)
    q, k, v, do = [torch.randn(B, h, S, D, device=DEV, dtype=torch.bfloat16, generator=gen) for h in (Hq, Hkv, Hkv, Hq)]
    sc = 1 / math.sqrt(D)
    for (mf, bf), sfn in ((masks.make_causal_mask_fns(128, 128), None),
                          (masks.make_causal_sliding_window_mask_fns(128, 128, 1000), scores.make_softcap_score_fn(30.0))):
        def passes(q, k, v, do):
            o, l, m = F._flex_attention_impl(q, k, v, None, None, True, False, sc, 1, 128, 128, 128, False, bf, mf, sfn)
            d = F.compute_delta(o, do)
            kw = dict(block_b=1, block_q=128, block_k_major=128, block_k=128, sm_scale=sc, debug=False, score_fn=sfn,
                      mask_fn=mf, block_mask_fn=bf)
            dq = F.flex_attention_bwd_dq(q, k, v, None, None, l, m, o, do, d, **kw)
            dk, dv = F.flash_attention_bwd_dkv(k, v, q, None, None, l, m, d, do, block_q_major=128, causal=False, **kw)
            return o, l, m, d, dq, dk, dv
        full = [x[-1:].clone() for x in passes(q, k, v, do)]
        alone = passes(*[x[-1:].contiguous() for x in (q, k, v, do)])
        for n, a, b_ in zip(("o", "l", "m", "delta", "dq", "dk", "dv"), alone, full):
            _same(f"{n} of the last entry alone", a, b_)
        del full, alone


@pytest.mark.parametrize("case", ["causal", "softcap_documents"])
def test_entry_points_replayed_from_a_captured_graph(F, case):
    """The three entry points recorded into a HIP graph (torch.cuda.graph, after two warm-up steps on a side stream:
    the block map of a mask is built once and kept) and replayed on new inputs: every replay gives the bits of the
    same calls made eagerly, the dS hand-over included.  Eager work and synchronisations lie between the replays."""
    import math
    import warnings
    from flex_attention_tpu_amd import masks, scores
    warnings.filterwarnings("ignore", message="score_fn with sm_scale")
    B, Hq, Hkv, S, D = 2, 8, 2, 2048, 128
    sc = 1 / math.sqrt(D)
    gen = torch.Generator(device=DEV).manual_seed(3)
    q, k, v, do = [torch.randn(B, h, S, D, device=DEV, dtype=torch.bfloat16, generator=gen) for h in (Hq, Hkv, Hkv, Hq)]
    mf, bf, sfn, sid = *masks.make_causal_mask_fns(128, 128), None, None
    if case == "softcap_documents":
        mf = bf = None
        sfn = scores.make_softcap_score_fn(30.0)
        sid = torch.repeat_interleave(torch.arange(4), torch.tensor([300, 700, 48, 1000])).to(torch.int32)

    def step(q, k, v, do):
        o, l, m = F._flex_attention_impl(q, k, v, None, sid, True, sid is not None, sc, 1, 128, 128, 128, False, bf, mf, sfn)
        d = F.compute_delta(o, do)
        kw = dict(block_b=1, block_q=128, block_k_major=128, block_k=128, sm_scale=sc, debug=False, score_fn=sfn,
                  mask_fn=mf, block_mask_fn=bf, causal=sid is not None)
        dq = F.flex_attention_bwd_dq(q, k, v, None, sid, l, m, o, do, d, **kw)
        dk, dv, ds = F.flash_attention_bwd_dkv(k, v, q, None, sid, l, m, d, do, block_q_major=128, return_ds=True, **kw)
        dqx = F.flex_attention_bwd_dq(q, k, v, None, sid, l, m, o, do, d, ds=ds, **kw)
        return o, l, m, dq, dk, dv, dqx
    static = [x.clone() for x in (q, k, v, do)]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step(*static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = step(*static)
    for rep in range(3):
        fresh = [x * (1 + 0.25 * rep) for x in (q, k, v, do)]
        for s_, f_ in zip(static, fresh):
            s_.copy_(f_)
        graph.replay()
        torch.cuda.synchronize()
        eager = step(*fresh)
        torch.cuda.synchronize()
        for n, a, b_ in zip(("o", "l", "m", "dq", "dk", "dv", "dq from dS"), out, eager):
            _same(f"{n} of replay {rep}", a, b_)


def test_host_threads_on_streams_of_their_own(F):
    """Four host threads, each on a stream of its own, run different workloads (masks, scores, dtypes, the dS
    hand-over) at the same time, eight steps each: every step gives the bits of the same calls made alone (the C
    entry points keep no state between calls, the error text is per thread, the Python caches are only read and
    extended)."""
    import math
    import threading
    import warnings
    from flex_attention_tpu_amd import masks, scores
    warnings.filterwarnings("ignore", message="score_fn with sm_scale")
    S, D = 1024, 128
    docs = torch.repeat_interleave(torch.arange(3), torch.tensor([300, 600, 124])).to(torch.int32)
    work = [
        ("causal bf16", torch.bfloat16, 2, 8, 8, masks.make_causal_mask_fns(128, 128), None, None, False),
        ("softcap documents bf16, dS hand-over", torch.bfloat16, 1, 8, 2, (None, None), scores.make_softcap_score_fn(30.0), docs, True),
        ("position bias, window bf16", torch.bfloat16, 2, 4, 4, masks.make_causal_sliding_window_mask_fns(128, 128, 300),
         scores.make_alibi_global_score_fn(4), None, False),
        ("plain fp32", torch.float32, 1, 4, 4, (None, None), None, None, False),
    ]

    def step(item, q, k, v, do):
        _, dtype, B, Hq, Hkv, (mf, bf), sfn, sid, exchange = item
        sc = 1 / math.sqrt(D)
        o, l, m = F._flex_attention_impl(q, k, v, None, sid, True, sid is not None, sc, 1, 128, 128, 128, False, bf, mf, sfn)
        d = F.compute_delta(o, do)
        kw = dict(block_b=1, block_q=128, block_k_major=128, block_k=128, sm_scale=sc, debug=False, score_fn=sfn,
                  mask_fn=mf, block_mask_fn=bf, causal=sid is not None)
        dk, dv, ds = F.flash_attention_bwd_dkv(k, v, q, None, sid, l, m, d, do, block_q_major=128, return_ds=exchange, **kw) \
            if exchange else (*F.flash_attention_bwd_dkv(k, v, q, None, sid, l, m, d, do, block_q_major=128, **kw), None)
        dq = F.flex_attention_bwd_dq(q, k, v, None, sid, l, m, o, do, d, ds=ds, **kw)
        return o, l, m, dq, dk, dv
    inputs, alone = [], []
    for n, item in enumerate(work):
        _, dtype, B, Hq, Hkv = item[:5]
        gen = torch.Generator(device=DEV).manual_seed(40 + n)
        t = [torch.randn(B, h, S, D, device=DEV, dtype=dtype, generator=gen) for h in (Hq, Hkv, Hkv, Hq)]
        inputs.append(t)
        alone.append(step(item, *t))
    torch.cuda.synchronize()
    failures = []

    def run(n):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for rep in range(8):
                    got = step(work[n], *inputs[n])
                    stream.synchronize()
                    for name, a, b_ in zip(("o", "l", "m", "dq", "dk", "dv"), got, alone[n]):
                        if not torch.equal(a, b_):
                            failures.append(f"{work[n][0]}: {name} of step {rep} differs")
        except Exception as e:   # noqa: BLE001  (reported by the main thread)
            failures.append(f"{work[n][0]}: {e!r}")
    threads = [threading.Thread(target=run, args=(n,)) for n in range(len(work))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not failures, failures[:4]
