"""The Python callable -> device functor compiler (compiler.py), without a GPU: the expression tree
against the Python function, its derivative against autograd, the printed C functions (compiled for
the host with g++) against both, and the constructs that must be refused."""
import os
import subprocess
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import custom_functors as cf  # noqa: E402
from flex_attention_tpu_amd import _lib, compiler, util  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def _grid(n=40, seed=3, tile=None):
    g = torch.Generator().manual_seed(seed)
    if tile is None:
        i = torch.randint(0, 2048, (n,), generator=g)
        j = torch.randint(0, 2048, (n,), generator=g)
    else:
        i, j = torch.arange(tile[0]), torch.arange(tile[1])
    s = (torch.randn(i.numel(), j.numel(), generator=g, dtype=torch.float64) * 5.0).requires_grad_(True)
    return s, i, j


@pytest.mark.parametrize("fn", [cf.alibi_mod, cf.softcap_mod, cf.mixed_mod], ids=lambda f: f.__name__)
def test_score_mod_tree_and_derivative(fn):
    c = compiler.compile_score_mod(fn, recognise=False)
    assert c.spec.kind == _lib.SCORE_CUSTOM
    s, i, j = _grid()
    for b, h in ((0, 0), (1, 3)):
        env = {"s": s, "b": b, "h": h, "i": i[:, None], "j": j[None, :], "mq": 128, "mk": 128}
        want = fn(s, b, h, i[:, None], j[None, :])
        got = torch.as_tensor(c.expr.ev(env))
        assert torch.allclose(got, want, rtol=1e-7, atol=1e-7)   # (torch computes int tensor * Python float in float32)
        (grad,) = torch.autograd.grad(want.sum(), s)
        dgot = torch.as_tensor(c.expr.d().ev(env), dtype=torch.float64).expand_as(grad)
        assert torch.allclose(dgot, grad, rtol=1e-7, atol=1e-7)


@pytest.mark.parametrize("fn", [cf.squared_tile, cf.tile_local_distance], ids=lambda f: f.__name__)
def test_tile_form_tree(fn):
    c = util.make_jax_score_fn(fn)
    assert c.spec.kind == _lib.SCORE_CUSTOM   # not one of the built-in functors: compiled
    g = torch.Generator().manual_seed(5)
    for m, n in ((16, 16), (32, 48)):
        q = torch.randn(m, 8, generator=g, dtype=torch.float64)
        k = torch.randn(n, 8, generator=g, dtype=torch.float64)
        env = {"s": q @ k.T, "b": 0, "h": 0, "i": torch.arange(m)[:, None], "j": torch.arange(n)[None, :], "mq": m, "mk": n}
        assert torch.allclose(torch.as_tensor(c.expr.ev(env)), fn(q, k), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("fn", [cf.prefix_lm_mask, cf.checker_mask], ids=lambda f: f.__name__)
def test_mask_tree_and_block_closure(fn):
    mask_fn, block_fn = compiler.compile_mask_fn(fn, 64, 32)
    assert mask_fn.spec.flags == _lib.MASK_CUSTOM and block_fn.spec == mask_fn.spec
    i, j = torch.arange(256), torch.arange(192)
    dense = fn(i, j)
    got = torch.as_tensor(mask_fn.expr.ev({"i": i[:, None], "j": j[None, :]}))
    assert torch.equal(got, dense)
    for qb in range(4):
        for kb in range(6):
            assert block_fn(qb, kb) == bool(dense[64 * qb:64 * qb + 64, 32 * kb:32 * kb + 32].any())


def test_generated_c_matches_python_on_the_host(tmp_path):
    """The header the kernels are compiled against, compiled for the host instead: custom_score,
    custom_dscore and custom_keep against the Python functions (operator precedence, Python's floor
    division and modulo, exact constants, tables)."""
    score = compiler.compile_score_mod(cf.mixed_mod)
    mask_fn, _ = compiler.compile_mask_fn(cf.checker_mask, 128, 128)
    header = tmp_path / "custom_functor.hpp"
    header.write_text(compiler.header_text(score.spec.custom, mask_fn.spec.custom))
    exe = tmp_path / "functor_check"
    subprocess.run(["g++", "-O1", "-std=c++17", "-D__host__=", "-D__device__=", "-include", str(header),
                    os.path.join(HERE, "host", "functor_check.cpp"), "-o", str(exe)], check=True)
    g = torch.Generator().manual_seed(9)
    n = 400
    s = (torch.randn(n, generator=g) * 5.0).to(torch.float32).double().requires_grad_(True)
    b = torch.randint(0, 3, (n,), generator=g)
    h = torch.randint(0, 4, (n,), generator=g)
    i = torch.randint(0, 4096, (n,), generator=g)
    j = torch.randint(0, 4096, (n,), generator=g)
    lines = "".join(f"{float(s[t]):.9g} {int(b[t])} {int(h[t])} {int(i[t])} {int(j[t])} 128 128\n" for t in range(n))
    out = subprocess.run([str(exe)], input=lines, capture_output=True, text=True, check=True).stdout.split()
    got = torch.tensor([float(x) for x in out], dtype=torch.float64).reshape(n, 3)
    want = torch.stack([cf.mixed_mod(s[t], int(b[t]), int(h[t]), i[t], j[t]) for t in range(n)])
    (grad,) = torch.autograd.grad(want.sum(), s)
    keep = torch.stack([cf.checker_mask(i[t:t + 1], j[t:t + 1])[0, 0] for t in range(n)])
    assert torch.allclose(got[:, 0], want.detach(), rtol=2e-6, atol=2e-6)   # float32 arithmetic in the functor
    assert torch.allclose(got[:, 1], grad, rtol=2e-6, atol=2e-6)
    assert torch.equal(got[:, 2].bool(), keep)


def test_recognised_closed_forms_keep_the_stream_kernels():
    cap = 30.0

    def softcap(q_tile, k_tile):
        return cap * torch.tanh(torch.matmul(q_tile, k_tile.T) / cap)

    def clipped_alibi(q_tile, k_tile):
        # equals the tile-local ALiBi on small tiles only: the second, larger probe tells them apart
        d = torch.abs(torch.arange(q_tile.shape[0])[:, None] - torch.arange(k_tile.shape[0])[None, :])
        return q_tile @ k_tile.T - 0.5 * torch.minimum(d, torch.tensor(45))
    assert util.make_jax_score_fn(softcap).spec.kind == _lib.SCORE_SOFTCAP
    assert util.make_jax_score_fn(clipped_alibi).spec.kind == _lib.SCORE_CUSTOM


def _causal(q_idx, k_idx):
    return q_idx[:, None] >= k_idx[None, :]


def _window(q_idx, k_idx):
    return q_idx[:, None] - k_idx[None, :] < 1000


def _causal_window(q_idx, k_idx):
    d = q_idx[:, None] - k_idx[None, :]
    return (d >= 0) & (d <= 1024)


def _causal_window_and_a_sink(q_idx, k_idx):
    d = q_idx[:, None] - k_idx[None, :]
    return ((d >= 0) & (d <= 1024)) | (k_idx[None, :] == 7)


def _s2(q_idx, k_idx):
    d = q_idx[:, None] - k_idx[None, :]
    return ((d >= 0) & (d < 128)) | ((k_idx[None, :] % 64 == 0) & (d >= 0))


def _s2_shifted(q_idx, k_idx):
    d = q_idx[:, None] - k_idx[None, :]
    return ((d >= 0) & (d < 128)) | ((k_idx[None, :] % 64 == 3) & (d >= 0))


def _identity(s, b, h, q_idx, kv_idx):
    return s


def _softcap(s, b, h, q_idx, kv_idx):
    return 50.0 * torch.tanh(s / 50.0)


def _nearly_softcap(s, b, h, q_idx, kv_idx):
    return 50.0 * torch.tanh(s / 50.0) + 1e-6 * s


def _alibi_by_formula(s, b, h, q_idx, kv_idx):
    return s + 2.0 ** (-8.0 * (h + 1) / 16) * (kv_idx - q_idx)


def _alibi_symmetric(s, b, h, q_idx, kv_idx):
    return s - 0.5 ** (h + 1) * torch.abs(q_idx - kv_idx)


def test_closures_that_equal_a_builtin_functor_get_it():
    """compile_score_mod / compile_mask_fn recognise the functors the kernels carry themselves (numerically, on
    the expression tree) and hand out their specifications: those calls run the generated-stream kernels on
    closed-form block maps.  Anything that differs anywhere on the probes stays a compiled functor."""
    from flex_attention_tpu_amd import masks, scores
    for fn, flags, window in ((_causal, _lib.MASK_CAUSAL, 0), (_window, _lib.MASK_WINDOW, 1000),
                              (_causal_window, _lib.MASK_CAUSAL | _lib.MASK_WINDOW, 1025)):
        mf, bf = compiler.compile_mask_fn(fn, 128, 64)
        assert mf.spec.flags == flags and mf.spec.window == window and mf.spec.custom is None and bf.spec == mf.spec
        qi, kj = torch.arange(900, 1300), torch.arange(0, 1400)
        assert torch.equal(torch.as_tensor(mf(qi, kj)), torch.as_tensor(fn(qi, kj)))
        assert compiler.compile_mask_fn(fn, 128, 64, recognise=False)[0].spec.flags == _lib.MASK_CUSTOM
    assert compiler.compile_mask_fn(_causal_window_and_a_sink, 128, 64)[0].spec.flags == _lib.MASK_CUSTOM
    s2 = compiler.compile_mask_fn(_s2, 128, 64)[0].spec      # the reference's local + strided mask (masks.py:143-179)
    assert (s2.flags, s2.window, s2.stride, s2.custom) == (_lib.MASK_S2, 128, 64, None)
    assert compiler.compile_mask_fn(_s2_shifted, 128, 64)[0].spec.flags == _lib.MASK_CUSTOM
    assert compiler.compile_score_mod(_identity).spec == scores.ScoreSpec(kind=_lib.SCORE_NONE)
    assert compiler.compile_score_mod(_softcap).spec == scores.ScoreSpec(kind=_lib.SCORE_SOFTCAP, cap=50.0)
    assert compiler.compile_score_mod(_softcap, recognise=False).spec.kind == _lib.SCORE_CUSTOM
    assert compiler.compile_score_mod(_nearly_softcap).spec.kind == _lib.SCORE_CUSTOM
    assert compiler.compile_score_mod(_alibi_symmetric).spec.kind == _lib.SCORE_CUSTOM
    assert compiler.compile_score_mod(cf.alibi_mod).spec == scores.ScoreSpec(kind=_lib.SCORE_ALIBI, slopes=cf.SLOPES)
    spec = compiler.compile_score_mod(_alibi_by_formula).spec     # (slopes from the head's index: as many as a call has heads)
    assert spec.kind == _lib.SCORE_ALIBI and spec.slopes is None and len(spec.slopes_open) == compiler.MAX_OPEN_HEADS
    assert all(abs(a - b) <= 1e-12 for a, b in zip(spec.slopes_open[:16], scores.alibi_slopes(16)))
    assert compiler.compile_score_mod(cf.mixed_mod).spec.kind == _lib.SCORE_CUSTOM


def test_powers_with_variable_exponents():
    def f(s, b, h, q_idx, kv_idx):
        return s * 0.5 ** (h + 1) + (torch.abs(s) + 1.0) ** 1.5
    g = compiler.compile_score_mod(f)
    assert g.spec.kind == _lib.SCORE_CUSTOM and "fa_pow" in g.spec.custom.body and "fa_pow" in g.spec.custom.dbody
    env = {"s": torch.linspace(-3, 3, 12, dtype=torch.float64), "b": 0, "h": 2, "i": 0, "j": 0}   # (not 0: |s| has no derivative there)
    s = env["s"].clone().requires_grad_(True)
    want = torch.autograd.grad(f(s, 0, 2, 0, 0).sum(), s)[0]
    assert torch.allclose(torch.as_tensor(g.expr.d().ev(env), dtype=torch.float64), want, rtol=1e-12, atol=1e-12)
    with pytest.raises(NotImplementedError, match="positive base"):
        compiler.compile_score_mod(lambda s, b, h, q_idx, kv_idx: (-2.0) ** h + s)


def test_plain_closures_are_compiled_at_the_entry_points():
    """tagged_closures, which every entry point calls first: a function object without a specification is compiled
    by its form (two arguments: the reference's tile form; five: score_mod; a mask function at the call's block
    sizes, with its block closure), once per function object; what carries a specification passes through."""
    from flex_attention_tpu_amd import masks, scores
    from flex_attention_tpu_amd._common import tagged_closures

    def tile_softcap(q_tile, k_tile):
        return 30.0 * torch.tanh(torch.matmul(q_tile, k_tile.T) / 30.0)
    s1, m1, b1 = tagged_closures(tile_softcap, _causal_window, None, 128, 128)
    assert s1.spec == scores.ScoreSpec(kind=_lib.SCORE_SOFTCAP, cap=30.0)
    assert m1.spec.flags == _lib.MASK_CAUSAL | _lib.MASK_WINDOW and m1.spec.window == 1025 and b1.spec == m1.spec
    s2, m2, b2 = tagged_closures(tile_softcap, _causal_window, None, 128, 128)
    assert s2 is s1 and m2 is m1 and b2 is b1                       # (compiled once)
    assert tagged_closures(_softcap, None, None, 128, 128)[0].spec.kind == _lib.SCORE_SOFTCAP
    assert tagged_closures(cf.mixed_mod, cf.checker_mask, None, 128, 64)[0].spec.kind == _lib.SCORE_CUSTOM
    assert tagged_closures(None, cf.checker_mask, None, 128, 64)[1].spec.flags == _lib.MASK_CUSTOM
    fac_s, fac_m = scores.make_softcap_score_fn(5.0), masks.make_causal_mask_fns(128, 128)
    assert tagged_closures(fac_s, fac_m[0], fac_m[1], 128, 128) == (fac_s, fac_m[0], fac_m[1])
    assert tagged_closures(None, None, None, 128, 128) == (None, None, None)
    with pytest.raises(NotImplementedError, match="score_fn must take"):
        tagged_closures(lambda a, b, c: a, None, None, 128, 128)


def test_unsupported_constructs_are_refused():
    def uses_softmax(s, b, h, q_idx, kv_idx):
        return torch.softmax(s, -1)

    def loops(s, b, h, q_idx, kv_idx):
        for _ in range(2):
            s = s + 1
        return s

    def mask_of_the_head(q_idx, k_idx, h=0):
        return q_idx[:, None] >= k_idx[None, :]

    def returns_number_as_mask(q_idx, k_idx):
        return q_idx[:, None] - k_idx[None, :]

    def other_product(q_tile, k_tile):
        return q_tile @ q_tile.T
    for fn in (uses_softmax, loops):
        with pytest.raises(NotImplementedError):
            compiler.compile_score_mod(fn)
    for fn in (mask_of_the_head, returns_number_as_mask):
        with pytest.raises(NotImplementedError):
            compiler.compile_mask_fn(fn, 128, 128)
    with pytest.raises(NotImplementedError):
        compiler.compile_score_fn(other_product)


def test_functor_keys_and_header_are_deterministic():
    a = compiler.compile_score_mod(cf.softcap_mod, recognise=False).spec.custom
    b = compiler.compile_score_mod(cf.softcap_mod, recognise=False).spec.custom
    m = compiler.compile_mask_fn(cf.prefix_lm_mask, 128, 128)[0].spec.custom
    assert a == b and compiler.functor_key(a, None) == compiler.functor_key(b, None)
    assert len({compiler.functor_key(a, None), compiler.functor_key(a, m), compiler.functor_key(None, m)}) == 3
    text = compiler.header_text(a, m)
    assert compiler.functor_key(a, m) in text and "custom_dscore" in text and "custom_keep" in text
    # the plain library refuses compiled closures
    lib = _lib.load()
    assert lib.flexattn_custom_tag() == b""
