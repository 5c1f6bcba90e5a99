"""Random score functions through the closure compiler, without a GPU.  A seeded grammar writes the source of
`score_mod(s, b, h, q_idx, kv_idx)` functions from the constructs the compiler documents (arithmetic, powers, tanh /
sigmoid / exp / sqrt / abs, minimum / maximum / clamp, where and conditional expressions, comparisons and boolean
operators, % and // on the indices, a per-head table, local assignments); each function is executed as Python and
compiled, and the expression tree must reproduce the function, its symbolic derivative torch's autograd, and the
printed C (built for the host with g++) both, in float32."""
import linecache
import os
import random
import subprocess
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from flex_attention_tpu_amd import _lib, compiler  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
TABLE = (0.5, 0.25, 0.125, 0.0625)
N_FUNCTIONS = 60


class _Grammar:
    """Bounded expressions: every sub-expression stays within a few units so that float32 on the host agrees with
    float64 in Python to 1e-4, and no denominator or root argument comes near zero."""

    def __init__(self, seed, q="q_idx", k="kv_idx", mask=False):
        self.r, self.q, self.k, self.mask = random.Random(seed), q, k, mask

    def const(self):
        return repr(round(self.r.uniform(0.1, 2.0), 3))

    def index(self, depth=0):
        r = self.r
        k = r.randint(0, 6 if depth < 2 else 3)
        if k == 0:
            return self.q
        if k == 1:
            return self.k
        if k == 2:
            return f"({self.q} - {self.k})"
        if k == 3:
            return f"({r.choice([self.q, self.k])} % {r.choice([3, 7, 16, 64])})"
        if k == 4:
            return f"({r.choice([self.q, self.k])} // {r.choice([5, 32, 128])})"
        if k == 5:
            return f"torch.abs({self.index(depth + 1)})"
        return f"({self.index(depth + 1)} {r.choice(['+', '-'])} {self.index(depth + 1)})"

    def cond(self, depth=0):
        r = self.r
        k = r.randint(0, 5 if depth < 2 else 1)
        if self.mask and k in (1, 2):   # (a mask sees no score and no head)
            k = 0
        if k == 0:
            return f"({self.index()} {r.choice(['<', '<=', '>', '>=', '==', '!='])} {r.randint(-40, 300)})"
        if k == 1:
            return f"({self.tensor(2)} {r.choice(['<', '>'])} {self.const()})"
        if k == 2:   # (a condition on the head alone is a Python bool: only next to a tensor condition)
            return f"((h {r.choice(['<', '>=', '=='])} {r.randint(0, 3)}) {r.choice(['&', '|'])} {self.cond(2)})"
        if k == 3:
            return f"({self.cond(depth + 1)} {r.choice(['&', '|'])} {self.cond(depth + 1)})"
        if k == 4:
            return f"(~{self.cond(depth + 1)})"
        return f"({self.index()} % 2 == {r.randint(0, 1)})"

    def small_index(self):
        """an index term scaled into a few units"""
        return f"{self.const()} * 0.001 * {self.index()}"

    def tensor(self, depth=0):
        """a value that is a tensor in Python too (torch's functions do not take Python numbers)"""
        v = self.value(depth)
        return v if ("s" in v.replace("SLOPES", "").replace("abs", "") or "idx" in v) else f"({v} + 0.0 * s)"

    def value(self, depth=0):
        r = self.r
        k = r.randint(0, 14) if depth < 3 else r.randint(0, 3)
        if k == 0:
            return "s"
        if k == 1:
            return f"{self.const()} * s"
        if k == 2:
            return f"({self.small_index()})"
        if k == 3:
            return r.choice([self.const(), "SLOPES[h]", "(b + 1) * 0.5"])
        if k == 14:   # (a Python conditional on the head)
            return f"({self.tensor(depth + 1)} if h {r.choice(['<', '>=', '=='])} {r.randint(0, 3)} else {self.tensor(depth + 1)})"
        a, c = self.tensor(depth + 1), self.tensor(depth + 1)
        if k == 4:
            return f"({a} + {c})"
        if k == 5:
            return f"({a} - {c})"
        if k == 6:
            return f"(torch.tanh({a}) * {c})"
        if k == 7:
            return f"({a} / (1.5 + torch.abs({c})))"
        if k == 8:
            return f"torch.{r.choice(['tanh', 'sigmoid'])}({a})"
        if k == 9:
            return f"torch.{r.choice(['minimum', 'maximum'])}({a}, {c})"
        if k == 10:
            return f"torch.where({self.cond()}, {a}, {c})"
        if k == 11:
            return r.choice([f"torch.tanh({a}) ** {r.randint(2, 4)}", f"torch.sqrt(1.0 + torch.abs({a}))",
                             f"torch.exp(-torch.abs({a}))", f"2.0 ** (-torch.abs({a}))"])
        if k == 12:
            return f"torch.clamp({a}, min=-{self.const()}, max={self.const()})"
        return f"torch.abs({a})"

    def function(self, name):
        lines = [f"def {name}(s, b, h, q_idx, kv_idx):"]
        if self.r.random() < 0.6:
            lines.append(f"    t = {self.value(1)}")
            lines.append(f"    near = {self.cond()}")
            body = f"torch.where(near, t, {self.value(1)}) + {self.const()} * s"
        else:
            body = f"{self.value()} + {self.const()} * torch.tanh(s)"
        lines.append(f"    return {body}")
        return "\n".join(lines) + "\n"


    def mask_function(self, name):
        return (f"def {name}(q_idx, k_idx):\n    qi = q_idx[:, None]\n    kj = k_idx[None, :]\n"
                f"    return {self.cond()} | (qi == kj)\n")


def _load(name, text):
    """The function of `text`, with its source registered so that inspect finds it."""
    filename = f"<random score function {name}>"
    linecache.cache[filename] = (len(text), None, text.splitlines(True), filename)
    scope = {"torch": torch, "SLOPES": TABLE}
    exec(compile(text, filename, "exec"), scope)
    return scope[name]


def _functions():
    for n in range(N_FUNCTIONS):
        name = f"random_mod_{n}"
        text = _Grammar(1000 + n).function(name)
        yield n, name, text, _load(name, text)


def _probes(seed, n=300):
    g = torch.Generator().manual_seed(seed)
    s = (torch.randn(n, generator=g) * 3.0).to(torch.float32).double()
    return (s.requires_grad_(True), torch.randint(0, 3, (n,), generator=g), torch.randint(0, 4, (n,), generator=g),
            torch.randint(0, 4096, (n,), generator=g), torch.randint(0, 4096, (n,), generator=g))


def _python_values(fn, s, b, h, i, j):
    want = torch.stack([torch.as_tensor(fn(s[t], int(b[t]), int(h[t]), i[t], j[t]), dtype=torch.float64) for t in range(s.numel())])
    (grad,) = torch.autograd.grad(want.sum(), s, allow_unused=True)
    return want.detach(), torch.zeros_like(want) if grad is None else grad


@pytest.mark.parametrize("n,name,text,fn", list(_functions()), ids=lambda x: x if isinstance(x, str) and x.startswith("random_mod") else "")
def test_random_score_function(tmp_path, n, name, text, fn):
    print(text)
    c = compiler.compile_score_mod(fn, recognise=False)
    assert c.spec.kind == _lib.SCORE_CUSTOM
    s, b, h, i, j = _probes(n)
    want, grad = _python_values(fn, s, b, h, i, j)
    # the tree and its symbolic derivative, element by element (b, h are scalars in the functor)
    got = torch.stack([torch.as_tensor(c.expr.ev({"s": s[t].detach(), "b": int(b[t]), "h": int(h[t]), "i": i[t], "j": j[t],
                                                  "mq": 128, "mk": 128}), dtype=torch.float64) for t in range(s.numel())])
    dgot = torch.stack([torch.as_tensor(c.expr.d().ev({"s": s[t].detach(), "b": int(b[t]), "h": int(h[t]), "i": i[t], "j": j[t],
                                                       "mq": 128, "mk": 128}), dtype=torch.float64) for t in range(s.numel())])
    assert torch.allclose(got, want, rtol=1e-6, atol=1e-6), float((got - want).abs().max())
    assert torch.allclose(dgot, grad, rtol=1e-6, atol=1e-6), float((dgot - grad).abs().max())
    if n % 3:
        return
    # the printed C functions, built for the host: float32 arithmetic against the float64 values
    header = tmp_path / "custom_functor.hpp"
    header.write_text(compiler.header_text(c.spec.custom, None))
    exe = tmp_path / "functor_check"
    subprocess.run(["g++", "-O1", "-std=c++17", "-D__host__=", "-D__device__=", "-include", str(header),
                    os.path.join(HERE, "host", "functor_check.cpp"), "-o", str(exe)], check=True)
    lines = "".join(f"{float(s[t].detach()):.9g} {int(b[t])} {int(h[t])} {int(i[t])} {int(j[t])} 128 128\n" for t in range(s.numel()))
    out = subprocess.run([str(exe)], input=lines, capture_output=True, text=True, check=True).stdout.split()
    host = torch.tensor([float(x) for x in out], dtype=torch.float64).reshape(-1, 3)
    # (a comparison of s with a constant may fall on the other side in float32 for a probe within rounding of it:
    #  such probes, if any, are left out of the comparison)
    ok = ((host[:, 0] - want).abs() <= 1e-4 * (1 + want.abs())) & ((host[:, 1] - grad).abs() <= 1e-4 * (1 + grad.abs()))
    assert int((~ok).sum()) <= 1, (int((~ok).sum()), float((host[:, 0] - want).abs().max()), float((host[:, 1] - grad).abs().max()))


def _masks():
    for n in range(24):
        name = f"random_mask_{n}"
        text = _Grammar(5000 + n, q="qi", k="kj", mask=True).mask_function(name)
        yield n, name, text, _load(name, text)


@pytest.mark.parametrize("n,name,text,fn", list(_masks()), ids=lambda x: x if isinstance(x, str) and x.startswith("random_mask") else "")
def test_random_mask_function(n, name, text, fn):
    """Random predicates on the indices: the tree against the Python function on a dense grid, the block closure
    against any() over every tile, at two granularities."""
    print(text)
    i, j = torch.arange(384), torch.arange(256)
    dense = fn(i, j)
    for bq, bk in ((64, 32), (128, 128)):
        mask_fn, block_fn = compiler.compile_mask_fn(fn, bq, bk, recognise=False)
        assert mask_fn.spec.flags == _lib.MASK_CUSTOM
        got = torch.as_tensor(mask_fn.expr.ev({"i": i[:, None], "j": j[None, :]}))
        assert torch.equal(got.expand_as(dense), dense)
        for qb in range(384 // bq):
            for kb in range(256 // bk):
                assert block_fn(qb, kb) == bool(dense[bq * qb:bq * qb + bq, bk * kb:bk * kb + bk].any()), (qb, kb)
