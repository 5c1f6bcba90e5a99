"""Python callable -> device functor compiler for score and mask closures.

The reference traces arbitrary ``score_fn`` / ``mask_fn`` closures into its Pallas kernels: the
forward calls ``score_fn(q_tile, k_tile)`` and ``mask_fn(q_idx, k_idx)`` on traced values
(flex_attention_kernel.py:248-255, 278-288), ``util.make_jax_score_fn`` rewrites a user function's
AST into ``lax.dot_general`` form first (util.py:22-189), and the backward kernels differentiate the
score function with ``jax.vjp`` over a table of eight primitives (util.py:196-259).

A HIP kernel cannot trace Python.  This module does the same job ahead of time:

1. the closure's source is parsed (``ast``) and executed symbolically into a small expression tree
   over ``s`` (the scaled dot product), the indices ``b, h, i, j`` and captured constants;
2. the tree is differentiated with respect to ``s`` by a rule table (the successor of the VJP table);
3. both are printed as C functions into a header, the kernels with a compiled main loop are
   compiled against it with hipcc into a library of their own (same C ABI as libflexattn.so), cached
   under ``_jit/<hash of the header>/``;
4. the returned closure carries a spec that makes the entry points call that library.

Before anything is compiled, the tree is evaluated next to the original Python function on random
probes and must agree with it; whatever the rewriter does not understand raises
``NotImplementedError`` naming the construct.

Accepted source: one ``def`` or ``lambda``; straight-line assignments and a ``return``; operators
``+ - * / // % **`` (integer power), comparisons, ``and / or / not``, ``& | ~`` on booleans,
conditional expressions; calls ``tanh exp log sqrt abs sigmoid minimum maximum min max where
clamp`` (as ``torch.x``, ``jnp.x``, ``np.x``, ``math.x`` or methods); casts are ignored; captured
``int / float / bool`` values are inlined, captured sequences or 1-D tensors of numbers become
constant arrays indexable by an integer expression (``slopes[h]``).
"""
from __future__ import annotations

import ast
import hashlib
import inspect
import math
import os
import textwrap
from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
JIT_DIR = os.path.join(PKG_DIR, "_jit")
CODEGEN_VERSION = 3


# ------------------------------------------------------------------------------------------------
# expression tree
# ------------------------------------------------------------------------------------------------
class Node:
    """Expression node.  kind: 'f' float, 'i' integer, 'b' boolean."""
    kind = "f"

    def c(self) -> str:            # C expression
        raise NotImplementedError

    def ev(self, env):             # torch evaluation (env: name -> tensor / number)
        raise NotImplementedError

    def d(self) -> "Node":         # derivative with respect to s
        return Const(0.0)

    def uses_s(self) -> bool:
        return False


def _as_float_c(n: Node) -> str:
    return n.c() if n.kind == "f" else f"(float)({n.c()})"


def _is_zero(n: Node) -> bool:
    return isinstance(n, Const) and n.kind == "f" and float(n.value) == 0.0


def _is_one(n: Node) -> bool:
    return isinstance(n, Const) and n.kind == "f" and float(n.value) == 1.0


class Const(Node):
    def __init__(self, value):
        if isinstance(value, bool):
            self.kind = "b"
        elif isinstance(value, (int, np.integer)):
            self.kind, value = "i", int(value)
        else:
            self.kind, value = "f", float(value)
        self.value = value

    def c(self):
        if self.kind == "b":
            return "true" if self.value else "false"
        if self.kind == "i":
            return f"({self.value})" if self.value < 0 else str(self.value)
        v = float(self.value)
        if math.isinf(v):
            return "(-__builtin_huge_valf())" if v < 0 else "__builtin_huge_valf()"
        if math.isnan(v):
            raise NotImplementedError("NaN constant in a score / mask function")
        return f"({float(np.float32(v)).hex()}f)"   # exact float32 literal

    def ev(self, env):
        return self.value


class Var(Node):
    """s (float) or one of the integer inputs b, h, i, j, mq, mk (tile edges for tile-local indices)."""
    def __init__(self, name):
        self.name = name
        self.kind = "f" if name == "s" else "i"

    def c(self):
        return self.name

    def ev(self, env):
        return env[self.name]

    def d(self):
        return Const(1.0 if self.name == "s" else 0.0)

    def uses_s(self):
        return self.name == "s"


class Table(Node):
    """Constant array indexed by an integer expression."""
    def __init__(self, name, values, index: Node):
        vals = [v for v in values]
        self.kind = "i" if all(isinstance(v, (int, np.integer)) and not isinstance(v, bool) for v in vals) else "f"
        self.name, self.values, self.index = name, vals, index
        if index.kind != "i":
            raise NotImplementedError(f"{name}[...] must be indexed by an integer expression")

    def c(self):
        return f"{self.name}[{self.index.c()}]"

    def ev(self, env):
        t = torch.tensor(self.values, dtype=torch.int64 if self.kind == "i" else torch.float64)
        idx = self.index.ev(env)
        return t[idx] if isinstance(idx, torch.Tensor) else t[int(idx)]

    def decl(self):
        ty = "int" if self.kind == "i" else "float"
        body = ", ".join(Const(v).c() for v in self.values)
        return f"  constexpr {ty} {self.name}[{len(self.values)}] = {{{body}}};"


ARITH = {"+", "-", "*", "/", "//", "%"}


class Bin(Node):
    def __init__(self, op, a: Node, b: Node):
        self.op, self.a, self.b = op, a, b
        if op in ARITH:
            if a.kind == "b" or b.kind == "b":
                a = self.a = Cast(a, "i") if a.kind == "b" else a
                b = self.b = Cast(b, "i") if b.kind == "b" else b
            self.kind = "f" if (op == "/" or "f" in (a.kind, b.kind)) else "i"
        elif op in ("<", "<=", ">", ">=", "==", "!=", "and", "or"):
            self.kind = "b"
        else:
            raise NotImplementedError(f"operator {op}")

    def c(self):
        a, b, op = self.a, self.b, self.op
        if op in ("and", "or"):
            return f"({a.c()} {'&&' if op == 'and' else '||'} {b.c()})"
        if op in ("<", "<=", ">", ">=", "==", "!="):
            if "f" in (a.kind, b.kind):
                return f"({_as_float_c(a)} {op} {_as_float_c(b)})"
            return f"({a.c()} {op} {b.c()})"
        if self.kind == "f":
            if op == "//":
                return f"floorf({_as_float_c(a)} / {_as_float_c(b)})"
            if op == "%":
                return f"fa_py_fmod({_as_float_c(a)}, {_as_float_c(b)})"
            return f"({_as_float_c(a)} {op} {_as_float_c(b)})"
        if op == "//":
            return f"fa_py_floordiv({a.c()}, {b.c()})"
        if op == "%":
            return f"fa_py_mod({a.c()}, {b.c()})"
        return f"({a.c()} {op} {b.c()})"

    def ev(self, env):
        x, y, op = self.a.ev(env), self.b.ev(env), self.op
        if op == "+": return x + y
        if op == "-": return x - y
        if op == "*": return x * y
        if op == "/": return torch.as_tensor(x, dtype=torch.float64) / y if not isinstance(x, float) else x / y
        if op == "//": return x // y
        if op == "%": return x % y
        if op == "<": return x < y
        if op == "<=": return x <= y
        if op == ">": return x > y
        if op == ">=": return x >= y
        if op == "==": return x == y
        if op == "!=": return x != y
        if op == "and": return torch.as_tensor(x) & torch.as_tensor(y)
        return torch.as_tensor(x) | torch.as_tensor(y)

    def d(self):
        if self.kind != "f" or not self.uses_s():
            return Const(0.0)
        a, b, op = self.a, self.b, self.op
        da, db = a.d(), b.d()
        if op == "+": return add(da, db)
        if op == "-": return sub(da, db)
        if op == "*": return add(mul(da, b), mul(a, db))
        if op == "/": return sub(div(da, b), div(mul(a, db), mul(b, b)))
        raise NotImplementedError(f"derivative of '{op}' applied to the score")

    def uses_s(self):
        return self.a.uses_s() or self.b.uses_s()


def add(a, b):
    if _is_zero(a): return b
    if _is_zero(b): return a
    return Bin("+", a, b)


def sub(a, b):
    if _is_zero(b): return a
    if _is_zero(a): return Un("-", b)
    return Bin("-", a, b)


def mul(a, b):
    if _is_zero(a) or _is_zero(b): return Const(0.0)
    if _is_one(a): return b
    if _is_one(b): return a
    return Bin("*", a, b)


def div(a, b):
    if _is_zero(a): return Const(0.0)
    if _is_one(b): return a
    return Bin("/", a, b)


class Un(Node):
    def __init__(self, op, a: Node):
        self.op, self.a = op, a
        self.kind = "b" if op == "not" else a.kind

    def c(self):
        return f"(!{self.a.c()})" if self.op == "not" else f"(-{self.a.c()})"

    def ev(self, env):
        x = self.a.ev(env)
        return ~torch.as_tensor(x) if self.op == "not" else -x

    def d(self):
        return Const(0.0) if self.op == "not" or not self.a.uses_s() else Un("-", self.a.d())

    def uses_s(self):
        return self.a.uses_s()


class Cast(Node):
    def __init__(self, a: Node, kind):
        self.a, self.kind = a, kind

    def c(self):
        return f"({'float' if self.kind == 'f' else 'int'})({self.a.c()})"

    def ev(self, env):
        x = torch.as_tensor(self.a.ev(env))
        return x.to(torch.float64) if self.kind == "f" else x.to(torch.int64)

    def d(self):
        return self.a.d() if self.kind == "f" else Const(0.0)

    def uses_s(self):
        return self.a.uses_s()


class Select(Node):
    def __init__(self, cond: Node, a: Node, b: Node):
        self.cond, self.a, self.b = cond, a, b
        self.kind = "f" if "f" in (a.kind, b.kind) else a.kind

    def c(self):
        if self.kind == "f":
            return f"({self.cond.c()} ? {_as_float_c(self.a)} : {_as_float_c(self.b)})"
        return f"({self.cond.c()} ? {self.a.c()} : {self.b.c()})"

    def ev(self, env):
        a, b = self.a.ev(env), self.b.ev(env)
        dt = torch.float64 if self.kind == "f" else (torch.bool if self.kind == "b" else torch.int64)
        return torch.where(torch.as_tensor(self.cond.ev(env)), torch.as_tensor(a, dtype=dt), torch.as_tensor(b, dtype=dt))

    def d(self):
        if self.kind != "f" or not self.uses_s():
            return Const(0.0)
        return Select(self.cond, self.a.d(), self.b.d())

    def uses_s(self):
        return self.a.uses_s() or self.b.uses_s()   # (a condition on s has derivative zero almost everywhere)


# name -> (C function, torch function, derivative rule f(x, dx, y) with y = the call itself)
FUNCS = {
    "tanh": ("fa_tanh", torch.tanh, lambda x, dx, y: mul(dx, sub(Const(1.0), mul(y, y)))),
    "exp": ("fa_exp", torch.exp, lambda x, dx, y: mul(dx, y)),
    "log": ("fa_log", torch.log, lambda x, dx, y: div(dx, x)),
    "sqrt": ("fa_sqrt", torch.sqrt, lambda x, dx, y: div(dx, mul(Const(2.0), y))),
    "abs": ("fabsf", torch.abs, lambda x, dx, y: mul(dx, Select(Bin("<", x, Const(0.0)), Const(-1.0), Const(1.0)))),
    "sigmoid": ("fa_sigmoid", torch.sigmoid, lambda x, dx, y: mul(dx, mul(y, sub(Const(1.0), y)))),
}


class Call(Node):
    def __init__(self, fn: str, a: Node):
        self.fn, self.a = fn, a
        self.kind = "i" if (fn == "abs" and a.kind == "i") else "f"

    def c(self):
        if self.kind == "i":
            return f"abs({self.a.c()})"
        return f"{FUNCS[self.fn][0]}({_as_float_c(self.a)})"

    def ev(self, env):
        x = self.a.ev(env)
        if self.kind == "i":
            return abs(x)
        return FUNCS[self.fn][1](torch.as_tensor(x, dtype=torch.float64))

    def d(self):
        if self.kind != "f" or not self.a.uses_s():
            return Const(0.0)
        return FUNCS[self.fn][2](self.a, self.a.d(), self)

    def uses_s(self):
        return self.a.uses_s()


class MinMax(Node):
    def __init__(self, is_max: bool, a: Node, b: Node):
        self.is_max, self.a, self.b = is_max, a, b
        self.kind = "f" if "f" in (a.kind, b.kind) else "i"

    def c(self):
        if self.kind == "f":
            return f"{'fmaxf' if self.is_max else 'fminf'}({_as_float_c(self.a)}, {_as_float_c(self.b)})"
        return f"({self.a.c()} {'>' if self.is_max else '<'} {self.b.c()} ? {self.a.c()} : {self.b.c()})"

    def ev(self, env):
        dt = torch.float64 if self.kind == "f" else torch.int64
        a, b = torch.as_tensor(self.a.ev(env), dtype=dt), torch.as_tensor(self.b.ev(env), dtype=dt)
        return torch.maximum(a, b) if self.is_max else torch.minimum(a, b)

    def d(self):
        if self.kind != "f" or not self.uses_s():
            return Const(0.0)
        first = Bin(">=" if self.is_max else "<=", self.a, self.b)
        return Select(first, self.a.d(), self.b.d())

    def uses_s(self):
        return self.a.uses_s() or self.b.uses_s()


class Pow(Node):
    def __init__(self, a: Node, n: int):
        self.a, self.n, self.kind = a, n, a.kind

    def c(self):
        x = self.a.c()
        return "(" + " * ".join([f"({x})"] * self.n) + ")" if self.n > 0 else ("1.0f" if self.kind == "f" else "1")

    def ev(self, env):
        return self.a.ev(env) ** self.n

    def d(self):
        if self.kind != "f" or not self.a.uses_s() or self.n == 0:
            return Const(0.0)
        return mul(mul(Const(float(self.n)), Pow(self.a, self.n - 1) if self.n > 1 else Const(1.0)), self.a.d())

    def uses_s(self):
        return self.a.uses_s()


class PowF(Node):
    """a ** b with a float result for a positive base (``2 ** (-8 * (h + 1) / 16)``, ``s ** 1.5``)."""
    def __init__(self, a: Node, b: Node):
        self.a, self.b, self.kind = a, b, "f"

    def c(self):
        return f"fa_pow({_as_float_c(self.a)}, {_as_float_c(self.b)})"

    def ev(self, env):
        return torch.pow(torch.as_tensor(self.a.ev(env), dtype=torch.float64), torch.as_tensor(self.b.ev(env), dtype=torch.float64))

    def d(self):
        if not self.uses_s():
            return Const(0.0)
        # d(a^b) = a^b (b' ln a + b a' / a)
        return mul(self, add(mul(self.b.d(), Call("log", self.a)), div(mul(self.b, self.a.d()), self.a)))

    def uses_s(self):
        return self.a.uses_s() or self.b.uses_s()


def walk(n: Node):
    yield n
    for attr in ("a", "b", "cond", "index"):
        ch = getattr(n, attr, None)
        if isinstance(ch, Node):
            yield from walk(ch)


# ------------------------------------------------------------------------------------------------
# symbolic execution of the closure's source
# ------------------------------------------------------------------------------------------------
class _Tile:
    """The q or k tile of a tile-form score function: only products and shapes are meaningful."""
    def __init__(self, which, transposed=False):
        self.which, self.transposed = which, transposed


class _Opaque:
    """A module or another object whose attributes are resolved by name only (torch, jnp, np, math ...)."""
    def __init__(self, name):
        self.name = name


class _Arange:
    def __init__(self, extent: Node):
        self.extent = extent


class Rewriter:
    def __init__(self, fn: Callable, form: str):
        self.fn, self.form = fn, form
        self.tables: Dict[str, Table] = {}
        src = textwrap.dedent(inspect.getsource(fn))
        tree = ast.parse(src)
        self.node = self._find(tree, fn)
        cv = inspect.getclosurevars(fn)
        self.outer = dict(cv.globals)
        self.outer.update(cv.nonlocals)
        self.outer.update({k: v for k, v in cv.builtins.items()})

    @staticmethod
    def _find(tree, fn):
        name = getattr(fn, "__name__", "<lambda>")
        cands = [n for n in ast.walk(tree) if (isinstance(n, ast.FunctionDef) and n.name == name)
                 or (isinstance(n, ast.Lambda) and name == "<lambda>")]
        if not cands:
            raise NotImplementedError("could not locate the function's source")
        if len(cands) > 1 and name == "<lambda>":
            n_args = fn.__code__.co_argcount
            cands = [c for c in cands if len(c.args.args) == n_args] or cands
        return cands[0]

    def fail(self, node, what):
        raise NotImplementedError(f"score / mask compiler: {what} (line {getattr(node, 'lineno', '?')}: "
                                  f"{ast.unparse(node) if hasattr(ast, 'unparse') else type(node).__name__})")

    def run(self, args: Sequence) -> Node:
        params = [a.arg for a in self.node.args.args]
        if len(params) != len(args):
            raise NotImplementedError(f"function takes {len(params)} arguments, expected {len(args)}")
        env = dict(zip(params, args))
        if isinstance(self.node, ast.Lambda):
            return self.expr(self.node.body, env)
        for st in self.node.body:
            if isinstance(st, ast.Expr) and isinstance(st.value, ast.Constant):
                continue  # docstring
            if isinstance(st, ast.Assign):
                val = self.expr(st.value, env)
                for tgt in st.targets:
                    self.assign(tgt, val, env)
            elif isinstance(st, ast.AnnAssign) and st.value is not None:
                self.assign(st.target, self.expr(st.value, env), env)
            elif isinstance(st, ast.Return):
                return self.expr(st.value, env)
            else:
                self.fail(st, "only assignments and a return are understood")
        self.fail(self.node, "function has no return")

    def assign(self, tgt, val, env):
        if isinstance(tgt, ast.Name):
            env[tgt.id] = val
        elif isinstance(tgt, (ast.Tuple, ast.List)) and isinstance(val, tuple) and len(val) == len(tgt.elts):
            for t, v in zip(tgt.elts, val):
                self.assign(t, v, env)
        else:
            self.fail(tgt, "unsupported assignment target")

    # -- values captured from the enclosing scopes ------------------------------------------------
    def lift(self, name, value, node):
        if isinstance(value, (bool, int, float, np.integer, np.floating)):
            return Const(value.item() if isinstance(value, np.generic) else value)
        if isinstance(value, torch.Tensor) and value.ndim == 0:
            return Const(value.item())
        if isinstance(value, (list, tuple, np.ndarray, torch.Tensor)):
            arr = np.asarray(value.detach().cpu() if isinstance(value, torch.Tensor) else value)
            if arr.ndim == 1 and arr.size > 0 and arr.dtype.kind in "iuf":
                vals = [int(v) if arr.dtype.kind in "iu" else float(v) for v in arr]
                return ("table", name, vals)
        if inspect.ismodule(value) or callable(value):
            return _Opaque(name)
        self.fail(node, f"captured value '{name}' of type {type(value).__name__} cannot be compiled")

    # -- expressions ----------------------------------------------------------------------------------
    def expr(self, e, env):
        if isinstance(e, ast.Constant):
            if isinstance(e.value, (bool, int, float)):
                return Const(e.value)
            if e.value is None:
                return None
            self.fail(e, "unsupported constant")
        if isinstance(e, ast.Name):
            if e.id in env:
                return env[e.id]
            if e.id in self.outer:
                return self.lift(e.id, self.outer[e.id], e)
            return _Opaque(e.id)
        if isinstance(e, ast.Tuple):
            return tuple(self.expr(x, env) for x in e.elts)
        if isinstance(e, ast.Attribute):
            base = self.expr(e.value, env)
            if isinstance(base, _Tile):
                if e.attr in ("T", "mT"):
                    return _Tile(base.which, not base.transposed)
                if e.attr == "shape":
                    return ("shape", base.which)
                if e.attr == "dtype":
                    return _Opaque("dtype")
            if isinstance(base, _Opaque):
                return _Opaque(f"{base.name}.{e.attr}")
            if isinstance(base, Node):
                return ("method", e.attr, base)
            if isinstance(base, tuple) and base and base[0] == "shape":
                self.fail(e, "unsupported shape attribute")
            self.fail(e, "unsupported attribute")
        if isinstance(e, ast.Subscript):
            return self.subscript(e, env)
        if isinstance(e, ast.UnaryOp):
            a = self.expr(e.operand, env)
            if not isinstance(a, Node):
                self.fail(e, "unsupported operand")
            if isinstance(e.op, ast.USub):
                return Const(-a.value) if isinstance(a, Const) and a.kind != "b" else Un("-", a)
            if isinstance(e.op, ast.UAdd):
                return a
            if isinstance(e.op, (ast.Not, ast.Invert)):
                if a.kind != "b":
                    self.fail(e, "'not' / '~' of a non-boolean")
                return Un("not", a)
        if isinstance(e, ast.BinOp):
            return self.binop(e, env)
        if isinstance(e, ast.BoolOp):
            vals = [self.expr(v, env) for v in e.values]
            out = vals[0]
            for v in vals[1:]:
                out = Bin("and" if isinstance(e.op, ast.And) else "or", out, v)
            return out
        if isinstance(e, ast.Compare):
            ops = {ast.Lt: "<", ast.LtE: "<=", ast.Gt: ">", ast.GtE: ">=", ast.Eq: "==", ast.NotEq: "!="}
            left = self.expr(e.left, env)
            out = None
            for op, right in zip(e.ops, e.comparators):
                r = self.expr(right, env)
                if type(op) not in ops or not isinstance(left, Node) or not isinstance(r, Node):
                    self.fail(e, "unsupported comparison")
                term = Bin(ops[type(op)], left, r)
                out = term if out is None else Bin("and", out, term)
                left = r
            return out
        if isinstance(e, ast.IfExp):
            c, a, b = self.expr(e.test, env), self.expr(e.body, env), self.expr(e.orelse, env)
            return Select(c, a, b)
        if isinstance(e, ast.Call):
            return self.call(e, env)
        self.fail(e, "unsupported expression")

    def binop(self, e, env):
        a, b = self.expr(e.left, env), self.expr(e.right, env)
        if isinstance(e.op, ast.MatMult):
            return self.dot(a, b, e)
        ops = {ast.Add: "+", ast.Sub: "-", ast.Mult: "*", ast.Div: "/", ast.FloorDiv: "//", ast.Mod: "%"}
        if not isinstance(a, Node) or not isinstance(b, Node):
            self.fail(e, "unsupported operands")
        if isinstance(e.op, ast.Pow):
            if isinstance(b, Const) and b.kind == "i" and 0 <= b.value <= 8:
                return Pow(a, b.value)
            if a.kind == "b" or b.kind == "b":
                self.fail(e, "'**' needs numbers")
            if isinstance(a, Const) and isinstance(b, Const):
                return Const(float(a.value) ** float(b.value))
            if isinstance(a, Const) and a.value <= 0:
                self.fail(e, "a power with a variable exponent needs a positive base")
            return PowF(a, b)   # (the base must be positive where it is evaluated: exp2(b log2 a) on the device)
        if isinstance(e.op, (ast.BitAnd, ast.BitOr)):
            if a.kind != "b" or b.kind != "b":
                self.fail(e, "'&' / '|' need boolean operands")
            return Bin("and" if isinstance(e.op, ast.BitAnd) else "or", a, b)
        if isinstance(e.op, ast.BitXor) and a.kind == "b" and b.kind == "b":
            return Bin("!=", a, b)
        if type(e.op) not in ops:
            self.fail(e, "unsupported operator")
        op = ops[type(e.op)]
        if isinstance(a, Const) and isinstance(b, Const) and a.kind != "b" and b.kind != "b":
            x, y = a.value, b.value
            return Const({"+": x + y, "-": x - y, "*": x * y, "/": x / y if y else float("nan"),
                          "//": x // y if y else 0, "%": x % y if y else 0}[op])
        return Bin(op, a, b)

    def dot(self, a, b, e):
        if isinstance(a, _Tile) and isinstance(b, _Tile) and a.which == "q" and not a.transposed \
                and b.which == "k" and b.transposed:
            return Var("s")
        self.fail(e, "the only matrix product understood is q_tile @ k_tile.T")

    def subscript(self, e, env):
        base = self.expr(e.value, env)
        sl = e.slice
        if isinstance(base, tuple) and base and base[0] == "shape":
            idx = self.expr(sl, env)
            if isinstance(idx, Const) and idx.value == 0:
                return Var("mq" if base[1] == "q" else "mk")
            self.fail(e, "only shape[0] of a tile is understood")
        if isinstance(base, tuple) and base and base[0] == "table":
            idx = self.expr(sl, env)
            if not isinstance(idx, Node):
                self.fail(e, "unsupported table index")
            _, name, vals = base
            cname = f"fa_tab_{name}"
            t = Table(cname, vals, Cast(idx, "i") if idx.kind == "b" else idx)
            self.tables[cname] = t
            return t
        # broadcasting subscripts x[:, None] / x[None, :] on index vectors and aranges
        if isinstance(sl, ast.Tuple) and len(sl.elts) == 2:
            kinds = ["none" if (isinstance(x, ast.Constant) and x.value is None) else
                     ("all" if isinstance(x, ast.Slice) and x.lower is None and x.upper is None and x.step is None else "?")
                     for x in sl.elts]
            if sorted(kinds) == ["all", "none"]:
                rows = kinds == ["all", "none"]
                if isinstance(base, _Arange):
                    ext = base.extent
                    if isinstance(ext, Var) and ext.name in ("mq", "mk"):
                        if (ext.name == "mq") != rows:
                            self.fail(e, "arange over the q tile must broadcast over rows, over the k tile over columns")
                        return Bin("%", Var("i"), Var("mq")) if rows else Bin("%", Var("j"), Var("mk"))
                    self.fail(e, "arange extent must be q_tile.shape[0] or k_tile.shape[0]")
                if isinstance(base, Var) and base.name in ("i", "j"):
                    if (base.name == "i") != rows:
                        self.fail(e, "q indices must broadcast over rows ([:, None]), k indices over columns ([None, :])")
                    return base
        self.fail(e, "unsupported subscript")

    def call(self, e, env):
        f = self.expr(e.func, env)
        args = [self.expr(a, env) for a in e.args]
        kw = {k.arg: self.expr(k.value, env) for k in e.keywords}
        if isinstance(f, tuple) and f and f[0] == "method":
            _, name, recv = f
            if name in ("float", "double"):
                return Cast(recv, "f")
            if name in ("long", "int"):
                return Cast(recv, "i")
            if name in ("to", "astype", "type", "bool", "detach", "clone", "contiguous"):
                return recv
            args = [recv] + args
        elif isinstance(f, _Opaque):
            name = f.name.split(".")[-1]
        else:
            self.fail(e, "unsupported call")
        name = {"absolute": "abs", "fabs": "abs", "fmin": "minimum", "fmax": "maximum"}.get(name, name)
        if name in ("matmul", "dot", "mm") and len(args) == 2:
            return self.dot(args[0], args[1], e)
        if name == "dot_general" and len(args) >= 2 and isinstance(args[0], _Tile) and isinstance(args[1], _Tile):
            # lax.dot_general(q, k, (((1,), (1,)), ((), ()))) contracts the head dimensions: q k^T
            if args[0].which == "q" and args[1].which == "k" and not args[0].transposed and not args[1].transposed:
                return Var("s")
            self.fail(e, "unsupported dot_general operands")
        if name == "transpose" and args and isinstance(args[0], _Tile):
            return _Tile(args[0].which, not args[0].transposed)
        if name == "arange" and len(args) == 1:
            return _Arange(args[0])
        if name in ("float", "float32", "float64") and len(args) == 1 and isinstance(args[0], Node):
            return Cast(args[0], "f")
        if name in ("int", "int32", "int64") and len(args) == 1 and isinstance(args[0], Node):
            return Cast(args[0], "i")
        if name in ("asarray", "as_tensor", "tensor", "array") and args and isinstance(args[0], Node):
            return args[0]
        nodes = [a for a in args if isinstance(a, Node)]
        if name in FUNCS and len(nodes) == 1 and len(args) == 1:
            return Call(name, nodes[0])
        if name in ("minimum", "maximum", "min", "max") and len(nodes) == 2 and len(args) == 2:
            return MinMax(name in ("maximum", "max"), nodes[0], nodes[1])
        if name == "where" and len(nodes) == 3:
            if nodes[0].kind != "b":
                self.fail(e, "where() needs a boolean condition")
            return Select(nodes[0], nodes[1], nodes[2])
        if name in ("clamp", "clip") and nodes:
            x = nodes[0]
            lo = kw.get("min", kw.get("a_min", args[1] if len(args) > 1 else None))
            hi = kw.get("max", kw.get("a_max", args[2] if len(args) > 2 else None))
            if isinstance(lo, Node):
                x = MinMax(True, x, lo)
            if isinstance(hi, Node):
                x = MinMax(False, x, hi)
            return x
        if name in ("logical_and", "logical_or") and len(nodes) == 2:
            return Bin("and" if name == "logical_and" else "or", nodes[0], nodes[1])
        if name == "logical_not" and len(nodes) == 1:
            return Un("not", nodes[0])
        self.fail(e, f"call to '{name}' is not understood")


# ------------------------------------------------------------------------------------------------
# code generation and the library of a functor pair
# ------------------------------------------------------------------------------------------------
@dataclass(frozen=True)
class CustomCode:
    """C bodies of a compiled closure: `kind` is 'score' or 'mask'."""
    kind: str
    body: str            # C statements + return for the function
    dbody: str = ""      # derivative (score only)
    source: str = ""     # text of the Python source, for messages

    @property
    def key(self) -> str:
        return hashlib.sha256((self.kind + "\0" + self.body + "\0" + self.dbody).encode()).hexdigest()[:16]


def _function_text(tables: Dict[str, Table], expr: Node, ret_kind: str) -> str:
    used = {n.name for n in walk(expr) if isinstance(n, Table)}
    lines = [tables[name].decl() for name in sorted(used)]
    if ret_kind == "f":
        lines.append(f"  return {_as_float_c(expr)};")
    else:
        if expr.kind != "b":
            raise NotImplementedError("a mask function must return a boolean")
        lines.append(f"  return {expr.c()};")
    return "\n".join(lines)


HEADER_PRELUDE = """// Generated by flex_attention_tpu_amd.compiler; do not edit.
#pragma once
#include <math.h>
namespace fa {
// Python's % and // on integers.  A divisor that is a power of two (tile sizes, which reach a tile-form function
// at run time, and most constants) takes a mask or a shift, which also hold for negative dividends in two's
// complement; anything else the integer division.
__host__ __device__ inline int fa_py_mod(int a, int b) {
  if (b > 0 && (b & (b - 1)) == 0) return a & (b - 1);
  const int r = a % b;
  return (r != 0 && ((r < 0) != (b < 0))) ? r + b : r;
}
__host__ __device__ inline int fa_py_floordiv(int a, int b) {
  if (b > 0 && (b & (b - 1)) == 0) return a >> __builtin_ctz((unsigned)b);
  const int q = a / b;
  return ((a % b != 0) && ((a < 0) != (b < 0))) ? q - 1 : q;
}
__host__ __device__ inline float fa_py_fmod(float a, float b) { const float r = fmodf(a, b); return (r != 0.f && ((r < 0.f) != (b < 0.f))) ? r + b : r; }
// Elementary functions: on the device the hardware's exp2 / log2 / rcp / sqrt (the arithmetic the kernels' own
// softmax and soft-cap use; tanh as 1 - 2 / (e^2x + 1) saturates correctly and is good to a few 1e-7 absolute),
// a handful of instructions per score where the library routines take several dozen; on the host, where the tests
// evaluate the generated code, libm.
__host__ __device__ inline float fa_exp(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_exp2f(x * 1.4426950408889634f);
#else
  return expf(x);
#endif
}
__host__ __device__ inline float fa_log(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_logf(x) * 0.6931471805599453f;
#else
  return logf(x);
#endif
}
__host__ __device__ inline float fa_pow(float a, float b) {   // (a > 0)
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_exp2f(b * __builtin_amdgcn_logf(a));
#else
  return powf(a, b);
#endif
}
__host__ __device__ inline float fa_sqrt(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_sqrtf(x);
#else
  return sqrtf(x);
#endif
}
__host__ __device__ inline float fa_tanh(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
  return 1.0f - 2.0f * __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(x * 2.8853900817779268f) + 1.0f);
#else
  return tanhf(x);
#endif
}
__host__ __device__ inline float fa_sigmoid(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
#else
  return 1.0f / (1.0f + expf(-x));
#endif
}
"""


def header_text(score: Optional[CustomCode], mask: Optional[CustomCode]) -> str:
    """The header a functor library is compiled against: custom_score / custom_dscore (value and
    derivative of the modified score with respect to s = sm_scale <q, k>) and custom_keep."""
    s_body = score.body if score else "  return s;"
    d_body = score.dbody if score else "  return 1.0f;"
    m_body = mask.body if mask else "  return true;"
    tag = functor_key(score, mask)
    return (HEADER_PRELUDE
            + f"#define FLEXATTN_CUSTOM_TAG \"{tag}\"\n"
            + f"#define FLEXATTN_CUSTOM_HAS_SCORE {1 if score else 0}\n"
            + f"#define FLEXATTN_CUSTOM_HAS_MASK {1 if mask else 0}\n"
            + "__host__ __device__ inline float custom_score(float s, int b, int h, int i, int j, int mq, int mk) {\n"
            + s_body + "\n}\n"
            + "__host__ __device__ inline float custom_dscore(float s, int b, int h, int i, int j, int mq, int mk) {\n"
            + d_body + "\n}\n"
            + "__host__ __device__ inline bool custom_keep(int i, int j) {\n" + m_body + "\n}\n"
            + "}  // namespace fa\n")


_sources_digest = None


def sources_digest() -> str:
    """Hash of the kernel sources a functor library is compiled from: a change there makes a new library."""
    global _sources_digest
    if _sources_digest is None:
        h = hashlib.sha256()
        csrc = os.path.join(PKG_DIR, "csrc")
        files = sorted(f for f in os.listdir(csrc) if f.endswith((".hip", ".hpp", ".py")))
        for path in [os.path.join(csrc, f) for f in files] + [os.path.join(os.path.dirname(PKG_DIR), "include", "flexattn.h")]:
            with open(path, "rb") as f:
                h.update(f.read())
        _sources_digest = h.hexdigest()[:16]
    return _sources_digest


def functor_key(score: Optional[CustomCode], mask: Optional[CustomCode]) -> str:
    text = f"v{CODEGEN_VERSION}|{sources_digest()}|{score.key if score else '-'}|{mask.key if mask else '-'}"
    return hashlib.sha256(text.encode()).hexdigest()[:16]


def library_path(score: Optional[CustomCode], mask: Optional[CustomCode]) -> str:
    key = functor_key(score, mask)
    return os.path.join(JIT_DIR, key, f"libflexattn_{key}.so")


def build_functor_library(score: Optional[CustomCode], mask: Optional[CustomCode], force: bool = False) -> str:
    """Compiles (hipcc, gfx950) the library of a functor pair unless it is cached; returns its path."""
    from . import build as B
    import fcntl
    path = library_path(score, mask)
    if os.path.exists(path) and not force:
        return path
    d = os.path.dirname(path)
    os.makedirs(d, exist_ok=True)
    # one builder per functor pair at a time (processes that compile the same closures at once: ranks of a job,
    # test workers); everything is written inside the pair's own directory, the library under a temporary name
    with open(os.path.join(d, ".lock"), "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)
        try:
            if os.path.exists(path) and not force:   # (another process built it while this one waited)
                return path
            header = os.path.join(d, "custom_functor.hpp")
            tmp = f"{header}.{os.getpid()}.tmp"
            with open(tmp, "w") as f:
                f.write(header_text(score, mask))
            os.replace(tmp, header)
            flags = [f'-DFLEXATTN_CUSTOM_HEADER="{header}"']
            if score is not None:
                flags.append("-DFLEXATTN_CUSTOM_ONLY")   # a custom score runs the compiled-loop kernels: skip the generated streams
            obj = os.path.join(d, "obj")
            B.build_library(force=True, out_path=path, build_dir=obj, extra_flags=flags, include_dir=obj)
        finally:
            fcntl.flock(lock, fcntl.LOCK_UN)
    return path


# ------------------------------------------------------------------------------------------------
# front ends
# ------------------------------------------------------------------------------------------------
def _probe_env(n=48, seed=7):
    g = torch.Generator().manual_seed(seed)
    i = torch.randint(0, 4096, (n, 1), generator=g)
    j = torch.randint(0, 4096, (1, n), generator=g)
    s = torch.randn(n, n, generator=g, dtype=torch.float64) * 6.0
    return {"s": s, "i": i, "j": j, "b": 1, "h": 2, "mq": 128, "mk": 128}


def _check_against_python(expr: Node, fn: Callable, form: str):
    """The rewritten tree must reproduce the Python function on random probes."""
    env = _probe_env()
    got = torch.as_tensor(expr.ev(env))
    try:
        if form == "score_mod":
            want = fn(env["s"], env["b"], env["h"], env["i"], env["j"])
        elif form == "mask":
            want = fn(env["i"].flatten(), env["j"].flatten())
        else:
            return  # tile form: checked by the caller on tiles
        want = torch.as_tensor(want)
    except Exception as e:  # noqa: BLE001
        raise NotImplementedError(f"the function could not be evaluated on torch probes: {e}") from e
    got = got.expand_as(want) if got.ndim <= want.ndim else got
    ok = torch.equal(got.to(torch.bool), want.to(torch.bool)) if form == "mask" else \
        torch.allclose(got.to(torch.float64), want.to(torch.float64), rtol=2e-6, atol=2e-6)
    # (the tolerance of float32: torch evaluates a Python float times an integer index tensor in float32, the tree
    # in float64; a misread construct differs by far more)
    if not ok:
        raise NotImplementedError("the compiled expression does not reproduce the Python function on random probes "
                                  "(a construct was misread): " + (inspect.getsource(fn).strip()[:200]))


MAX_OPEN_HEADS = 256   # heads for which a slope computed from the head's index is checked ahead of the call


def _recognised_score_spec(expr: Node):
    """The ScoreSpec of a functor the kernels carry themselves (plain scores, tanh soft-cap, ALiBi with global
    indices and a slope per head) if the expression equals one, else None.  Numeric, on the expression tree in
    float64: soft-cap logits far into saturation give the cap, one (i, j) pair gives a head's slope, and the closed
    form must then reproduce the expression on every probe (random and extreme logits, indices up to 70000,
    several batch entries, every head).  A slope per head needs the number of heads: only functions that take it
    from a table indexed by ``h`` qualify, and the table's length is the number of heads of the specification."""
    from . import _lib
    from .scores import ScoreSpec
    nodes = list(walk(expr))
    names = {n.name for n in nodes if isinstance(n, Var)}
    if names & {"mq", "mk"}:
        return None
    head_tables = [n for n in nodes if isinstance(n, Table) and isinstance(n.index, Var) and n.index.name == "h"]
    other_h = any(isinstance(n, Var) and n.name == "h" for n in nodes) and \
        sum(1 for n in nodes if isinstance(n, Var) and n.name == "h") != len(head_tables)
    H = min((len(t.values) for t in head_tables), default=None)
    g = torch.Generator().manual_seed(5)
    s = torch.cat([torch.randn(61, generator=g, dtype=torch.float64) * 4.0,
                   torch.tensor([0.0, 1e5, -1e5], dtype=torch.float64)])[:, None, None]
    i = torch.tensor([0, 1, 5, 130, 4095, 70000])[None, :, None]
    j = torch.tensor([0, 2, 5, 131, 4000, 65536])[None, None, :]
    shape = (s.shape[0], i.shape[1], j.shape[2])

    def ev(b, h):
        out = torch.as_tensor(expr.ev({"s": s, "b": b, "h": h, "i": i, "j": j}), dtype=torch.float64)
        return out.expand(shape) if out.ndim else out.reshape(1, 1, 1).expand(shape)
    try:
        heads = list(range(H)) if H is not None else [0, 1, 5]
        outs = {(b, h): ev(b, h) for b in (0, 3) for h in heads}
    except Exception:  # noqa: BLE001  (a probe outside the function's domain: no closed form claimed)
        return None
    if not all(bool(torch.isfinite(o).all()) for o in outs.values()):
        return None
    se = s.expand(shape)
    if all(bool(((o - se).abs() <= 1e-12 * (1.0 + se.abs())).all()) for o in outs.values()):
        return ScoreSpec(kind=_lib.SCORE_NONE)
    first = outs[(0, heads[0])]
    same_everywhere = all(torch.equal(o, first) for o in outs.values()) and \
        bool((first == first[:, :1, :1]).all())
    if same_everywhere:
        cap = float(first[-2, 0, 0])   # the logit 1e5
        if cap > 0.0 and bool(((first - cap * torch.tanh(se / cap)).abs() <= 1e-9 * (1.0 + cap)).all()):
            return ScoreSpec(kind=_lib.SCORE_SOFTCAP, cap=cap)
        return None
    dist = (j - i).to(torch.float64).expand(shape)

    def slope_of(h):
        """The head's slope if the expression is s + slope (j - i) for it, on every probe and batch entry."""
        o0 = outs[(0, h)] if (0, h) in outs else ev(0, h)
        a = float((o0 - se)[0, 0, 1] / dist[0, 0, 1])
        for b in (0, 3):
            o = outs[(b, h)] if (b, h) in outs else ev(b, h)
            if not bool(torch.isfinite(o).all()) or \
                    not bool(((o - se - a * dist).abs() <= 1e-9 * (1.0 + abs(a) * dist.abs())).all()):
                return None
        return a
    if H is not None and not other_h:   # slopes from a table: as many heads as the table has entries
        slopes = [slope_of(h) for h in heads]
        return ScoreSpec(kind=_lib.SCORE_ALIBI, slopes=tuple(slopes)) if None not in slopes else None
    # slopes computed from h (2 ** (-8 (h + 1) / H) and the like): checked for the first MAX_OPEN_HEADS heads, of
    # which a call takes as many as it has
    slopes = []
    try:
        for h in range(MAX_OPEN_HEADS):
            slopes.append(slope_of(h))
    except Exception:  # noqa: BLE001  (a table that ends, a domain error: the heads so far)
        pass
    if None in slopes or len(slopes) < 1 or (H is not None and len(slopes) < H):
        return None
    return ScoreSpec(kind=_lib.SCORE_ALIBI, slopes=None, slopes_open=tuple(slopes))


def compile_score_mod(fn: Callable, recognise: bool = True) -> Callable:
    """``fn(s, b, h, q_idx, kv_idx) -> s'`` (element-wise; s = sm_scale <q, k>, global indices) compiled into
    the kernels.  Returns a closure with the same call signature carrying ``.spec``.  A function that equals one
    of the kernels' own functors (the identity, ``cap * tanh(s / cap)``, ``s + SLOPES[h] * (kv_idx - q_idx)``) gets
    that functor's specification, and with it the generated-stream kernels, instead of a compiled functor
    (``recognise=False`` compiles it regardless)."""
    from . import _lib
    from .scores import ScoreSpec
    rw = Rewriter(fn, "score_mod")
    expr = rw.run([Var("s"), Var("b"), Var("h"), Var("i"), Var("j")])
    if not isinstance(expr, Node) or expr.kind == "b":
        raise NotImplementedError("a score function must return a number")
    _check_against_python(expr, fn, "score_mod")
    code = CustomCode("score", _function_text(rw.tables, expr, "f"), _function_text(rw.tables, expr.d(), "f"),
                      inspect.getsource(fn).strip())

    def score_mod(s, b, h, q_idx, kv_idx):
        return fn(s, b, h, q_idx, kv_idx)
    builtin = _recognised_score_spec(expr) if recognise else None
    score_mod.spec = builtin if builtin is not None else ScoreSpec(kind=_lib.SCORE_CUSTOM, custom=code)
    score_mod.expr = expr
    score_mod.__wrapped__ = fn
    return score_mod


def compile_score_fn(fn: Callable) -> Callable:
    """Tile form of the reference, ``fn(q_tile, k_tile) -> [Bq, Bk]`` (scores.py:3-18): ``q_tile @ k_tile.T``
    (or dot / matmul / dot_general of the two) becomes ``s``; ``arange(q_tile.shape[0])[:, None]`` and
    ``arange(k_tile.shape[0])[None, :]`` become the row / column inside the (block_q, block_k) tile the
    entry points are called with."""
    from . import _lib
    from .scores import ScoreSpec
    rw = Rewriter(fn, "tile")
    expr = rw.run([_Tile("q"), _Tile("k")])
    if not isinstance(expr, Node) or expr.kind == "b":
        raise NotImplementedError("a score function must return a number")
    # check on a tile: rows / columns are tile-local, so i, j run over one tile from zero
    g = torch.Generator().manual_seed(11)
    m, n, dd = 24, 40, 16
    q = torch.randn(m, dd, generator=g, dtype=torch.float64)
    k = torch.randn(n, dd, generator=g, dtype=torch.float64)
    try:
        want = torch.as_tensor(fn(q, k)).to(torch.float64)
    except Exception as e:  # noqa: BLE001
        raise NotImplementedError(f"score function could not be evaluated on torch tiles: {e}") from e
    env = {"s": q @ k.T, "i": torch.arange(m)[:, None], "j": torch.arange(n)[None, :], "b": 0, "h": 0, "mq": m, "mk": n}
    got = torch.as_tensor(expr.ev(env)).to(torch.float64)
    if want.shape != (m, n) or not torch.allclose(got.expand(m, n), want, rtol=1e-9, atol=1e-9):
        raise NotImplementedError("the compiled expression does not reproduce the Python function on a probe tile")
    code = CustomCode("score", _function_text(rw.tables, expr, "f"), _function_text(rw.tables, expr.d(), "f"),
                      inspect.getsource(fn).strip())

    def score_fn(q_tile, k_tile):
        return fn(q_tile, k_tile)
    score_fn.spec = ScoreSpec(kind=_lib.SCORE_CUSTOM, custom=code)
    score_fn.expr = expr
    score_fn.__wrapped__ = fn
    return score_fn


def _recognised_mask_fns(expr: Node, block_q: int, block_k: int):
    """The (mask_fn, block_mask_fn) pair of this package's own factories (causal, sliding window, both, the S2 local
    + strided mask) if the predicate equals one of them, else None: those masks have closed-form block maps and run the generated-stream
    kernels.  Numeric, on the expression tree: the keys kept by one query far out (position 2^22) give the
    candidate's window, and the factory's own ``mask_fn`` must then agree with the predicate on index grids around
    the origin, around that query and around both ends of its window."""
    from . import masks
    i0 = 1 << 22

    def ev(qi, kj):
        out = torch.as_tensor(expr.ev({"i": qi[:, None], "j": kj[None, :]}))
        return out.to(torch.bool).expand(qi.numel(), kj.numel())
    try:
        row = ev(torch.tensor([i0]), torch.arange(0, i0 + 64))[0]
    except Exception:  # noqa: BLE001
        return None
    kept = torch.nonzero(row).flatten()
    if kept.numel() == 0:
        return None
    causal = int(kept[-1]) == i0
    if not causal and int(kept[-1]) != i0 + 63:
        return None
    # the run of kept keys that ends at the query is the window; kept keys in front of it at equal distances from
    # key 0 on are the strided part of the reference's S2 mask (masks.py:143-179)
    gaps = torch.nonzero(kept[1:] - kept[:-1] != 1).flatten()
    run_start = int(kept[int(gaps[-1]) + 1]) if gaps.numel() else int(kept[0])
    stride = None
    if causal and gaps.numel() and int(kept[0]) == 0 and kept.numel() > 1:
        stride = int(kept[1])
    window = i0 - run_start + 1 if run_start > 0 else None
    if not causal and window is None:
        return None      # (keeps everything: no mask is the caller's way to say so)
    if stride is not None and window is not None and stride > 1:
        # (a strided key right in front of the window joins its run: the window one shorter is tried as well)
        cands = [masks.make_s2_mask_fns(block_q, block_k, w_, stride) for w_ in (window, window - 1) if w_ > 0]
    elif gaps.numel():
        return None      # (kept keys in pieces that are no S2 pattern)
    elif causal and window is None:
        cands = [masks.make_causal_mask_fns(block_q, block_k)]
    elif causal:
        cands = [masks.make_causal_sliding_window_mask_fns(block_q, block_k, window)]
    else:
        cands = [masks.make_sliding_window_mask_fns(block_q, block_k, window)]
    w = window or 0
    grids = [(torch.arange(0, 320), torch.arange(0, 320)),
             (torch.arange(i0 - 96, i0 + 96), torch.arange(i0 - 96, i0 + 96)),
             (torch.arange(i0 - 96, i0 + 96), torch.arange(max(0, i0 - w - 96), i0 - w + 96)),
             (torch.arange(max(0, w - 96), w + 96), torch.arange(0, 192)),
             (torch.arange(1000, 1192), torch.arange(0, 1200))]
    try:
        want = [ev(qi, kj) for qi, kj in grids]
        for cand in cands:
            if all(torch.equal(x, torch.as_tensor(cand[0](qi, kj)).to(torch.bool)) for x, (qi, kj) in zip(want, grids)):
                return cand
    except Exception:  # noqa: BLE001
        return None
    return None


def compile_mask_fn(fn: Callable, block_q: int, block_k: int, recognise: bool = True) -> Tuple[Callable, Callable]:
    """``fn(q_idx, k_idx) -> bool[Bq, Bk]`` on 1-D global index arrays (the reference's ``mask_fn``,
    masks.py:15-16) compiled into the kernels.  Returns ``(mask_fn, block_mask_fn)``: the block closure is
    ``any(mask_fn over the tile)``, which the GPU builder reproduces bit for bit by evaluating the compiled
    predicate on every element of every tile.  A predicate that equals one of this package's own masks (causal,
    sliding window, both) returns that factory's pair instead: a closed-form block map and the generated-stream
    kernels (``recognise=False`` compiles it regardless)."""
    from . import _lib
    from .masks import MaskSpec
    rw = Rewriter(fn, "mask")
    expr = rw.run([Var("i"), Var("j")])
    if not isinstance(expr, Node) or expr.kind != "b":
        raise NotImplementedError("a mask function must return a boolean")
    if any(isinstance(n, Var) and n.name not in ("i", "j") for n in walk(expr)):
        raise NotImplementedError("a mask function may depend on q_idx and k_idx only")
    _check_against_python(expr, fn, "mask")
    if recognise:
        builtin = _recognised_mask_fns(expr, block_q, block_k)
        if builtin is not None:
            return builtin
    code = CustomCode("mask", _function_text(rw.tables, expr, "b"), "", inspect.getsource(fn).strip())
    spec = MaskSpec(flags=_lib.MASK_CUSTOM, custom=code)

    def mask_fn(q_idx, k_idx):
        return fn(q_idx, k_idx)

    def block_mask_fn(q_block_idx, k_block_idx):
        qi = torch.arange(q_block_idx * block_q, (q_block_idx + 1) * block_q)
        kj = torch.arange(k_block_idx * block_k, (k_block_idx + 1) * block_k)
        return bool(torch.as_tensor(fn(qi, kj)).any())
    mask_fn.spec = block_mask_fn.spec = spec
    mask_fn.expr = expr
    return mask_fn, block_mask_fn
