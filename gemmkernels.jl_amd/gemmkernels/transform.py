"""Transforms: elementwise functions applied where data moves between memory levels
(reference src/transform.jl:20-30).

A Julia closure cannot cross a C ABI, so ``Elementwise`` lowers its function to a short list of ops
from a closed vocabulary (scale, add, relu, neg, abs, clamp, square).  The function is traced by
calling it once on a symbolic value: arithmetic with constants and the helpers ``relu``, ``clamp``,
``maximum``, ``square`` are recognised; anything else raises ConfigError.  Ops are evaluated in fp32
on the device, one rounding per op.
"""
from __future__ import annotations

from typing import Callable, List, Optional, Tuple

from .errors import ConfigError

IDENTITY, SCALE, ADD, RELU, NEG, ABS, CLAMP, SQUARE = range(8)
MAX_OPS = 4


class _Sym:
    """Symbolic scalar that records the ops applied to it."""

    def __init__(self, ops=()):
        self.ops: Tuple[Tuple[int, float, float], ...] = tuple(ops)

    def _with(self, op):
        return _Sym(self.ops + (op,))

    @staticmethod
    def _const(v) -> float:
        if isinstance(v, _Sym):
            raise ConfigError("unsupported transform: only arithmetic with constants can be lowered")
        return float(v)

    def __mul__(self, v):
        if v is self:
            return self._with((SQUARE, 0.0, 0.0))
        return self._with((SCALE, self._const(v), 0.0))

    __rmul__ = __mul__

    def __truediv__(self, v):
        return self._with((SCALE, 1.0 / self._const(v), 0.0))

    def __add__(self, v):
        return self._with((ADD, self._const(v), 0.0))

    __radd__ = __add__

    def __sub__(self, v):
        return self._with((ADD, -self._const(v), 0.0))

    def __rsub__(self, v):
        return self._with((NEG, 0.0, 0.0))._with((ADD, self._const(v), 0.0))

    def __neg__(self):
        return self._with((NEG, 0.0, 0.0))

    def __pos__(self):
        return self

    def __abs__(self):
        return self._with((ABS, 0.0, 0.0))

    def __pow__(self, p):
        if p == 2:
            return self._with((SQUARE, 0.0, 0.0))
        raise ConfigError("unsupported transform: only x**2 can be lowered")

    def __bool__(self):
        raise ConfigError("unsupported transform: data-dependent control flow cannot be lowered; "
                          "use Transform.relu / Transform.maximum / Transform.clamp")

    __lt__ = __gt__ = __le__ = __ge__ = lambda self, other: self.__bool__()


def relu(x):
    """max(x, 0)"""
    return x._with((RELU, 0.0, 0.0)) if isinstance(x, _Sym) else max(x, 0)


def maximum(x, lo):
    if isinstance(x, _Sym):
        return relu(x) if float(lo) == 0.0 else x._with((CLAMP, float(lo), float("inf")))
    return max(x, lo)


def clamp(x, lo, hi):
    return x._with((CLAMP, float(lo), float(hi))) if isinstance(x, _Sym) else min(max(x, lo), hi)


def square(x):
    return x._with((SQUARE, 0.0, 0.0)) if isinstance(x, _Sym) else x * x


def identity(x):
    return x


class Elementwise:
    """``Transform.Elementwise(f)``; ``Elementwise()`` is the identity (src/transform.jl:24)."""

    def __init__(self, func: Optional[Callable] = None, ops: Optional[List[Tuple[int, float, float]]] = None,
                 expr: Optional[str] = None):
        self.func = identity if func is None else func
        self.expr = expr
        if expr is not None:
            # a C expression in the fp32 variable x, outside the closed vocabulary: the launch compiles
            # a kernel specialised for it at run time (the counterpart of the reference inlining an
            # arbitrary Julia functor, src/transform.jl:26-30)
            if "x" not in expr:
                raise ConfigError("unsupported transform: the expression does not depend on x")
            self.ops = ()
            return
        if ops is not None:
            self.ops = tuple((int(k), float(p0), float(p1)) for k, p0, p1 in ops)
        else:
            out = self.func(_Sym())
            if not isinstance(out, _Sym):
                raise ConfigError("unsupported transform: the function does not depend on its argument")
            self.ops = tuple(op for op in out.ops if op[0] != IDENTITY)
        if len(self.ops) > MAX_OPS:
            raise ConfigError(f"unsupported transform: more than {MAX_OPS} elementwise ops in one hook")

    @property
    def is_identity(self) -> bool:
        return len(self.ops) == 0 and self.expr is None

    def c_expression(self) -> Optional[str]:
        """The hook as a C expression in x (None for the identity): the given expression, or the op
        list spelled with the helper functions every specialised kernel is compiled with."""
        if self.expr is not None:
            return self.expr
        if not self.ops:
            return None

        def lit(v: float) -> str:
            import numpy as np
            return float(np.float32(v)).hex() + "f"          # exact binary32 literal

        e = "x"
        for kind, p0, p1 in self.ops:
            if kind == SCALE:
                e = f"({e} * {lit(p0)})"
            elif kind == ADD:
                e = f"({e} + {lit(p0)})"
            elif kind == RELU:
                e = f"gk_relu({e})"
            elif kind == NEG:
                e = f"(-{e})"
            elif kind == ABS:
                e = f"gk_abs({e})"
            elif kind == CLAMP:
                e = f"gk_clamp({e}, {lit(p0)}, {lit(p1)})"
            elif kind == SQUARE:
                e = f"gk_square({e})"
        return e

    def __call__(self, x, tile=None):
        """Host evaluation (src/transform.jl:26)."""
        return self.func(x)

    def __repr__(self):
        return f"Transform.Elementwise(expr={self.expr!r})" if self.expr is not None else f"Transform.Elementwise({list(self.ops)})"
