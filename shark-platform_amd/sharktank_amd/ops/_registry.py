"""Type-dispatched operator registry with the plug-in protocol of sharktank.ops
(sharktank/sharktank/ops/_registry.py:174-318): an `@overridable` signature owns a list of overrides keyed by
argument types; a call walks the matching overrides from the most to the least salient (later registration
wins among equals) until one returns something other than `NotImplemented`; if none does, the call fails with
`NotImplementedError("Overridable operator ... does not have an implementation for argument types: [...]")`.
"""

from __future__ import annotations

import functools
from typing import Any, Callable, Iterable, List, Optional, Tuple

from torch import Tensor

from ..types.tensors import PrimitiveTensor, QuantizedTensor

__all__ = [
    "AllOfExprs",
    "AllOfExprsVariadic",
    "AllOfType",
    "AnyOfType",
    "BoolTypeExpr",
    "IsOfType",
    "SignatureDispatcher",
    "overridable",
    "_test_enable_last_op_dispatch",
    "_test_get_last_op_dispatch",
]

_track_last_dispatch = False
_last_dispatch = None


def _test_enable_last_op_dispatch(en: bool = True):
    global _track_last_dispatch, _last_dispatch
    _last_dispatch = None
    _track_last_dispatch = en


def _test_get_last_op_dispatch():
    assert _track_last_dispatch, "Cannot get last op dispatched without calling _test_enable_last_op_dispatch()"
    return _last_dispatch


class BoolTypeExpr:
    """A predicate over the tuple of argument types."""

    def __init__(self, expr: Callable[..., bool]):
        self._expr = expr

    def __call__(self, *types: type) -> bool:
        return self._expr(*types)


class AllOfType(BoolTypeExpr):
    """Every argument type is a subclass of one of `types`."""

    def __init__(self, *types: type):
        self._types = types
        super().__init__(lambda *ts: all(any(issubclass(t, r) for r in types) for t in ts))


IsOfType = AllOfType


class AnyOfType(BoolTypeExpr):
    """At least one argument type is a subclass of one of `types`."""

    def __init__(self, *types: type):
        self._types = types
        super().__init__(lambda *ts: any(issubclass(t, r) for t in ts for r in types))


class AllOfExprs(BoolTypeExpr):
    """Argument i satisfies expression i (extra arguments are ignored)."""

    def __init__(self, *exprs: BoolTypeExpr):
        self._exprs = exprs
        super().__init__(lambda *ts: len(ts) >= len(exprs) and all(e(t) for e, t in zip(exprs, ts)))


class AllOfExprsVariadic(BoolTypeExpr):
    """Like AllOfExprs, and trailing arguments must satisfy the last expression."""

    def __init__(self, *exprs: BoolTypeExpr):
        if not exprs:
            raise ValueError("At least one expression is required.")
        self._exprs = list(exprs)

        def expr(*ts: type):
            if len(ts) < len(exprs):
                return False
            padded = list(exprs) + [exprs[-1]] * (len(ts) - len(exprs))
            return all(e(t) for e, t in zip(padded, ts))

        super().__init__(expr)


class _Override:
    __slots__ = ("salience", "order", "target", "type_spec", "auto_unbox", "auto_dequant")

    def __init__(self, salience, order, target, type_spec, auto_unbox, auto_dequant):
        self.salience, self.order, self.target = salience, order, target
        self.type_spec, self.auto_unbox, self.auto_dequant = type_spec, auto_unbox, auto_dequant

    def matches(self, arg_types: Tuple[type, ...]) -> bool:
        spec = self.type_spec
        if spec and isinstance(spec[0], BoolTypeExpr):
            if len(spec) > 1:
                raise TypeError(f"Override with multiple arguments not allowed when using BoolTypeExpr. Type spec: {spec}")
            return spec[0](*arg_types)
        if len(spec) != len(arg_types):
            return False
        for want, have in zip(spec, arg_types):
            if want is None or issubclass(have, want):
                continue
            if issubclass(want, Tensor):
                if self.auto_unbox and issubclass(have, PrimitiveTensor):
                    continue
                if self.auto_dequant and issubclass(have, QuantizedTensor):
                    continue
            return False
        return True


class SignatureDispatcher:
    def __init__(self, sigf: Callable):
        self._overrides: List[_Override] = []
        self._cache: dict = {}
        self._trampoline: Optional[Callable] = None
        self._count = 0

    def __call__(self, *args, **kwargs):
        assert self._trampoline is not None
        selected, *results = self._trampoline(self, *args, **kwargs)
        if _track_last_dispatch:
            global _last_dispatch
            _last_dispatch = selected
        if len(results) == 1:
            return results[0]
        return None if not results else results

    def override(self, *type_spec, salience: int = 0, auto_unbox: bool = True, auto_dequant: bool = False):
        def decorator(f):
            if f.__name__ == "_":
                f.__name__ = f"{self.__name__}__override"
            self._count += 1
            self._overrides.append(_Override(salience, self._count, f, type_spec, auto_unbox, auto_dequant))
            self._overrides.sort(key=lambda o: (o.salience, o.order))
            self._cache.clear()
            return f

        return decorator

    def find_overrides(self, tensors: Iterable[Any]) -> Iterable[Callable]:
        """Matching override targets, most salient (then most recently registered) first."""
        key = tuple(type(t) for t in tensors)
        found = self._cache.get(key)
        if found is None:
            found = [o.target for o in self._overrides if o.matches(key)]
            self._cache[key] = found
        return reversed(found)

    def fail(self, tensors: Iterable[Any]):
        spec = [type(t) for t in tensors]
        raise NotImplementedError(
            f"Overridable operator {self.__module__}.{self.__qualname__} does not "
            f"have an implementation for argument types: {spec}"
        )

    def trampoline(self, trampoline: Callable):
        assert self._trampoline is None
        self._trampoline = trampoline


def overridable(f):
    dispatcher = SignatureDispatcher(f)
    functools.update_wrapper(dispatcher, f)
    return dispatcher
