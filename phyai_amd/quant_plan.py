"""Active quantization plan: which layers get which weight spec.

A small restatement of the reference's plan plumbing
(``phyai/layers/quant/plan.py:15-70``, ``active.py:16-35``,
``materialize.py:13-23``): a ``QuantPlan`` is an ordered list of
``(glob pattern over the dotted layer prefix, spec factory)`` rules plus a
default; ``use_quant_plan(plan)`` installs it for the duration of model
construction and every linear layer built without an explicit ``spec=`` asks it.
There is no arithmetic here.
"""

from __future__ import annotations

import contextlib
import contextvars
import dataclasses
import fnmatch
from typing import Callable, Iterator

from phyai_amd.quant import Bf16Spec, Fp8Spec, Granularity

SpecFactory = Callable[[], object]


def _lower(target) -> object | None:
    """A rule's right-hand side -> spec: ``None`` (skip), a spec factory, or a semantic
    ``QuantScheme`` (lowered as the reference's ``materialize`` does)."""
    if target is None:
        return None
    if callable(target):
        return target()
    from phyai_amd.quant.scheme import QuantScheme, materialize

    if isinstance(target, QuantScheme):
        return materialize(target)
    return target


@dataclasses.dataclass
class QuantPlan:
    """Ordered rule table; the first matching rule decides (reference ``plan.py:43-70``).  A rule is
    a ``Rule(Matcher, QuantScheme | None)`` - what the config importers produce - or, as a
    shorthand, ``(glob over the layer prefix, spec factory)``; ``ignore`` globs are checked first."""

    rules: list = dataclasses.field(default_factory=list)
    default: object | None = None
    ignore: list[str] = dataclasses.field(default_factory=list)

    def resolve(self, prefix: str, layer_cls: type | None = None) -> object | None:
        if any(fnmatch.fnmatchcase(prefix, pat) for pat in self.ignore):
            return None
        for rule in self.rules:
            if isinstance(rule, tuple):
                pat, target = rule
                if fnmatch.fnmatchcase(prefix, pat):
                    return _lower(target)
            elif rule.matcher.matches(prefix, layer_cls):
                return _lower(rule.scheme)
        return _lower(self.default)

    @staticmethod
    def fp8_per_channel(ignore: list[str] | None = None) -> "QuantPlan":
        """Every linear becomes W8A8 fp8 with per-channel weight scales, except ``ignore`` globs."""
        return QuantPlan(default=lambda: Fp8Spec(granularity=Granularity.PER_CHANNEL), ignore=list(ignore or []))


_ACTIVE: contextvars.ContextVar[QuantPlan | None] = contextvars.ContextVar("phyai_amd_quant_plan", default=None)


def get_active_plan() -> QuantPlan | None:
    return _ACTIVE.get()


@contextlib.contextmanager
def use_quant_plan(plan: QuantPlan | None) -> Iterator[None]:
    token = _ACTIVE.set(plan)
    try:
        yield
    finally:
        _ACTIVE.reset(token)


def resolve_spec(*, scheme: object | None, prefix: str, layer_cls: type | None) -> object | None:
    """``scheme`` (a spec factory or a spec instance) wins over the active plan."""
    if scheme is not None:
        return scheme() if callable(scheme) else scheme
    plan = get_active_plan()
    if plan is not None and prefix:
        return plan.resolve(prefix, layer_cls)
    return None


__all__ = ["QuantPlan", "get_active_plan", "use_quant_plan", "resolve_spec", "Bf16Spec"]
