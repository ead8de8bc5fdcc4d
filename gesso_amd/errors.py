"""Typed failures of the engine.

The reference gives every failure a code and a detail dictionary
(``src/errors.jl:39-56``, ``:90-97``).  Here each code is an exception class so callers
can catch the kind they can act on; ``detail`` carries the named fields.
"""
from __future__ import annotations


class GessoError(Exception):
    """Base of all engine failures; ``detail`` holds named facts about the failure."""

    code = "ERR_RUNTIME"

    def __init__(self, message: str, **detail):
        super().__init__(message)
        self.detail = detail

    def __str__(self):
        base = super().__str__()
        if not self.detail:
            return base
        facts = ", ".join(f"{k}={v!r}" for k, v in self.detail.items() if k != "results")   # results: whole outputs
        return f"{base} ({facts})" if facts else base


class ConfigError(GessoError, ValueError):
    """A configuration that is malformed or asks for what the architecture does not have."""

    code = "ERR_INVALID_CONFIG"


class WeightError(GessoError):
    """Missing, unexpected or wrongly shaped tensors; lists all of them at once."""

    code = "ERR_INVALID_WEIGHTS"


class ResourceLimit(GessoError):
    """A pool (pages, slots) or a request's context is exhausted (``kv_manager.jl:246-257``)."""

    code = "ERR_RESOURCE_LIMIT"


class OutOfPages(ResourceLimit):
    """No free page in a group's pool: a scheduler event, not a fault of the request."""


class OutOfSlots(ResourceLimit):
    """No free state slot."""


class InvalidPlan(GessoError, ValueError):
    """A call that cannot be carried out as asked (bad ids, unknown request, bad sizes)."""

    code = "ERR_INVALID_PLAN"


class NumericalInstability(GessoError):
    """Non-finite logits where a token was to be chosen (``session.jl:444-458``)."""

    code = "ERR_NUMERICAL_INSTABILITY"


class StepFailed(GessoError):
    """A step broke off after it had begun to write the cache; ``detail["requests"]`` lists the requests whose
    state was dropped with it (they are no longer live).  The cause is chained (``__cause__``)."""

    code = "ERR_STEP_FAILED"


class KernelError(GessoError):
    """The HIP extension is missing, failed to build, or refused a size."""

    code = "ERR_KERNEL"
