"""gesso_amd: a small, whole inference engine for one MI355X (gfx950).

From a request's tokens to its next token: typed configuration and architecture registry,
weights by tensor name, layers composed of parts, a paged cache with per-request state slots,
one step function over mixed batches, a scheduler with sampling, and hand-written HIP kernels.
"""
from . import parts as _parts  # noqa: F401  registers part kinds
from .models import lfm2 as _lfm2  # noqa: F401  registers the architecture
from .errors import (ConfigError, GessoError, InvalidPlan, KernelError, NumericalInstability, OutOfPages,
                     OutOfSlots, ResourceLimit, StepFailed, WeightError)

from .engine.batch import StepEntry
from .engine.engine import Engine
from .engine.scheduler import Request, Scheduler
from .engine.session import BatchRequest, BatchResult, Session, cancel, generate, run_batch
from .parts.runtime import RuntimeOptions
from .sampling.sampler import Sampler

__version__ = "0.1.0"
