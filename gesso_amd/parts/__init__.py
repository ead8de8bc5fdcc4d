from . import attention, block, rmsnorm, rope, shortconv, swiglu  # noqa: F401  (registers the kinds)
from .base import MATRIX, TABLE, VECTOR, PagedKV, Part, SlotState, TensorSpec
from .registry import build, part_class, register, unregister
from .rmsnorm import ResidualStream
from .runtime import DeferredLinear, Runtime, RuntimeOptions
