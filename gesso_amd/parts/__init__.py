from . import attention, block, gated_mlp, gated_state, latent_attention, linear_attention, rmsnorm, rope, routed_moe, shortconv, state_space, swiglu, table_moe  # noqa: F401  (registers the kinds)
from .base import INDEX, MATRIX, TABLE, VECTOR, PagedKV, Part, SlotState, TensorSpec
from .registry import build, part_class, register, unregister
from .rmsnorm import ResidualStream
from .runtime import DeferredLinear, Runtime, RuntimeOptions
