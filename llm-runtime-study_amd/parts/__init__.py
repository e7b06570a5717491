"""Parts a layer is composed of; importing this package registers the built-in kinds."""

from .base import (BothNeeds, LazyTensors, PagedKVNeed, Part, PartSpec, Renamed, StateNeed, TensorSpec, Under, create, register, under)
from . import attention, block, delta, latent, mlp, moe, norm, rope, sidebyside, ssm, transform  # noqa: F401  (registration)

__all__ = ["BothNeeds", "PagedKVNeed", "Part", "PartSpec", "StateNeed", "TensorSpec", "create", "register"]
