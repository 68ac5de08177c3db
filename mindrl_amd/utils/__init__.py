"""Helpers built on the buffers, with the interfaces of mindspore_rl.utils."""
from .discounted_return import DiscountedReturn
from .n_step_buffer import NStepBuffer

__all__ = ["DiscountedReturn", "NStepBuffer"]
