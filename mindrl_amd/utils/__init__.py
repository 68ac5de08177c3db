"""Helpers built on the buffers, with the interfaces of mindspore_rl.utils."""
from .n_step_buffer import NStepBuffer

__all__ = ["NStepBuffer"]
