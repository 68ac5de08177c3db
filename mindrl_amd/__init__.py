"""MI355X-native replay buffers behind the mindspore_rl.core buffer API.

    from mindrl_amd.core import UniformReplayBuffer, PriorityReplayBuffer

Device memory and streams come from PyTorch-ROCm; all buffer work runs in
libmrb.so (hand-written HIP for gfx950) through ctypes.
"""
from . import dtype  # noqa: F401
from .dtype import *  # noqa: F401,F403

__version__ = "0.1.0"
