"""Buffer classes with the constructor and method signatures of mindspore_rl.core."""
from .priority_replay_buffer import PriorityReplayBuffer
from .uniform_replay_buffer import UniformReplayBuffer

__all__ = ["PriorityReplayBuffer", "UniformReplayBuffer"]
