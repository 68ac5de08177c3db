"""Buffer classes with the constructor and method signatures of mindspore_rl.core."""
from .factory import ReplayBufferSet, create_replay_buffer
from .priority_replay_buffer import PriorityReplayBuffer
from .reservoir_replay_buffer import ReservoirReplayBuffer
from .uniform_replay_buffer import UniformReplayBuffer

__all__ = ["PriorityReplayBuffer", "ReplayBufferSet", "ReservoirReplayBuffer", "UniformReplayBuffer",
           "create_replay_buffer"]
