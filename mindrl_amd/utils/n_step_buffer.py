"""NStepBuffer with the interface of mindspore_rl/utils/n_step_buffer.py:25-112."""
import torch

from .. import _lib
from ..core._rows import stream_ptr
from ..core.uniform_replay_buffer import UniformReplayBuffer


class NStepBuffer:
    """Keeps the most recent transitions and hands out the last `td_step` of them.

    Same constructor and methods as the reference class
    (mindspore_rl/utils/n_step_buffer.py:51-112): two UniformReplayBuffers, `buffer`
    (capacity `buffer_size`) and `td_data` (capacity `td_step`). The reference's
    get_data() reads the last td_step rows one get_item() at a time and inserts each
    into td_data (n_step_buffer.py:85-92); here that loop is one buffer-to-buffer
    launch with the same result.

    Args:
        data_shapes, data_types: shape / element type of each tensor of an element.
        td_step (int): number of most recent elements get_data() returns.
        buffer_size (int): capacity of the buffer. Default: 10000.
    """

    def __init__(self, data_shapes, data_types, td_step, buffer_size=10000):
        self.buffer = UniformReplayBuffer(1, buffer_size, data_shapes, data_types)
        self.td_data = UniformReplayBuffer(1, td_step, data_shapes, data_types)
        self.td = int(td_step)

    def push(self, exp):
        """Appends an element to the buffer (n_step_buffer.py:62-73). Returns True."""
        self.buffer.insert(exp)
        return True

    def get_data(self):
        """(check, td_data.buffer): check is False while the buffer holds no more than
        td_step elements (n_step_buffer.py:75-92); otherwise td_data receives the last
        td_step elements, oldest first."""
        count = int(self.buffer.count)
        if count <= self.td:
            return torch.tensor([False]), self.td_data.buffer
        _lib.check(_lib.lib().mrb_urb_append_from(self.td_data._h, self.buffer._h, count - self.td, self.td,
                                                  stream_ptr()))
        return torch.tensor([True]), self.td_data.buffer

    def clear(self):
        """Resets both buffers' sizes (n_step_buffer.py:94-103). Returns True."""
        self.buffer.reset()
        self.td_data.reset()
        return True

    def size(self):
        """Number of elements in the buffer (n_step_buffer.py:105-112)."""
        return self.buffer.size()

    def destroy(self):
        self.buffer.destroy()
        self.td_data.destroy()
