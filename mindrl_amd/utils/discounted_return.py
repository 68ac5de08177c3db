"""DiscountedReturn with the interface of mindspore_rl/utils/discounted_return.py:25-92."""
import torch

from .. import _lib
from ..core._rows import device, stream_ptr
from ..dtype import as_torch_dtype


class DiscountedReturn:
    r"""Discounted return :math:`G_t = R_t + \gamma (1 - done_t) G_{t+1}` over sequences that may
    hold several episodes, `done` marking the episode ends and `last_state_value` the value after
    the final step (mindspore_rl/utils/discounted_return.py:25-59).

    Args:
        gamma (float): discount factor in [0, 1].
        need_bprop (bool): the reference then avoids its fused operator so that autograd can
            differentiate the loop (discounted_return.py:81-92); not available here.
        dtype: output type; float32 only.

    Inputs: reward [Timestep, Batch, ...] float32, done [Timestep, Batch] bool,
    last_state_value [Batch, ...] float32 (the Batch axis may be omitted everywhere,
    as in tests/st/test_discounted_return.py:47-53). Returns a tensor shaped like reward.
    """

    def __init__(self, gamma, need_bprop=False, dtype=torch.float32):
        if gamma > 1.0 or gamma < 0.0:
            raise ValueError(f"The discounted factor should be a number in range [0, 1], but got {gamma}.")
        if need_bprop:
            raise NotImplementedError("DiscountedReturn(need_bprop=True): only the forward pass is implemented")
        if as_torch_dtype(dtype) != torch.float32:
            raise TypeError("DiscountedReturn computes in float32")
        self.gamma = float(gamma)
        self._dev = device()

    def construct(self, reward, done, last_state_value):
        r = torch.as_tensor(reward).to(device=self._dev, dtype=torch.float32).contiguous()
        d = torch.as_tensor(done).to(device=self._dev, dtype=torch.bool).contiguous()
        v = torch.as_tensor(last_state_value).to(device=self._dev, dtype=torch.float32).contiguous()
        if r.dim() == 0 or r.shape[0] != d.shape[0]:
            raise ValueError("reward and done must share the leading Timestep axis")
        timesteps = r.shape[0]
        batch = d.numel() // timesteps if timesteps else 0
        if timesteps == 0 or batch == 0 or d.numel() != timesteps * batch or r.numel() % (timesteps * batch):
            raise ValueError("done must be [Timestep, Batch] and reward [Timestep, Batch, ...]")
        inner = r.numel() // (timesteps * batch)
        if v.numel() != batch * inner:
            raise ValueError("last_state_value must be [Batch, ...] matching reward")
        out = torch.empty_like(r)
        _lib.check(_lib.lib().mrb_discounted_return(r.data_ptr(), d.data_ptr(), v.data_ptr(), out.data_ptr(),
                                                    timesteps, batch, inner, self.gamma, stream_ptr()))
        self._keep = (r, d, v)
        return out

    __call__ = construct
