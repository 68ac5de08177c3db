"""DiscountedReturn with the interface of mindspore_rl/utils/discounted_return.py:25-92."""
import torch

from .. import _lib
from ..core._rows import device, stream_ptr
from ..dtype import as_torch_dtype


def _launch(reward, done, last_value, gamma):
    """One kernel launch on contiguous device tensors; returns a tensor shaped like reward."""
    timesteps = reward.shape[0]
    batch = done.numel() // timesteps
    inner = reward.numel() // (timesteps * batch)
    out = torch.empty_like(reward)
    _lib.check(_lib.lib().mrb_discounted_return(reward.data_ptr(), done.data_ptr(), last_value.data_ptr(),
                                                out.data_ptr(), timesteps, batch, inner, gamma, stream_ptr()))
    return out


class _DiscountedReturnFn(torch.autograd.Function):
    """Differentiable wrapper. With c_t = (1 - done_t) * gamma the forward recurrence is
    G_t = R_t + c_t * G_{t+1}; its adjoint runs forwards in time, A_t = dG_t + c_{t-1} * A_{t-1}
    (A_0 = dG_0), which is the same recurrence on time-reversed inputs, so the same kernel
    computes it: dR_t = A_t and d(last_state_value) = c_{T-1} * A_{T-1}."""

    @staticmethod
    def forward(ctx, reward, done, last_value, gamma):
        ctx.save_for_backward(done)
        ctx.gamma = gamma
        return _launch(reward, done, last_value, gamma)

    @staticmethod
    def backward(ctx, grad_out):
        (done,) = ctx.saved_tensors
        gamma = ctx.gamma
        g = grad_out.contiguous().flip(0).contiguous()
        # reversed step s uses c_{T-2-s}; the last reversed step multiplies a zero bootstrap
        shifted = torch.cat([done[:-1].flip(0), torch.zeros_like(done[:1])], 0).contiguous()
        zeros = torch.zeros(g.shape[1:], dtype=g.dtype, device=g.device)
        adj = _launch(g, shifted, zeros, gamma)  # adj[s] = A_{T-1-s}
        grad_reward = adj.flip(0)
        keep = (1.0 - done[-1].to(g.dtype)) * gamma
        grad_last = keep.reshape(keep.shape + (1,) * (adj.dim() - 1 - keep.dim())) * adj[0]
        return grad_reward, None, grad_last, None


class DiscountedReturn:
    r"""Discounted return :math:`G_t = R_t + \gamma (1 - done_t) G_{t+1}` over sequences that may
    hold several episodes, `done` marking the episode ends and `last_state_value` the value after
    the final step (mindspore_rl/utils/discounted_return.py:25-59).

    Args:
        gamma (float): discount factor in [0, 1].
        need_bprop (bool): the reference then avoids its fused operator so that autograd can
            differentiate the loop (discounted_return.py:81-92); here the returned tensor is then
            differentiable with respect to reward and last_state_value (the backward pass is the
            same kernel on time-reversed inputs).
        dtype: output type; float32 only.

    Inputs: reward [Timestep, Batch, ...] float32, done [Timestep, Batch] bool,
    last_state_value [Batch, ...] float32 (the Batch axis may be omitted everywhere,
    as in tests/st/test_discounted_return.py:47-53). Returns a tensor shaped like reward.
    """

    def __init__(self, gamma, need_bprop=False, dtype=torch.float32):
        if gamma > 1.0 or gamma < 0.0:
            raise ValueError(f"The discounted factor should be a number in range [0, 1], but got {gamma}.")
        if as_torch_dtype(dtype) != torch.float32:
            raise TypeError("DiscountedReturn computes in float32")
        self.gamma = float(gamma)
        self.need_bprop = bool(need_bprop)
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
        if self.need_bprop and (r.requires_grad or v.requires_grad):
            return _DiscountedReturnFn.apply(r, d.reshape(timesteps, batch), v, self.gamma)
        out = _launch(r.detach(), d, v.detach(), self.gamma)
        self._keep = (r, d, v)
        return out

    __call__ = construct
