"""UniformReplayBuffer with the interface of
mindspore_rl/core/uniform_replay_buffer.py:50-172, backed by libmrb.so."""
import ctypes as C

import numpy as np
import torch

from .. import _lib
from ._rows import (FieldLayout, create_with_layout, device, get_counters, load_fields, pointers, save_fields,
                    set_counters, storage_views, stream_ptr)


class _BufferAppend:
    """Stands in for P.BufferAppend (uniform_replay_buffer.py:82): called as
    buffer_append(buffer, exp, count, head); buffer, count and head are the owner's own state."""

    def __init__(self, owner):
        self._owner_ref = owner

    def __call__(self, buffer, exp, count=None, head=None):
        self._owner_ref.insert(exp)
        return True


class _BufferSample:
    """Stands in for P.BufferSample (uniform_replay_buffer.py:87-89): batch_size attribute,
    called as buffer_sample(buffer, count, head)."""

    def __init__(self, owner):
        self._owner_ref = owner
        self.batch_size = owner._sample_size

    def __call__(self, buffer=None, count=None, head=None):
        return self._owner_ref.sample()


class _BufferGet:
    """Stands in for P.BufferGetItem (uniform_replay_buffer.py:83): buffer_get(buffer, count, head, index)."""

    def __init__(self, owner):
        self._owner_ref = owner

    def __call__(self, buffer, count, head, index):
        return self._owner_ref.get_item(index)


class UniformReplayBuffer:
    """FIFO replay buffer resident in HBM.

    Same constructor and methods as the reference class
    (mindspore_rl/core/uniform_replay_buffer.py:75-172): each element is a list
    of tensors described by `shapes`/`types`; storage is one
    [capacity, *shape_i] tensor per field (`.buffer`), with int32 `count` and
    `head`.

    Args:
        sample_size (int): rows returned by sample().
        capacity (int): number of rows kept; the oldest row is overwritten when full.
        shapes (list[tuple]): shape of each tensor of an element.
        types (list): element type of each tensor (torch / numpy dtype or name).
        packed_rows (bool or int): False (default): every field is a [capacity, *shape_i] array of its own, the
            reference's layout. True (or a byte limit): rows of at most 64 (that many) bytes are kept packed in
            one array; `.buffer` then holds strided views of the same shapes. Results never differ.
    """

    def __init__(self, sample_size, capacity, shapes, types, seed=0, packed_rows=False):
        self._dev = device()
        self._layout = FieldLayout(shapes, types)
        self._capacity = int(capacity)
        self._sample_size = int(sample_size)
        h = C.c_int64(0)
        create_with_layout(packed_rows, lambda: _lib.check(_lib.lib().mrb_urb_create(
            self._capacity, len(self._layout), self._layout.c_bytes, C.byref(h))))
        self._h = h.value
        _lib.check(_lib.lib().mrb_urb_seed(self._h, int(seed) & (2**64 - 1)))
        self.buffer = storage_views(self._h, self._layout, self._capacity, self, self._dev)
        # Attributes that subclasses and callers of the reference class reach into: the append and sample
        # primitives (mindspore_rl/algorithm/mappo/mappo_replaybuffer.py:43 calls
        # `self.buffer_append(self.buffer, exp, self.count, self.head)`;
        # mindspore_rl/algorithm/gail/gail.py:163-164 reads `buffer_sample.batch_size`).
        self.buffer_append = _BufferAppend(self)
        self.buffer_sample = _BufferSample(self)
        self.buffer_get = _BufferGet(self)

    # -- reference methods ---------------------------------------------------
    def insert(self, exp):
        """Appends one element (tensors of shape_i) or a batch ([n, *shape_i]); FIFO
        replacement when full. Returns the whole buffer, as the reference does
        (uniform_replay_buffer.py:101-115)."""
        n = self._layout.batch_of(exp)
        src = self._layout.to_device(exp, self._dev)
        _lib.check(_lib.lib().mrb_urb_append(self._h, pointers(src), n, stream_ptr()))
        self._keep = src  # alive until the next call on this stream-ordered buffer
        return self.buffer

    def get_item(self, index):
        """Element at logical position `index`, 0 = oldest (uniform_replay_buffer.py:117-128)."""
        out = self._layout.empty(None, self._dev)
        _lib.check(_lib.lib().mrb_urb_get_item(self._h, int(index), pointers(out), stream_ptr()))
        return tuple(out)

    def sample(self, indices=None, out=None):
        """`sample_size` rows drawn uniformly with replacement (uniform_replay_buffer.py:130-139).

        indices: optional int64 tensor of physical slots in [0, count) to use
        instead of the buffer's generator (its length sets the batch)."""
        if indices is None:
            n = self._sample_size
            dst = self._layout.check_out(out, n, self._dev) if out is not None else self._layout.empty(n, self._dev)
            _lib.check(_lib.lib().mrb_urb_sample(self._h, n, None, pointers(dst), stream_ptr()))
            return tuple(dst)
        idx = torch.as_tensor(indices).to(device=self._dev, dtype=torch.int64).contiguous().reshape(-1)
        n = idx.numel()
        dst = self._layout.check_out(out, n, self._dev) if out is not None else self._layout.empty(n, self._dev)
        _lib.check(_lib.lib().mrb_urb_gather(self._h, idx.data_ptr(), n, pointers(dst), stream_ptr()))
        self._keep = idx
        return tuple(dst)

    def sample_with_indices(self):
        """As sample(), also returning the drawn slots (int64[sample_size])."""
        n = self._sample_size
        dst = self._layout.empty(n, self._dev)
        idx = torch.empty(n, dtype=torch.int64, device=self._dev)
        _lib.check(_lib.lib().mrb_urb_sample(self._h, n, idx.data_ptr(), pointers(dst), stream_ptr()))
        return idx, tuple(dst)

    def reset(self):
        """count = 0; head is left as it is (uniform_replay_buffer.py:141-150)."""
        _lib.check(_lib.lib().mrb_urb_reset(self._h))
        return True

    def size(self):
        """Number of stored rows, as a numpy int32 scalar array (uniform_replay_buffer.py:152-160)."""
        return np.array(self._state()[0], dtype=np.int32)

    def full(self):
        """bool tensor of shape (1,): count >= capacity (uniform_replay_buffer.py:162-172)."""
        return torch.tensor([self._state()[0] >= self._capacity])

    # -- attributes read by the reference's callers ----------------------------
    @property
    def count(self):
        return torch.tensor(self._state()[0], dtype=torch.int32)

    @property
    def head(self):
        return torch.tensor(self._state()[1], dtype=torch.int32)

    @property
    def capacity(self):
        return self._capacity

    @property
    def sample_size(self):
        return self._sample_size

    # -- extras ----------------------------------------------------------------
    def check(self):
        """Synchronises and raises if a kernel saw an out-of-range index."""
        flags = C.c_uint32(0)
        _lib.check(_lib.lib().mrb_urb_check(self._h, C.byref(flags), stream_ptr()))
        if flags.value:
            raise IndexError("UniformReplayBuffer: index outside [0, count) (flags=%d)" % flags.value)

    def state_dict(self):
        """Everything needed to rebuild this buffer: rows, count, head and the generator's position.
        (The reference never persists its buffers; this is this library's own format.)"""
        torch.cuda.current_stream().synchronize()
        count, head, seed, calls = get_counters(_lib.lib().mrb_urb_get_counters, self._h)
        nrows = self._capacity if (head != 0 or count == self._capacity) else count
        return {"kind": "uniform", "capacity": self._capacity, "count": count, "head": head,
                "seed": seed & ((1 << 64) - 1), "calls": calls, "fields": save_fields(self.buffer, nrows)}

    def load_state_dict(self, state):
        """Restores a state_dict() taken from a buffer of the same capacity, shapes and types."""
        if state.get("kind") != "uniform" or state["capacity"] != self._capacity:
            raise ValueError("state does not belong to a UniformReplayBuffer of capacity %d" % self._capacity)
        load_fields(self.buffer, state["fields"], self._layout)
        set_counters(_lib.lib().mrb_urb_set_counters, self._h,
                     [state["count"], state["head"], state["seed"], state["calls"]])

    def _state(self):
        c, h = C.c_int32(0), C.c_int32(0)
        _lib.check(_lib.lib().mrb_urb_state(self._h, C.byref(c), C.byref(h)))
        return c.value, h.value

    def destroy(self):
        if getattr(self, "_h", 0):
            self.buffer = ()
            h, self._h = self._h, 0
            _lib.check(_lib.lib().mrb_urb_destroy(h))

    def set_option(self, name, value):
        """Sets a launch option of this buffer ("row_split"; prioritized buffers also "sample_path",
        "lds_levels", "fused_rebuild", "device_counters"). Options change how kernels are launched, never a
        result."""
        _lib.set_option(self._h, name, value)

    def __del__(self):
        # the native buffer (rows, trees) is released with the Python object if destroy() was not called
        try:
            if getattr(self, "_h", 0):
                self.destroy()
        except Exception:  # interpreter shutdown: the library or torch may already be gone
            pass

    def __repr__(self):
        return "UniformReplayBuffer<>"
