"""ReservoirReplayBuffer with the interface of
mindspore_rl/core/reservoir_replay_buffer.py:23-100, backed by libmrb.so."""
import ctypes as C
import os

import torch

from .. import _lib
from ._rows import (FieldLayout, create_with_layout, device, get_counters, load_fields, pointers, save_fields,
                    set_counters, storage_views, stream_ptr)


class ReservoirReplayBuffer:
    """Reservoir-sampling buffer (Vitter's Algorithm R) resident in HBM: keeps an
    unbiased sample of everything ever pushed.

    Same constructor and methods as the reference class
    (mindspore_rl/core/reservoir_replay_buffer.py:61-100).

    Args:
        capacity (int): rows kept.
        sample_size (int): rows returned by sample() (may exceed capacity: draws are with replacement).
        shapes, dtypes: shape / element type of each tensor of a transition.
        seed0, seed1 (int): generator seed; seed1 if non-zero, else seed0, else entropy.
    """

    def __init__(self, capacity, sample_size, shapes, dtypes, seed0=0, seed1=0, packed_rows=False):
        self._dev = device()
        self._layout = FieldLayout(shapes, dtypes)
        self._capacity = int(capacity)
        self._sample_size = int(sample_size)
        seed = int(seed1) or int(seed0) or int.from_bytes(os.urandom(8), "little")
        h = C.c_int64(0)
        # packed_rows: as in UniformReplayBuffer (rows of at most 64 bytes, or the given limit, in one array)
        create_with_layout(packed_rows, lambda: _lib.check(_lib.lib().mrb_res_create(
            self._capacity, len(self._layout), self._layout.c_bytes, seed & (2**64 - 1), C.byref(h))))
        self._h = h.value
        self._handle = torch.tensor([self._h], dtype=torch.int64)
        self._keep = None

    def push(self, *transition):
        """Pushes one transition (tensors of shape_i) or a batch ([n, *shape_i])
        (reservoir_replay_buffer.py:68-79). Returns the handle tensor int64[1]."""
        if len(transition) == 1 and isinstance(transition[0], (list, tuple)):
            transition = tuple(transition[0])
        n = self._layout.batch_of(transition)
        src = self._layout.to_device(transition, self._dev)
        _lib.check(_lib.lib().mrb_res_push(self._h, pointers(src), n, stream_ptr()))
        self._keep = src
        return self._handle

    insert = push

    def sample(self, with_indices=False):
        """`sample_size` rows drawn uniformly with replacement (reservoir_replay_buffer.py:81-89)."""
        n = self._sample_size
        dst = self._layout.empty(n, self._dev)
        idx = torch.empty(n, dtype=torch.int64, device=self._dev) if with_indices else None
        _lib.check(_lib.lib().mrb_res_sample(self._h, n, idx.data_ptr() if with_indices else None, pointers(dst),
                                             stream_ptr()))
        return (idx, tuple(dst)) if with_indices else tuple(dst)

    def destroy(self):
        """Releases the native buffer (reservoir_replay_buffer.py:91-100)."""
        if self._h:
            h, self._h = self._h, 0
            _lib.check(_lib.lib().mrb_res_destroy(h))
        return self._handle

    def size(self):
        return self._state()[0]

    def total(self):
        return self._state()[1]

    def _state(self):
        s, t = C.c_int64(0), C.c_int64(0)
        _lib.check(_lib.lib().mrb_res_state(self._h, C.byref(s), C.byref(t)))
        return s.value, t.value

    def state_dict(self):
        """Rows, size, rows ever pushed and the generator's position (this library's own format; the
        reference never persists its buffers)."""
        torch.cuda.current_stream().synchronize()
        size, total, seed, calls = get_counters(_lib.lib().mrb_res_get_counters, self._h)
        return {"kind": "reservoir", "capacity": self._capacity, "size": size, "total": total,
                "seed": seed & ((1 << 64) - 1), "calls": calls, "fields": save_fields(self.storage(), size)}

    def load_state_dict(self, state):
        """Restores a state_dict() taken from a buffer of the same capacity, shapes and types."""
        if state.get("kind") != "reservoir" or state["capacity"] != self._capacity:
            raise ValueError("state does not belong to a ReservoirReplayBuffer of capacity %d" % self._capacity)
        load_fields(self.storage(), state["fields"], self._layout)
        set_counters(_lib.lib().mrb_res_set_counters, self._h,
                     [state["size"], state["total"], state["seed"], state["calls"]])

    def storage(self):
        """Views of the row storage, one [capacity, *shape_i] tensor per field."""
        return storage_views(self._h, self._layout, self._capacity, self, self._dev)

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
        return "ReservoirReplayBuffer<>"
