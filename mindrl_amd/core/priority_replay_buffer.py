"""PriorityReplayBuffer with the interface of
mindspore_rl/core/priority_replay_buffer.py:30-138, backed by libmrb.so."""
import ctypes as C
import os

import numpy as np
import torch

from .. import _lib
from ._rows import (FieldLayout, create_with_layout, device, flat_on_device, get_counters, load_fields, pointers,
                    save_fields, set_counters, storage_views, stream_ptr)


class PriorityReplayBuffer:
    """Proportional prioritized replay (Schaul et al.) resident in HBM: FIFO rows
    plus a sum tree and a min tree over next_pow2(capacity) leaves.

    Same constructor and methods as the reference class
    (mindspore_rl/core/priority_replay_buffer.py:60-138).

    Args:
        alpha (float): priority exponent; 0 = uniform, 1 = fully prioritized.
        capacity (int): number of rows kept.
        sample_size (int): rows returned by sample().
        shapes, types: shape / element type of each tensor of an element.
        seed0, seed1 (int): generator seed; seed1 if non-zero, else seed0, else entropy.
        output_ring (int): 0 (the default): sample() returns fresh tensors on every call, as the
            reference does. N > 0 (opt-in, for loops that consume a batch before drawing the N-th next
            one): sample() hands out its result tensors from N preallocated sets in turn, so a call
            allocates nothing; a returned batch is then overwritten by the N-th sample() call after
            it - clone() what must live longer.
        packed_rows (bool or int): False (default): every field is a [capacity, *shape_i] array of its own, the
            reference's layout. True (or a byte limit): rows of at most 64 (that many) bytes are kept packed in
            one array, so that a sampled row's fields share cache lines; storage() then returns strided views.
            Results never differ.
    """

    def __init__(self, alpha, capacity, sample_size, shapes, types, seed0=0, seed1=0, output_ring=0, packed_rows=False):
        self._dev = device()
        self._layout = FieldLayout(shapes, types)
        self._capacity = int(capacity)
        self._sample_size = int(sample_size)
        self._alpha = float(alpha)
        seed = int(seed1) or int(seed0) or int.from_bytes(os.urandom(8), "little")
        h = C.c_int64(0)
        create_with_layout(packed_rows, lambda: _lib.check(_lib.lib().mrb_per_create(
            self._capacity, self._alpha, len(self._layout), self._layout.c_bytes, seed & (2**64 - 1), C.byref(h))))
        self._h = h.value
        self._handle = torch.tensor([self._h], dtype=torch.int64)
        self._keep = None
        self._ring_size = int(output_ring)
        self._ring, self._ring_at = None, 0  # output sets, built by the first sample()

    def _next_outputs(self):
        """The next preallocated (indices, weights, fields, field pointer array) set."""
        if self._ring is None:
            n = self._sample_size
            self._ring = []
            for _ in range(self._ring_size):
                fields = self._layout.empty(n, self._dev)
                self._ring.append((torch.empty(n, dtype=torch.int64, device=self._dev),
                                   torch.empty(n, dtype=torch.float32, device=self._dev), fields, pointers(fields)))
        out = self._ring[self._ring_at]
        self._ring_at = (self._ring_at + 1) % self._ring_size
        return out

    # -- reference methods ---------------------------------------------------
    def insert(self, *transition, priorities=None):
        """Pushes one transition (tensors of shape_i) or a batch ([n, *shape_i]); the
        oldest row is replaced when full; new rows take the running max priority
        (priority_replay_buffer.py:78-90). `priorities` (f32[n]), if given, are
        applied to the new rows as update_priorities would. Returns the handle
        tensor int64[1]."""
        if len(transition) == 1 and isinstance(transition[0], (list, tuple)):
            transition = tuple(transition[0])
        n = self._layout.rows_if_ready(transition, self._dev)
        if n is not None:
            src = transition
        else:
            n = self._layout.batch_of(transition)
            src = self._layout.to_device(transition, self._dev)
        pr = None
        if priorities is not None:
            pr = flat_on_device(priorities, torch.float32, self._dev)
            if pr.numel() != n:
                raise ValueError("priorities must hold one value per pushed row")
        _lib.check(_lib.lib().mrb_per_push(self._h, pointers(src), n, pr.data_ptr() if pr is not None else None,
                                           stream_ptr()))
        self._keep = (src, pr)
        return self._handle

    # the reference's own test calls the method by this name (tests/st/test_priority_replay_buffer.py:46)
    push = insert

    def sample(self, beta, uniforms=None, out=None):
        """Stratified proportional sample of `sample_size` rows
        (priority_replay_buffer.py:92-106).

        Returns (indices int64[B], weights f32[B], *transitions [B, *shape_i]).
        `uniforms` (f32[B] in [0,1)) replaces the buffer's generator, stratum k
        using uniforms[k]. `out` = (indices, weights, [fields]) writes into the caller's tensors.
        Without `out` the result is a set of fresh tensors, unless the buffer was built with
        `output_ring` > 0: then it comes from that ring of preallocated output sets and stays valid
        until `output_ring` further sample() calls have been made."""
        n = self._sample_size
        u = None
        if uniforms is not None:
            u = flat_on_device(uniforms, torch.float32, self._dev)
            if u.numel() != n:
                raise ValueError("uniforms must hold sample_size = %d values" % n)
        if out is not None:
            idx, w, fields = out
            fields = self._layout.check_out(fields, n, self._dev)
            fptr = pointers(fields)
        elif self._ring_size > 0:
            idx, w, fields, fptr = self._next_outputs()
        else:
            idx = torch.empty(n, dtype=torch.int64, device=self._dev)
            w = torch.empty(n, dtype=torch.float32, device=self._dev)
            fields = self._layout.empty(n, self._dev)
            fptr = pointers(fields)
        _lib.check(_lib.lib().mrb_per_sample(self._h, n, float(beta), u.data_ptr() if u is not None else None,
                                             idx.data_ptr(), w.data_ptr(), fptr, stream_ptr()))
        self._keep = u
        return (idx, w) + tuple(fields)

    def sample_with_next(self, beta, slot_field, row_field, uniforms=None):
        """sample(beta) plus, in the same launch, field `row_field` of the row whose slot number each sampled
        row holds in its field `slot_field` (an int64[1] field): for transitions that store the next
        observation as a slot number instead of a copy. Returns sample()'s tuple with one more tensor
        [B, *shape_row_field] at the end - what `gather(transitions[slot_field])[row_field]` would give, without
        the second launch and the second tree descent. Fresh output tensors on every call."""
        n = self._sample_size
        slot_field, row_field = int(slot_field), int(row_field)
        if not 0 <= slot_field < len(self._layout) or not 0 <= row_field < len(self._layout):
            raise ValueError("slot_field and row_field must name fields of the transition")
        u = None
        if uniforms is not None:
            u = flat_on_device(uniforms, torch.float32, self._dev)
            if u.numel() != n:
                raise ValueError("uniforms must hold sample_size = %d values" % n)
        idx = torch.empty(n, dtype=torch.int64, device=self._dev)
        w = torch.empty(n, dtype=torch.float32, device=self._dev)
        fields = self._layout.empty(n, self._dev)
        nxt = torch.empty((n,) + tuple(self._layout.shapes[row_field]), dtype=self._layout.dtypes[row_field],
                          device=self._dev)
        _lib.check(_lib.lib().mrb_per_sample_next(self._h, n, float(beta), u.data_ptr() if u is not None else None,
                                                  slot_field, row_field, idx.data_ptr(), w.data_ptr(),
                                                  pointers(fields), nxt.data_ptr(), stream_ptr()))
        self._keep = u
        return (idx, w) + tuple(fields) + (nxt,)

    def sample_many(self, nbatch, beta, uniforms=None):
        """`nbatch` batches in one launch: what `nbatch` successive sample(beta) calls would return on an
        unchanged buffer, stacked: (indices int64[nbatch, B], weights f32[nbatch, B], *transitions
        [nbatch, B, *shape_i]). For learners that draw several batches between priority updates; one launch
        amortises the launch and the tree descent. `uniforms`: f32[nbatch, B] or None (generator)."""
        nbatch, n = int(nbatch), self._sample_size
        u = None
        if uniforms is not None:
            u = flat_on_device(uniforms, torch.float32, self._dev)
            if u.numel() != nbatch * n:
                raise ValueError("uniforms must hold nbatch * sample_size = %d values" % (nbatch * n))
        idx = torch.empty((nbatch, n), dtype=torch.int64, device=self._dev)
        w = torch.empty((nbatch, n), dtype=torch.float32, device=self._dev)
        fields = [torch.empty((nbatch, n) + s, dtype=d, device=self._dev)
                  for s, d in zip(self._layout.shapes, self._layout.dtypes)]
        _lib.check(_lib.lib().mrb_per_sample_many(self._h, nbatch, n, float(beta), u.data_ptr() if u is not None else None,
                                                  idx.data_ptr(), w.data_ptr(), pointers(fields), stream_ptr()))
        self._keep = u
        return (idx, w) + tuple(fields)

    def update_priorities(self, indices, priorities):
        """leaf[indices[j]] = priorities[j] ** alpha in order, last write wins
        (priority_replay_buffer.py:108-120). Returns the handle tensor."""
        idx = flat_on_device(indices, torch.int64, self._dev)
        pr = flat_on_device(priorities, torch.float32, self._dev)
        if idx.numel() != pr.numel():
            raise ValueError("indices and priorities differ in length")
        _lib.check(_lib.lib().mrb_per_update(self._h, idx.data_ptr(), pr.data_ptr(), idx.numel(), stream_ptr()))
        self._keep = (idx, pr)
        return self._handle

    def update_priorities_and_insert(self, indices, priorities, *transition, insert_priorities=None):
        """update_priorities(indices, priorities) followed by insert(*transition, priorities=insert_priorities),
        as ONE library call (mrb_per_update_push): the result is the two calls', bit for bit, with fewer kernel
        launches - a learner's step is bound by them (the reference's loop issues the two back to back,
        mindspore_rl/algorithm/dqn/dqn_trainer.py:76-87). Returns the handle tensor."""
        idx = flat_on_device(indices, torch.int64, self._dev)
        pr = flat_on_device(priorities, torch.float32, self._dev)
        if idx.numel() != pr.numel():
            raise ValueError("indices and priorities differ in length")
        if len(transition) == 1 and isinstance(transition[0], (list, tuple)):
            transition = tuple(transition[0])
        n = self._layout.rows_if_ready(transition, self._dev)
        if n is not None:
            src = transition
        else:
            n = self._layout.batch_of(transition)
            src = self._layout.to_device(transition, self._dev)
        ipr = None
        if insert_priorities is not None:
            ipr = flat_on_device(insert_priorities, torch.float32, self._dev)
            if ipr.numel() != n:
                raise ValueError("insert_priorities must hold one value per pushed row")
        _lib.check(_lib.lib().mrb_per_update_push(self._h, idx.data_ptr(), pr.data_ptr(), idx.numel(), pointers(src), n,
                                                  ipr.data_ptr() if ipr is not None else None, stream_ptr()))
        self._keep = (idx, pr, src, ipr)
        return self._handle

    def update_priorities_insert_and_sample(self, indices, priorities, *transition, beta, insert_priorities=None,
                                            uniforms=None, out=None):
        """update_priorities(indices, priorities), insert(*transition, priorities=insert_priorities) and
        sample(beta, uniforms, out) as ONE library call (mrb_per_update_push_sample): a learner's whole step on the
        buffer (mindspore_rl/algorithm/dqn/dqn_trainer.py:76-87 and the sample of the next iteration). The results
        are the three calls', bit for bit; on a small buffer (capacity up to 16,384, up to 384 entries, one
        transition, up to 512 sampled rows) they take one kernel launch instead of two or three. Returns what
        sample() returns."""
        idx = flat_on_device(indices, torch.int64, self._dev)
        pr = flat_on_device(priorities, torch.float32, self._dev)
        if idx.numel() != pr.numel():
            raise ValueError("indices and priorities differ in length")
        if len(transition) == 1 and isinstance(transition[0], (list, tuple)):
            transition = tuple(transition[0])
        n = self._layout.rows_if_ready(transition, self._dev)
        if n is not None:
            src = transition
        else:
            n = self._layout.batch_of(transition)
            src = self._layout.to_device(transition, self._dev)
        ipr = None
        if insert_priorities is not None:
            ipr = flat_on_device(insert_priorities, torch.float32, self._dev)
            if ipr.numel() != n:
                raise ValueError("insert_priorities must hold one value per pushed row")
        b = self._sample_size
        u = None
        if uniforms is not None:
            u = flat_on_device(uniforms, torch.float32, self._dev)
            if u.numel() != b:
                raise ValueError("uniforms must hold sample_size = %d values" % b)
        if out is not None:
            oidx, w, fields = out
            fields = self._layout.check_out(fields, b, self._dev)
            fptr = pointers(fields)
        elif self._ring_size > 0:
            oidx, w, fields, fptr = self._next_outputs()
        else:
            oidx = torch.empty(b, dtype=torch.int64, device=self._dev)
            w = torch.empty(b, dtype=torch.float32, device=self._dev)
            fields = self._layout.empty(b, self._dev)
            fptr = pointers(fields)
        _lib.check(_lib.lib().mrb_per_update_push_sample(
            self._h, idx.data_ptr(), pr.data_ptr(), idx.numel(), pointers(src), n,
            ipr.data_ptr() if ipr is not None else None, b, float(beta), u.data_ptr() if u is not None else None,
            oidx.data_ptr(), w.data_ptr(), fptr, stream_ptr()))
        self._keep = (idx, pr, src, ipr, u)
        return (oidx, w) + tuple(fields)

    def gather(self, indices, out=None):
        """Rows at the given slots (int64, each in [0, size)): one [n, *shape_i] tensor per field.
        For transitions that store the slot of their successor instead of a copy of it, e.g.
        `next_rows = buf.gather(sampled_next_idx)`."""
        idx = flat_on_device(indices, torch.int64, self._dev)
        n = idx.numel()
        dst = self._layout.check_out(out, n, self._dev) if out is not None else self._layout.empty(n, self._dev)
        _lib.check(_lib.lib().mrb_per_gather(self._h, idx.data_ptr(), n, pointers(dst), stream_ptr()))
        self._keep = idx
        return tuple(dst)

    def full(self):
        """Always False, as in the reference (priority_replay_buffer.py:122-124)."""
        return torch.tensor(False)

    def reset(self):
        """Not supported, as in the reference (priority_replay_buffer.py:126-128)."""
        raise ValueError("reset() is not supported by PriorityReplayBuffer.")

    def destroy(self):
        """Releases the native buffer (priority_replay_buffer.py:130-138)."""
        if self._h:
            h, self._h = self._h, 0
            self._ring = None
            _lib.check(_lib.lib().mrb_per_destroy(h))
        return self._handle

    # -- extras ----------------------------------------------------------------
    def size(self):
        return self._state()[0]

    @property
    def max_priority(self):
        return self._state(True)[2]

    @property
    def capacity(self):
        return self._capacity

    @property
    def sample_size(self):
        return self._sample_size

    def _state(self, with_max=False):
        s, hd, mp = C.c_int64(0), C.c_int64(0), C.c_float(0)
        _lib.check(_lib.lib().mrb_per_state(self._h, C.byref(s), C.byref(hd), C.byref(mp) if with_max else None,
                                            stream_ptr()))
        return s.value, hd.value, mp.value

    def export_tree(self):
        """(sum_heap, min_heap) as numpy float32[2 * leaves], root at 1, leaf i at leaves + i."""
        leaves = C.c_int64(0)
        _lib.check(_lib.lib().mrb_per_export_tree(self._h, None, None, C.byref(leaves), stream_ptr()))
        s = np.empty(2 * leaves.value, np.float32)
        m = np.empty(2 * leaves.value, np.float32)
        _lib.check(_lib.lib().mrb_per_export_tree(self._h, s.ctypes.data, m.ctypes.data, None, stream_ptr()))
        return s, m

    def storage(self):
        """Views of the row storage, one [capacity, *shape_i] tensor per field."""
        return storage_views(self._h, self._layout, self._capacity, self, self._dev)

    def state_dict(self):
        """Everything needed to rebuild this buffer: rows, the leaves of the sum tree (internal nodes
        are rebuilt on load, which reproduces them bit for bit), size, pushes, running max priority and
        the generator's position. (The reference never persists its buffers; this is this library's
        own format.)"""
        size, pushes, seed, calls = get_counters(_lib.lib().mrb_per_get_counters, self._h)
        sum_heap, _ = self.export_tree()
        leaves = sum_heap.size // 2
        return {"kind": "priority", "capacity": self._capacity, "alpha": self._alpha, "size": size, "pushes": pushes,
                "seed": seed & ((1 << 64) - 1), "calls": calls, "max_priority": float(self.max_priority),
                "leaves": torch.from_numpy(sum_heap[leaves:leaves + size].copy()),
                "fields": save_fields(self.storage(), size)}

    def load_state_dict(self, state):
        """Restores a state_dict() taken from a buffer of the same capacity, alpha, shapes and types.
        Nothing of this buffer changes unless the whole state fits."""
        if state.get("kind") != "priority" or state["capacity"] != self._capacity:
            raise ValueError("state does not belong to a PriorityReplayBuffer of capacity %d" % self._capacity)
        if np.float32(state["alpha"]) != np.float32(self._alpha):
            # the saved leaves are priorities ** alpha: they mean something else under another exponent
            raise ValueError("state was saved with alpha %r, this buffer has alpha %r" % (state["alpha"], self._alpha))
        leaves = torch.as_tensor(state["leaves"]).to(device=self._dev, dtype=torch.float32).contiguous()
        size, pushes = int(state["size"]), int(state["pushes"])
        if leaves.numel() != size or size != min(pushes, self._capacity) or pushes < 0:
            raise ValueError("state holds %d leaves for size %d after %d pushes" % (leaves.numel(), size, pushes))
        load_fields(self.storage(), state["fields"], self._layout)
        # the tree first, the counters last: a failure on the way leaves size and pushes as they were
        _lib.check(_lib.lib().mrb_per_load_leaves(self._h, leaves.data_ptr() if leaves.numel() else None,
                                                  leaves.numel(), float(state["max_priority"]), stream_ptr()))
        set_counters(_lib.lib().mrb_per_set_counters, self._h, [size, pushes, state["seed"], state["calls"]])
        torch.cuda.current_stream().synchronize()

    def check(self):
        """Synchronises; raises if a kernel recorded a data error since the last check."""
        flags = C.c_uint32(0)
        _lib.check(_lib.lib().mrb_per_check(self._h, C.byref(flags), stream_ptr()))
        f = flags.value
        if f & _lib.DERR_INDEX:
            raise IndexError("update_priorities: index outside [0, capacity)")
        if f & _lib.DERR_PRIORITY:
            raise ValueError("update_priorities: negative or non-finite priority")
        if f & _lib.DERR_TOTAL:
            raise ValueError("sample: total priority is not positive and finite")
        return f

    def set_option(self, name, value):
        """Sets a launch option of this buffer ("row_split"; prioritized buffers also "sample_path", "row_wave",
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
        return "PriorityReplayBuffer<>"
