"""Host-side plumbing shared by both buffer classes: field layout, tensor
marshalling to device pointers, and views over library-owned storage."""
import ctypes as C
import threading

import numpy as np
import torch

from .. import _lib
from ..dtype import as_torch_dtype


def device():
    if not torch.cuda.is_available():
        raise RuntimeError("mindrl_amd buffers need a HIP device (torch.cuda.is_available() is False); "
                           "there is no CPU fallback")
    return torch.device("cuda", torch.cuda.current_device())


# torch's own accessors of the current device and its current stream, without the Stream object that
# torch.cuda.current_stream() builds on every call (2.9 us a call against 0.1 us; the calls here are 4-9 us).
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def stream_ptr():
    """The current stream of the current device as the integer value of its hipStream_t (0 = the null stream)."""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


class _DeviceView:
    """Exposes library-owned device memory to torch through __cuda_array_interface__."""

    def __init__(self, ptr, shape, typestr, owner, strides=None):
        self.owner = owner  # keeps the buffer object (and so the allocation) alive
        self.__cuda_array_interface__ = {
            "shape": tuple(shape), "typestr": typestr, "data": (int(ptr), False), "version": 2, "strides": strides,
        }


_TYPESTR = {
    torch.float16: "<f2", torch.float32: "<f4", torch.float64: "<f8", torch.int8: "|i1", torch.int16: "<i2",
    torch.int32: "<i4", torch.int64: "<i8", torch.uint8: "|u1", torch.bool: "|b1",
}


def view_of(ptr, shape, dtype, owner, dev, row_stride=None):
    """torch tensor aliasing `ptr` (no copy). `row_stride`: bytes from one row (index of the first dimension) to
    the next, when that is not the row's own size (packed rows: the tensor is then a strided view)."""
    item = torch.empty((), dtype=dtype).element_size()
    strides = None
    if row_stride is not None and row_stride != item * int(np.prod(shape[1:], dtype=np.int64)):
        inner, acc = [], item
        for n in reversed(shape[1:]):
            inner.append(acc)
            acc *= n
        strides = (int(row_stride),) + tuple(reversed(inner))
    if dtype == torch.bfloat16:
        t = torch.as_tensor(_DeviceView(ptr, shape, "<i2", owner, strides), device=dev)
        return t.view(torch.bfloat16)
    return torch.as_tensor(_DeviceView(ptr, shape, _TYPESTR[dtype], owner, strides), device=dev)


_create_lock = threading.Lock()


def create_with_layout(packed_rows, create):
    """Runs `create()` (a libmrb *_create call) with the library-wide option "packed_rows" set for its duration:
    False / 0 = every field an array of its own (the reference's layout), True = rows of at most 64 bytes are
    kept packed, an int = rows of at most that many bytes."""
    limit = 64 if packed_rows is True else int(packed_rows or 0)
    with _create_lock:
        _lib.set_option(0, "packed_rows", limit)
        try:
            return create()
        finally:
            _lib.set_option(0, "packed_rows", 0)


def storage_views(handle, layout, capacity, owner, dev):
    """One [capacity, *shape_i] tensor per field over the buffer's own memory (strided when rows are packed)."""
    views = []
    for i, (s, d) in enumerate(zip(layout.shapes, layout.dtypes)):
        p, stride = C.c_void_p(), C.c_int64(0)
        _lib.check(_lib.lib().mrb_field_layout(handle, i, C.byref(p), C.byref(stride)))
        views.append(view_of(p.value, (capacity,) + s, d, owner, dev, stride.value))
    return tuple(views)


def as_tensor(x):
    """A torch tensor over `x` without a copy where that is possible: torch tensors as they are, any other
    object that speaks DLPack (`__dlpack__` / `__dlpack_device__`: arrays of other frameworks, device-resident
    ones included) through torch.from_dlpack - its memory is shared, nothing passes through the host -, and
    everything else (numpy arrays, lists, scalars) through numpy."""
    if isinstance(x, torch.Tensor):
        return x
    if hasattr(x, "__dlpack__") and hasattr(x, "__dlpack_device__") and not isinstance(x, np.ndarray):
        return torch.from_dlpack(x)
    return torch.as_tensor(np.asarray(x))


class FieldLayout:
    """Shapes/dtypes of one buffer element, as given to the reference constructors
    (`shapes`, `types`: mindspore_rl/core/uniform_replay_buffer.py:75)."""

    def __init__(self, shapes, types):
        if len(shapes) != len(types):
            raise ValueError("shapes and types differ in length")
        if not 0 < len(shapes) <= _lib.MAX_FIELDS:
            raise ValueError("a buffer element has between 1 and %d tensors" % _lib.MAX_FIELDS)
        self.shapes = []
        for s in shapes:
            if isinstance(s, (int, np.integer)):
                s = (int(s),)
            self.shapes.append(tuple(int(v) for v in s))
        self.dtypes = [as_torch_dtype(t) for t in types]
        self.numel = [int(np.prod(s, dtype=np.int64)) if len(s) else 1 for s in self.shapes]
        self.bytes = [n * torch.empty((), dtype=d).element_size() for n, d in zip(self.numel, self.dtypes)]
        self.c_bytes = (C.c_int64 * len(self.bytes))(*self.bytes)

    def __len__(self):
        return len(self.shapes)

    def batch_of(self, fields):
        """Number of rows in `fields` (each either shape_i or [n, *shape_i])."""
        if len(fields) != len(self):
            raise ValueError("expected %d tensors per element, got %d" % (len(self), len(fields)))
        n = None
        for f, numel in zip(fields, self.numel):
            if isinstance(f, torch.Tensor):
                total = f.numel()
            elif hasattr(f, "shape") and not isinstance(f, np.ndarray):  # a DLPack producer: no host copy to count
                total = int(np.prod(tuple(f.shape), dtype=np.int64)) if len(tuple(f.shape)) else 1
            else:
                total = int(np.prod(tuple(np.shape(f)), dtype=np.int64)) if len(np.shape(f)) else 1
            if total % numel:
                raise ValueError("tensor of shape %s does not hold whole elements of %d values" % (tuple(np.shape(f)), numel))
            rows = total // numel
            if n is None:
                n = rows
            elif rows != n:
                raise ValueError("fields disagree on the number of rows (%d vs %d)" % (n, rows))
        return n

    def rows_if_ready(self, fields, dev):
        """Number of rows when `fields` already are contiguous device tensors of the declared dtypes holding
        whole elements (the training path: nothing to convert, one pass), else None."""
        if len(fields) != len(self.numel):
            return None
        n = -1
        for f, d, numel in zip(fields, self.dtypes, self.numel):
            if not (isinstance(f, torch.Tensor) and f.dtype == d and f.device == dev and f.is_contiguous()):
                return None
            rows, rest = divmod(f.numel(), numel)
            if rest or (n >= 0 and rows != n):
                return None
            n = rows
        return n

    def to_device(self, fields, dev):
        """Contiguous device tensors of the declared dtypes (copies host data if needed)."""
        out = []
        for f, d in zip(fields, self.dtypes):
            if isinstance(f, torch.Tensor) and f.is_cuda and f.dtype == d and f.is_contiguous() and f.device == dev:
                out.append(f)  # the common case: nothing to convert
                continue
            out.append(as_tensor(f).to(device=dev, dtype=d, non_blocking=False).contiguous())
        return out

    def empty(self, n, dev):
        """Output tensors [n, *shape_i] (or shape_i when n is None)."""
        if n is None:
            return [torch.empty(s, dtype=d, device=dev) for s, d in zip(self.shapes, self.dtypes)]
        return [torch.empty((n,) + s, dtype=d, device=dev) for s, d in zip(self.shapes, self.dtypes)]

    def check_out(self, out, n, dev):
        if len(out) != len(self):
            raise ValueError("out must hold %d tensors" % len(self))
        for t, s, d in zip(out, self.shapes, self.dtypes):
            want = ((n,) + s) if n is not None else s
            if tuple(t.shape) != want or t.dtype != d or t.device != dev or not t.is_contiguous():
                raise ValueError("out tensor must be contiguous %s %s on %s" % (want, d, dev))
        return list(out)


def flat_on_device(x, dtype, dev):
    """1-D contiguous device tensor of `dtype` holding x; x itself when it already is one (the common case
    on the training path: no conversion, no copy)."""
    if isinstance(x, torch.Tensor) and x.dtype == dtype and x.device == dev and x.is_contiguous():
        return x if x.dim() == 1 else x.reshape(-1)
    if not isinstance(x, torch.Tensor) and hasattr(x, "__dlpack__") and not isinstance(x, np.ndarray):
        x = as_tensor(x)
    return torch.as_tensor(x).to(device=dev, dtype=dtype).contiguous().reshape(-1)


def pointers(tensors):
    return _lib.ptr_array([t.data_ptr() for t in tensors])


def get_counters(fn, handle):
    arr = (C.c_int64 * 4)()
    _lib.check(fn(handle, arr))
    return [int(v) for v in arr]


def set_counters(fn, handle, values):
    arr = (C.c_int64 * 4)(*[int(v) - (1 << 64) if int(v) >= (1 << 63) else int(v) for v in values])
    _lib.check(fn(handle, arr))


def save_fields(views, nrows):
    """Host copies of the first `nrows` rows of each field's storage."""
    return [v[:nrows].cpu() for v in views]


def load_fields(views, saved, layout):
    if len(saved) != len(views):
        raise ValueError("state holds %d fields, buffer has %d" % (len(saved), len(views)))
    for v, t, shape, dtype in zip(views, saved, layout.shapes, layout.dtypes):
        t = torch.as_tensor(t)
        if tuple(t.shape[1:]) != shape or t.dtype != dtype or t.shape[0] > v.shape[0]:
            raise ValueError("saved field %s %s does not fit storage %s %s" % (tuple(t.shape), t.dtype, tuple(v.shape), dtype))
        v[: t.shape[0]].copy_(t)
