"""Element types accepted for a buffer's `types` argument.

The reference passes mindspore dtypes (mindspore_rl/core/uniform_replay_buffer.py:75,
example: `types = [ms.float32, ms.int32, ms.float32, ms.float32]`). Here the
same names are torch dtypes; numpy dtypes, type strings ("float32") and objects
whose str() ends in such a name (e.g. "mindspore.float32") are accepted too.
"""
import numpy as np
import torch

float16 = torch.float16
float32 = torch.float32
float64 = torch.float64
bfloat16 = torch.bfloat16
int8 = torch.int8
int16 = torch.int16
int32 = torch.int32
int64 = torch.int64
uint8 = torch.uint8
bool_ = torch.bool

_BY_NAME = {
    "float16": float16, "half": float16, "float32": float32, "float": float32, "float64": float64,
    "double": float64, "bfloat16": bfloat16, "int8": int8, "int16": int16, "int32": int32, "int": int32,
    "int64": int64, "long": int64, "uint8": uint8, "bool": bool_, "bool_": bool_,
}

__all__ = ["float16", "float32", "float64", "bfloat16", "int8", "int16", "int32", "int64", "uint8", "bool_",
           "as_torch_dtype", "itemsize"]


def as_torch_dtype(t):
    """Normalises a type designator to a torch dtype."""
    if isinstance(t, torch.dtype):
        return t
    if isinstance(t, str):
        name = t
    else:
        try:
            name = np.dtype(t).name
        except TypeError:
            name = str(t)
    name = name.split(".")[-1].lower()
    if name not in _BY_NAME:
        raise TypeError("unsupported element type %r" % (t,))
    return _BY_NAME[name]


def itemsize(t):
    return torch.empty((), dtype=as_torch_dtype(t)).element_size()
