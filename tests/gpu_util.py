"""Helpers for the GPU parity tests: run the same operation on the HIP buffer
(through the Python classes, i.e. ctypes -> C ABI -> kernels) and on the CPU
oracle, and compare."""
import numpy as np
import torch


def t2n(t):
    return t.detach().cpu().numpy()


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.int32)


def assert_tree_equal(per_gpu, per_cpu, what=""):
    gs, gm = per_gpu.export_tree()
    cs, cm = per_cpu.export_tree()
    assert gs.size == cs.size, what
    bad = np.nonzero(bits(gs[1:]) != bits(cs[1:]))[0]
    assert bad.size == 0, "%s: sum tree differs at heap nodes %s (gpu %s cpu %s)" % (
        what, bad[:8] + 1, gs[1:][bad[:8]], cs[1:][bad[:8]])
    bad = np.nonzero(bits(gm[1:]) != bits(cm[1:]))[0]
    assert bad.size == 0, "%s: min tree differs at heap nodes %s" % (what, bad[:8] + 1)
    return gs, gm


def assert_sample_equal(g_out, c_out, what="", rtol=1e-6):
    """Indices and rows bit-exact; weights within rtol (fp32, tolerance of the parity contract)."""
    gi, gw, gf = t2n(g_out[0]), t2n(g_out[1]), [t2n(f) for f in g_out[2:]]
    ci, cw, cf = c_out
    assert gi.dtype == np.int64 and gw.dtype == np.float32
    assert np.array_equal(gi, ci), "%s: indices differ at %s" % (what, np.nonzero(gi != ci)[0][:8])
    np.testing.assert_allclose(gw, cw, rtol=rtol, atol=0, err_msg=what)
    if cf is not None:
        for k, (a, b) in enumerate(zip(gf, cf)):
            assert a.shape == b.shape and a.dtype == b.dtype, (what, k, a.shape, b.shape, a.dtype, b.dtype)
            assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), "%s: field %d rows differ" % (what, k)
    return bool(np.array_equal(bits(gw), bits(cw)))


NP2T = {np.dtype(np.float32): torch.float32, np.dtype(np.int32): torch.int32, np.dtype(np.int64): torch.int64,
        np.dtype(np.uint8): torch.uint8, np.dtype(np.bool_): torch.bool, np.dtype(np.float16): torch.float16,
        np.dtype(np.int16): torch.int16, np.dtype(np.float64): torch.float64, np.dtype(np.int8): torch.int8}


def torch_types(dtypes):
    return [NP2T[np.dtype(d)] for d in dtypes]


def random_rows(rng, n, shapes, dtypes):
    out = []
    for s, d in zip(shapes, dtypes):
        d = np.dtype(d)
        if d == np.bool_:
            out.append(rng.random((n,) + tuple(s)) < 0.3)
        elif d.kind == "f":
            out.append(rng.normal(size=(n,) + tuple(s)).astype(d))
        else:
            info = np.iinfo(d)
            out.append(rng.integers(max(info.min, -1000), min(info.max, 1000) + 1, (n,) + tuple(s)).astype(d))
    return out


def to_dev(arrays):
    return [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in arrays]
