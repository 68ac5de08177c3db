"""mrb_per_update_noalloc (update_priorities from a static device scratch, no allocation) against
mrb_per_update: both trees and the running max priority bit for bit, on two calls in a row, the second
with a smaller input, then a small call that takes the election-in-LDS path. Through ctypes -> C ABI."""
import ctypes as C

import numpy as np
import pytest
import torch

from gpu_util import bits, t2n

pytestmark = pytest.mark.gpu


def test_update_noalloc_matches_update():
    if not torch.cuda.is_available():
        pytest.fail("no HIP device: the GPU tests cannot run (there is no CPU fallback)")
    from mindrl_amd import _lib
    from mindrl_amd.core import PriorityReplayBuffer
    L = _lib.lib()
    rng = np.random.default_rng(77)
    cap = 50_000  # 16 tree levels: stamp pass, one rebuild round and the top
    shapes, types = [(3,), (1,)], [torch.float32, torch.int32]
    a = PriorityReplayBuffer(0.6, cap, 32, shapes, types, seed0=5)   # updated through mrb_per_update
    b = PriorityReplayBuffer(0.6, cap, 32, shapes, types, seed0=5)   # updated through mrb_per_update_noalloc
    rows = [torch.randn(cap, 3, device="cuda"), torch.arange(cap, dtype=torch.int32, device="cuda").reshape(cap, 1)]
    a.insert(*rows)
    b.insert(*rows)
    sp = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    for n in (20_000, 3_000, 700):  # the second smaller than the first; the third without a stamp pass
        idx = rng.integers(0, cap, n)
        idx[rng.integers(0, n, n // 10)] = idx[rng.integers(0, n, n // 10)]  # duplicates: last write wins
        pr = (np.abs(rng.normal(size=n)) + 1e-6).astype(np.float32)
        d_idx, d_pr = torch.from_numpy(idx).cuda(), torch.from_numpy(pr).cuda()
        _lib.check(L.mrb_per_update(a._h, d_idx.data_ptr(), d_pr.data_ptr(), n, sp))
        _lib.check(L.mrb_per_update_noalloc(b._h, d_idx.data_ptr(), d_pr.data_ptr(), n, sp))
        (sa, ma), (sb, mb) = a.export_tree(), b.export_tree()
        assert np.array_equal(bits(sa[1:]), bits(sb[1:])), "sum trees differ after n = %d" % n
        assert np.array_equal(bits(ma[1:]), bits(mb[1:])), "min trees differ after n = %d" % n
        assert np.float32(a.max_priority) == np.float32(b.max_priority)
        u = torch.from_numpy(rng.random(32).astype(np.float32)).cuda()
        oa, ob = a.sample(0.5, uniforms=u), b.sample(0.5, uniforms=u)
        assert np.array_equal(t2n(oa[0]), t2n(ob[0])) and np.array_equal(bits(t2n(oa[1])), bits(t2n(ob[1])))
    assert a.check() == 0 and b.check() == 0
    # more entries than the static scratch holds: a clear error, nothing enqueued
    big = torch.zeros(262_145, dtype=torch.int64, device="cuda")
    bigp = torch.ones(262_145, dtype=torch.float32, device="cuda")
    assert L.mrb_per_update_noalloc(b._h, big.data_ptr(), bigp.data_ptr(), 262_145, sp) == _lib.MRB_EINVAL
    assert b"262144" in L.mrb_last_error()
    _lib.check(L.mrb_per_update_noalloc(b._h, big.data_ptr(), bigp.data_ptr(), 262_144, sp))  # the limit itself is fine
    _lib.check(L.mrb_per_update(a._h, big.data_ptr(), bigp.data_ptr(), 262_144, sp))
    (sa, _), (sb, _) = a.export_tree(), b.export_tree()
    assert np.array_equal(bits(sa[1:]), bits(sb[1:]))
    a.destroy()
    b.destroy()
