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


def test_update_noalloc_allocates_nothing_replays_from_a_graph_and_takes_the_sparse_path():
    """What the entry point exists for: (1) the device's free memory is the same before and after its calls;
    (2) a call of at most 1024 entries recorded into a HIP graph replays, on new inputs, to the trees that the
    eager twin (mrb_per_update) builds; (3) on a tree of 23 levels a call of 5,000 entries - the entry-driven
    lowest round - and small calls (one wave's path walk, the election in LDS) match the twin bit for bit."""
    if not torch.cuda.is_available():
        pytest.fail("no HIP device: the GPU tests cannot run (there is no CPU fallback)")
    from mindrl_amd import _lib
    from mindrl_amd.core import PriorityReplayBuffer
    L = _lib.lib()
    rng = np.random.default_rng(78)
    shapes, types = [(1,)], [torch.int32]

    def twins(cap):
        a = PriorityReplayBuffer(0.6, cap, 32, shapes, types, seed0=5)
        b = PriorityReplayBuffer(0.6, cap, 32, shapes, types, seed0=5)
        for start in range(0, cap, 1 << 20):
            n = min(1 << 20, cap - start)
            rows = torch.arange(start, start + n, dtype=torch.int32, device="cuda").reshape(n, 1)
            a.insert(rows), b.insert(rows)
        return a, b

    def same_trees(a, b, what):
        (sa, ma), (sb, mb) = a.export_tree(), b.export_tree()
        assert np.array_equal(bits(sa[1:]), bits(sb[1:])), "sum trees differ: " + what
        assert np.array_equal(bits(ma[1:]), bits(mb[1:])), "min trees differ: " + what
        assert np.float32(a.max_priority) == np.float32(b.max_priority), what

    sp = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    # (3) and (1): 23 levels; 5,000 entries (sparse lowest round), 40 (one wave), 700 (election in LDS), 3,000
    a, b = twins(5_000_000)
    inputs = []
    for n in (5_000, 40, 700, 3_000):
        idx = rng.integers(0, 5_000_000, n)
        idx[: n // 10] = idx[0]  # duplicates: last write wins
        pr = (rng.pareto(1.5, n) + 1e-6).astype(np.float32)
        inputs.append((n, torch.from_numpy(idx).cuda(), torch.from_numpy(pr).cuda()))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for n, d_idx, d_pr in inputs:
        _lib.check(L.mrb_per_update_noalloc(b._h, d_idx.data_ptr(), d_pr.data_ptr(), n, sp))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "mrb_per_update_noalloc changed the device's free memory"
    for n, d_idx, d_pr in inputs:
        _lib.check(L.mrb_per_update(a._h, d_idx.data_ptr(), d_pr.data_ptr(), n, sp))
    same_trees(a, b, "5,000,000 leaves")
    a.destroy(), b.destroy()
    # (2): recorded once, replayed on new inputs
    a, b = twins(50_000)
    n = 1000
    d_idx = torch.zeros(n, dtype=torch.int64, device="cuda")
    d_pr = torch.ones(n, dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        graph.capture_begin()
        _lib.check(L.mrb_per_update_noalloc(b._h, d_idx.data_ptr(), d_pr.data_ptr(), n, C.c_void_p(side.cuda_stream)))
        graph.capture_end()
    torch.cuda.synchronize()
    for rep in range(4):
        idx = rng.integers(0, 50_000, n)
        idx[:50] = idx[0]
        pr = (rng.pareto(1.5, n) + 1e-6).astype(np.float32)
        d_idx.copy_(torch.from_numpy(idx)), d_pr.copy_(torch.from_numpy(pr))
        graph.replay()
        torch.cuda.synchronize()
        _lib.check(L.mrb_per_update(a._h, d_idx.data_ptr(), d_pr.data_ptr(), n, sp))
        same_trees(a, b, "replay %d" % rep)
        # eager work between the replays, through both entry points
        e_idx = torch.from_numpy(rng.integers(0, 50_000, 2_000)).cuda()
        e_pr = torch.from_numpy((rng.pareto(1.5, 2_000) + 1e-6).astype(np.float32)).cuda()
        _lib.check(L.mrb_per_update(a._h, e_idx.data_ptr(), e_pr.data_ptr(), 2_000, sp))
        _lib.check(L.mrb_per_update_noalloc(b._h, e_idx.data_ptr(), e_pr.data_ptr(), 2_000, sp))
        same_trees(a, b, "eager after replay %d" % rep)
    assert a.check() == 0 and b.check() == 0
    del graph
    a.destroy(), b.destroy()
