"""GPU parity: the HIP library (through ctypes and the C ABI) against the CPU
oracle on identical seeded inputs. Bar: indices, gathered rows, ring contents
and both trees bit-exact; importance weights within 1e-6 relative (fp32)."""
import ctypes as C

import numpy as np
import pytest
import torch

from gpu_util import (assert_sample_equal, assert_tree_equal, bits, random_rows, t2n, to_dev, torch_types)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mrb():
    if not torch.cuda.is_available():
        pytest.fail("no HIP device: the GPU parity tests cannot run (there is no CPU fallback)")
    from mindrl_amd import _lib
    from mindrl_amd.core import PriorityReplayBuffer, ReservoirReplayBuffer, UniformReplayBuffer
    _lib.lib()

    class NS:
        pass

    ns = NS()
    ns.lib, ns.PER, ns.URB, ns.RES = _lib, PriorityReplayBuffer, UniformReplayBuffer, ReservoirReplayBuffer
    yield ns


# ------------------------------------------------------------------ uniform
URB_LAYOUTS = [
    ([(4,), (1,), (1,), (4,), (1,)], [np.float32, np.int32, np.float32, np.float32, np.bool_]),   # 41 B row
    ([(17,), (6,), (1,), (17,), (1,)], [np.float32, np.float32, np.float32, np.float32, np.bool_]),  # 165 B row
    ([(3, 5), (2,), (7,)], [np.float16, np.int64, np.uint8]),
    ([(64,), (1,)], [np.float32, np.int16]),
]


@pytest.mark.parametrize("layout", range(len(URB_LAYOUTS)))
@pytest.mark.parametrize("cap", [1, 7, 64, 1000])
def test_uniform_ring_random_ops(mrb, orc, layout, cap):
    shapes, dtypes = URB_LAYOUTS[layout]
    rng = np.random.default_rng(100 * layout + cap)
    g = mrb.URB(8, cap, shapes, torch_types(dtypes), seed=77)
    c = orc.OracleUniform(cap, shapes, dtypes, seed=77)
    for step in range(25):
        n = int(rng.integers(1, 2 * cap + 3)) if step % 5 else 1
        rows = random_rows(rng, n, shapes, dtypes)
        if n == 1 and step % 2:
            g.insert([torch.from_numpy(r[0]).cuda() for r in rows])  # single element, shape_i
        else:
            g.insert(to_dev(rows))
        c.append(rows, n)
        assert int(g.count) == c.count and int(g.head) == c.head
        assert int(g.size()) == c.count and bool(g.full()[0]) == (c.count >= cap)
        for f in range(len(shapes)):  # raw storage, slot by slot
            assert np.array_equal(t2n(g.buffer[f]).view(np.uint8), c.field(f).view(np.uint8)), (step, f)
        j = int(rng.integers(-c.count, c.count))
        for a, b in zip(g.get_item(j), c.get_item(j)):
            assert np.array_equal(t2n(a).view(np.uint8), b.view(np.uint8))
        idx = rng.integers(0, c.count, 33)
        for a, b in zip(g.sample(indices=torch.from_numpy(idx).cuda()), c.gather(idx)):
            assert np.array_equal(t2n(a).view(np.uint8), b.view(np.uint8))
        if c.count >= 8:
            gi, gf = g.sample_with_indices()
            ci, cf = c.sample(8)
            assert np.array_equal(t2n(gi), ci)
            for a, b in zip(gf, cf):
                assert np.array_equal(t2n(a).view(np.uint8), b.view(np.uint8))
        if step == 12:
            g.reset()
            c.reset()
    g.check()
    g.destroy()


@pytest.mark.parametrize("layout,cap", [(0, 37), (1, 5000)])
def test_uniform_loop_recorded_into_a_hip_graph_with_device_counters(mrb, orc, layout, cap):
    """The loop the reference compiles as one graph (mindspore_rl/algorithm/dqn/dqn_trainer.py:65-88: insert, then
    sample, every step) on the uniform buffer: insert 3 rows + sample, recorded ONCE with device_counters and
    replayed 20 times on new rows - the buffer grows, fills, wraps and the draws move on; every replay against the
    oracle, with eager get_item / gather / insert / reset between replays and the counters read back."""
    shapes, dtypes = URB_LAYOUTS[layout]
    rng = np.random.default_rng(7 * cap + layout)
    batch, nin = 8, 3
    g = mrb.URB(batch, cap, shapes, torch_types(dtypes), seed=21)
    c = orc.OracleUniform(cap, shapes, dtypes, seed=21)
    first = random_rows(rng, cap - 25, shapes, dtypes)
    g.insert(to_dev(first)), c.append(first, cap - 25)
    g.set_option("device_counters", 1)
    new_rows = [torch.zeros((nin,) + tuple(s), dtype=t).cuda() for s, t in zip(shapes, torch_types(dtypes))]
    out = g._layout.empty(batch, g._dev)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        graph.capture_begin()
        g.insert(new_rows)
        g.sample(out=out)
        graph.capture_end()
    torch.cuda.synchronize()
    for rep in range(20):
        fresh = random_rows(rng, nin, shapes, dtypes)
        for dst, src in zip(new_rows, fresh):
            dst.copy_(torch.from_numpy(src))
        graph.replay()
        torch.cuda.synchronize()
        c.append(fresh, nin)
        _, want = c.sample(batch)
        for a, b in zip(out, want):
            assert np.array_equal(t2n(a).view(np.uint8), b.view(np.uint8)), (cap, rep)
        assert int(g.count) == c.count and int(g.head) == c.head, (cap, rep)
        for f in range(len(shapes)):
            assert np.array_equal(t2n(g.buffer[f]).view(np.uint8), c.field(f).view(np.uint8)), (cap, rep, f)
        if rep % 4 == 1:  # eager calls in between
            j = int(rng.integers(-c.count, c.count))
            for a, b in zip(g.get_item(j), c.get_item(j)):
                assert np.array_equal(t2n(a).view(np.uint8), b.view(np.uint8))
            idx = rng.integers(0, c.count, 19)
            for a, b in zip(g.sample(indices=torch.from_numpy(idx).cuda()), c.gather(idx)):
                assert np.array_equal(t2n(a).view(np.uint8), b.view(np.uint8))
            more = random_rows(rng, 7, shapes, dtypes)
            g.insert(to_dev(more)), c.append(more, 7)
            gi, gf = g.sample_with_indices()
            ci, cf = c.sample(batch)
            assert np.array_equal(t2n(gi), ci)
            for a, b in zip(gf, cf):
                assert np.array_equal(t2n(a).view(np.uint8), b.view(np.uint8))
        if rep == 13:
            g.reset(), c.reset()
            refill = random_rows(rng, batch + 2, shapes, dtypes)
            g.insert(to_dev(refill)), c.append(refill, batch + 2)
    g.check()
    g.set_option("device_counters", 0)
    assert int(g.count) == c.count and int(g.head) == c.head
    gi, gf = g.sample_with_indices()
    ci, cf = c.sample(batch)
    assert np.array_equal(t2n(gi), ci)
    del graph
    g.destroy()


def test_config2_sac_shape_full_size(mrb, orc):
    """The benchmark's config 2 at its real size: capacity 1,000,000, rows f32[17] + f32[6] + f32[1] + f32[17] + bool
    (165 B, mindspore_rl/algorithm/sac/config.py:95-100), filled by 1000 appends of 1000 rows
    (mindspore_rl/core/uniform_replay_buffer.py:101-115), then batches of 256 gathered at seeded host-drawn
    indices integers(0, count) (uniform_replay_buffer.py:130-139). Storage, count / head and every gathered
    row are compared with the oracle."""
    shapes, dtypes = URB_LAYOUTS[1]
    cap, chunk, batch = 1_000_000, 1000, 256
    rng = np.random.default_rng(1002)
    g = mrb.URB(batch, cap, shapes, torch_types(dtypes), seed=1002)
    c = orc.OracleUniform(cap, shapes, dtypes, seed=1002)
    for i in range(cap // chunk + 3):  # three chunks past the capacity: the ring wraps
        rows = [rng.normal(size=(chunk, 17)).astype(np.float32), rng.uniform(-1, 1, (chunk, 6)).astype(np.float32),
                rng.normal(size=(chunk, 1)).astype(np.float32), rng.normal(size=(chunk, 17)).astype(np.float32),
                rng.random((chunk, 1)) < 0.01]
        g.insert(to_dev(rows))
        c.append(rows, chunk)
        if i in (0, 499, cap // chunk - 1, cap // chunk + 2):
            assert (int(g.count), int(g.head)) == (c.count, c.head), i
    assert (c.count, c.head) == (cap, 3 * chunk)
    for f in range(len(shapes)):
        assert np.array_equal(t2n(g.buffer[f]).view(np.uint8), c.field(f).view(np.uint8)), f
    for call in range(20):
        idx = rng.integers(0, c.count, batch)
        for a, b in zip(g.sample(indices=torch.from_numpy(idx).cuda()), c.gather(idx)):
            assert np.array_equal(t2n(a).view(np.uint8), b.view(np.uint8)), call
    gi, gf = g.sample_with_indices()  # the buffer's own generator on the full ring
    ci, cf = c.sample(batch)
    assert np.array_equal(t2n(gi), ci)
    for a, b in zip(gf, cf):
        assert np.array_equal(t2n(a).view(np.uint8), b.view(np.uint8))
    for j in (0, -1, cap // 2):
        for a, b in zip(g.get_item(j), c.get_item(j)):
            assert np.array_equal(t2n(a).view(np.uint8), b.view(np.uint8))
    g.check()
    g.destroy()


@pytest.mark.parametrize("shape", ["wide", "deep", "narrow"])
def test_sample_many_equals_successive_samples(mrb, orc, shape):
    """mrb_per_sample_many against the oracle's successive sample() calls: with given draws and with the
    generator (whose call counter then advances by the number of batches), on wide rows (one launch), on
    a 21-level tree (shared top group) and through the LDS-top kernel (one launch per batch)."""
    rng = np.random.default_rng(99)
    if shape == "wide":
        shapes, dtypes, cap, batch, path = [(300,), (1,), (3,)], [np.float32, np.int32, np.uint8], 3000, 48, 1
    elif shape == "deep":
        shapes, dtypes, cap, batch, path = [(2,)], [np.float32], (1 << 20) + 5, 40, 1
    else:
        shapes, dtypes, cap, batch, path = [(1,), (1,)], [np.int32, np.float32], 5000, 64, 2
    g, c = make_pair(mrb, orc, 0.6, cap, batch, seed=21, shapes=shapes, dtypes=dtypes)
    g.set_option("sample_path", path)
    fill = min(cap, 6000)
    rows = random_rows(rng, fill, shapes, dtypes)
    g.insert(*to_dev(rows)), c.push(rows, fill)
    idx = rng.integers(0, fill, 900)
    pr = (rng.pareto(1.5, 900) + 1e-6).astype(np.float32)
    g.update_priorities(torch.from_numpy(idx).cuda(), torch.from_numpy(pr).cuda()), c.update(idx, pr)
    for nb in (1, 3, 7):
        u = rng.random((nb, batch)).astype(np.float32)
        got = g.sample_many(nb, 0.6, uniforms=torch.from_numpy(u).cuda())
        gen = g.sample_many(nb, 0.6)
        for i in range(nb):
            assert_sample_equal([x[i] for x in got], c.sample(batch, 0.6, u[i]), "%s nb %d batch %d" % (shape, nb, i))
        for i in range(nb):
            assert_sample_equal([x[i] for x in gen], c.sample(batch, 0.6), "%s generator nb %d batch %d" % (shape, nb, i))
    assert_sample_equal(g.sample(0.6), c.sample(batch, 0.6), "generator position after sample_many")
    with pytest.raises(ValueError):
        g.sample_many(0, 0.5)
    g.check()
    g.destroy()


@pytest.mark.parametrize("path", [1, 2])
def test_hip_graph_replays_update_and_sample(mrb, orc, path):
    """update_priorities (<= 1024 entries) + sample with given draws, recorded once into a HIP graph and
    replayed five times on new inputs, with eager calls and synchronisations between the replays: every
    replay equals the oracle's update + sample, and so does the eager work in between."""
    rng = np.random.default_rng(31 + path)
    shapes, dtypes = ([(300,), (1,)], [np.float32, np.int32]) if path == 1 else ([(1,), (2,)], [np.int32, np.float32])
    cap, batch, nupd = 3000, 64, 200
    g, c = make_pair(mrb, orc, 0.6, cap, batch, seed=5, shapes=shapes, dtypes=dtypes)
    g.set_option("sample_path", path)
    rows = random_rows(rng, cap, shapes, dtypes)  # a full buffer: the number of stored rows stays what was recorded
    g.insert(*to_dev(rows)), c.push(rows, cap)
    u_dev = torch.zeros(batch, dtype=torch.float32, device="cuda")
    idx_dev = torch.zeros(nupd, dtype=torch.int64, device="cuda")
    pr_dev = torch.ones(nupd, dtype=torch.float32, device="cuda")
    out = (torch.empty(batch, dtype=torch.int64, device="cuda"), torch.empty(batch, dtype=torch.float32, device="cuda"),
           g._layout.empty(batch, g._dev))
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        graph.capture_begin()
        g.update_priorities(idx_dev, pr_dev)
        g.sample(0.7, uniforms=u_dev, out=out)
        graph.capture_end()
    torch.cuda.synchronize()
    for rep in range(5):
        idx = rng.integers(0, cap, nupd)
        idx[:20] = idx[0]  # duplicates: the last entry wins
        pr = (rng.pareto(1.5, nupd) + 1e-6).astype(np.float32)
        u = rng.random(batch).astype(np.float32)
        idx_dev.copy_(torch.from_numpy(idx)), pr_dev.copy_(torch.from_numpy(pr)), u_dev.copy_(torch.from_numpy(u))
        graph.replay()
        torch.cuda.synchronize()
        c.update(idx, pr)
        assert_sample_equal((out[0], out[1]) + tuple(out[2]), c.sample(batch, 0.7, u), "path %d replay %d" % (path, rep))
        assert_tree_equal(g, c, "path %d replay %d" % (path, rep))
        # eager work between the replays
        e_idx = rng.integers(0, cap, 50)
        e_pr = (rng.pareto(1.5, 50) + 1e-6).astype(np.float32)
        g.update_priorities(torch.from_numpy(e_idx).cuda(), torch.from_numpy(e_pr).cuda()), c.update(e_idx, e_pr)
        u2 = rng.random(batch).astype(np.float32)
        assert_sample_equal(g.sample(0.4, uniforms=torch.from_numpy(u2).cuda()), c.sample(batch, 0.4, u2), "eager %d" % rep)
    del graph
    g.destroy()


@pytest.mark.parametrize("cap,path", [(3000, 1), (70000, 1), (70000, 2), (3_000_000, 1)])
def test_hip_graph_replays_a_whole_loop_with_device_counters(mrb, orc, cap, path):
    """push 3 rows + generator-driven sample + update_priorities of the sampled rows, recorded ONCE with the
    option device_counters and replayed 12 times on new rows and priorities: the buffer fills up, the ring wraps,
    the draws advance - every replay equals the oracle's push, sample, update; eager calls between replays keep
    working, and the counters read back agree."""
    rng = np.random.default_rng(cap)
    # (trees of 12, 17 and 22 levels: the top alone, one round fused with it, two rounds in launches of their own)
    shapes, dtypes = ([(300,), (1,), (2,)], [np.float32, np.int32, np.uint8]) if cap < 10 ** 6 else ([(2,), (1,)], [np.float32, np.int32])
    batch, npush = 48, 3
    g, c = make_pair(mrb, orc, 0.6, cap, batch, seed=13, shapes=shapes, dtypes=dtypes)
    fill = cap - 20  # not full: the row count changes during the replays, then the ring wraps
    rows = random_rows(rng, fill, shapes, dtypes)
    g.insert(*to_dev(rows)), c.push(rows, fill)
    g.set_option("device_counters", 1)
    g.set_option("sample_path", path)
    new_rows = [torch.zeros((npush,) + tuple(s), dtype=t).cuda() for s, t in zip(shapes, torch_types(dtypes))]
    prio_rows = [torch.zeros((2,) + tuple(s), dtype=t).cuda() for s, t in zip(shapes, torch_types(dtypes))]
    prio_dev = torch.ones(2, dtype=torch.float32, device="cuda")  # a second push, with priorities of its own
    pr_dev = torch.ones(batch, dtype=torch.float32, device="cuda")
    out = (torch.empty(batch, dtype=torch.int64, device="cuda"), torch.empty(batch, dtype=torch.float32, device="cuda"),
           g._layout.empty(batch, g._dev))
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        graph.capture_begin()
        g.insert(*new_rows)
        g.insert(*prio_rows, priorities=prio_dev)
        g.sample(0.5, out=out)
        g.update_priorities(out[0], pr_dev)
        graph.capture_end()
    torch.cuda.synchronize()
    for rep in range(12):
        fresh = random_rows(rng, npush, shapes, dtypes)
        fresh2 = random_rows(rng, 2, shapes, dtypes)
        ppr = (rng.pareto(1.5, 2) + 1e-6).astype(np.float32)
        pr = (rng.pareto(1.5, batch) + 1e-6).astype(np.float32)
        for dst, src in zip(new_rows + prio_rows, fresh + fresh2):
            dst.copy_(torch.from_numpy(src))
        pr_dev.copy_(torch.from_numpy(pr)), prio_dev.copy_(torch.from_numpy(ppr))
        graph.replay()
        torch.cuda.synchronize()
        c.push(fresh, npush)
        c.push(fresh2, 2, ppr)
        want = c.sample(batch, 0.5)
        assert_sample_equal((out[0], out[1]) + tuple(out[2]), want, "cap %d replay %d" % (cap, rep))
        c.update(want[0], pr)
        assert_tree_equal(g, c, "cap %d replay %d" % (cap, rep))
        assert g.size() == c.size and g._state()[1] == c.head
        if rep % 3 == 1:  # eager calls in between use the same counters
            extra = random_rows(rng, 5, shapes, dtypes)
            g.insert(*to_dev(extra)), c.push(extra, 5)
            assert_sample_equal(g.sample(0.9), c.sample(batch, 0.9), "eager after replay %d" % rep)
            if cap >= 70000:  # a push too large for the one-launch rebuild, with priorities, placed by the device
                big = random_rows(rng, 4500, shapes, dtypes)
                bpr = (rng.pareto(1.5, 4500) + 1e-6).astype(np.float32)
                g.insert(*to_dev(big), priorities=torch.from_numpy(bpr).cuda()), c.push(big, 4500, bpr)
                assert_tree_equal(g, c, "cap %d big push after replay %d" % (cap, rep))
            two = g.sample_many(2, 0.6)  # two batches in one launch: the generator moves on by two calls
            for i in range(2):
                assert_sample_equal([x[i] for x in two], c.sample(batch, 0.6), "eager sample_many after replay %d" % rep)
    with pytest.raises(ValueError):
        g.update_priorities(torch.zeros(2000, dtype=torch.int64).cuda(), torch.ones(2000).cuda())
    g.set_option("device_counters", 0)
    assert g.size() == c.size
    assert_sample_equal(g.sample(0.3), c.sample(batch, 0.3), "after switching back")
    del graph
    g.destroy()


@pytest.mark.parametrize("cap", [1, 2, 5, 1000, 70_000, 3_000_000])
def test_single_row_pushes(mrb, orc, cap):
    """insert() of one row - one wave's walk from the leaf to the root - on trees of 0 to 22 levels: plain pushes,
    pushes with a priority (valid, zero, above the running max, invalid: flagged, the row takes the running max),
    across the ring's wrap, compared with the oracle after every push; then the same recorded ONCE into a HIP graph
    with the ring position on the device and replayed on new rows and priorities."""
    rng = np.random.default_rng(9300 + cap % 1000)
    shapes, dtypes = [(3,), (1,)], [np.float32, np.int32]
    g, c = make_pair(mrb, orc, 0.6, cap, 4, seed=5, shapes=shapes, dtypes=dtypes)
    fill = max(0, cap - 7)
    if fill:
        rows = random_rows(rng, fill, shapes, dtypes)
        pr = rng.lognormal(0, 1, fill).astype(np.float32)
        g.insert(*to_dev(rows), priorities=torch.from_numpy(pr).cuda()), c.push(rows, fill, pr)
    for step in range(24):
        row = random_rows(rng, 1, shapes, dtypes)
        kind = step % 6
        what = "cap %d step %d kind %d" % (cap, step, kind)
        if kind in (0, 3):
            g.insert(*to_dev(row)), c.push(row, 1)
        else:
            p = np.array([{1: rng.pareto(1.5) + 1e-6, 2: 0.0, 4: float(c.max_priority) * 3 + 1, 5: np.nan}[kind]], np.float32)
            g.insert(*to_dev(row), priorities=torch.from_numpy(p).cuda())
            if kind == 5:
                c.push(row, 1)  # an invalid priority: the row keeps the running max, the call is flagged
                with pytest.raises(ValueError):
                    g.check()
            else:
                c.push(row, 1, p)
        assert_tree_equal(g, c, what)
        assert bits(np.float32(g.max_priority)) == bits(np.float32(c.max_priority)), what
        assert g.size() == c.size and g._state()[1] == c.head, what
    g.check()
    u = rng.random(4).astype(np.float32)
    assert_sample_equal(g.sample(0.5, uniforms=torch.from_numpy(u).cuda()), c.sample(4, 0.5, u), "cap %d" % cap)
    # recorded once, replayed: the ring position lives on the device
    g.set_option("device_counters", 1)
    one = [torch.zeros((1,) + tuple(sh), dtype=t).cuda() for sh, t in zip(shapes, torch_types(dtypes))]
    two = [torch.zeros((1,) + tuple(sh), dtype=t).cuda() for sh, t in zip(shapes, torch_types(dtypes))]
    p_dev = torch.ones(1, dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        graph.capture_begin()
        g.insert(*one)
        g.insert(*two, priorities=p_dev)
        graph.capture_end()
    torch.cuda.synchronize()
    for rep in range(10):
        r1, r2 = random_rows(rng, 1, shapes, dtypes), random_rows(rng, 1, shapes, dtypes)
        p = (rng.pareto(1.5, 1) + 1e-6).astype(np.float32)
        for dst, src in zip(one + two, r1 + r2):
            dst.copy_(torch.from_numpy(src))
        p_dev.copy_(torch.from_numpy(p))
        graph.replay()
        torch.cuda.synchronize()
        c.push(r1, 1), c.push(r2, 1, p)
        assert_tree_equal(g, c, "cap %d replay %d" % (cap, rep))
        assert g.size() == c.size and g._state()[1] == c.head
    g.set_option("device_counters", 0)
    del graph
    g.destroy()


def test_sample_output_ring(mrb, orc):
    """sample() hands out preallocated output sets in turn: `output_ring` calls return distinct tensors, the
    next call reuses the first set; output_ring=0 allocates fresh tensors; an explicit out= is written in
    place. The results are the oracle's in every mode."""
    shapes, dtypes = [(6,), (1,)], [np.float32, np.int32]
    rng = np.random.default_rng(12)
    cap, batch = 500, 16
    rows = random_rows(rng, cap, shapes, dtypes)
    for ring in (3, 0):
        g = mrb.PER(0.6, cap, batch, shapes, torch_types(dtypes), seed0=6, output_ring=ring)
        c = orc.OraclePER(0.6, cap, shapes, dtypes, seed=6)
        g.insert(*to_dev(rows)), c.push(rows, cap)
        outs = []
        for call in range(4):
            out = g.sample(0.5)
            assert_sample_equal(out, c.sample(batch, 0.5), "ring %d call %d" % (ring, call))
            outs.append(out)
        ptrs = [o[2].data_ptr() for o in outs]
        if ring:
            assert len(set(ptrs[:3])) == 3 and ptrs[3] == ptrs[0]  # the fourth call overwrote the first batch
            assert torch.equal(outs[3][0], outs[0][0])
        else:
            assert len(set(ptrs)) == 4
        mine = (torch.empty(batch, dtype=torch.int64, device="cuda"), torch.empty(batch, device="cuda"),
                [torch.empty((batch,) + s, dtype=t, device="cuda") for s, t in zip(shapes, torch_types(dtypes))])
        u = rng.random(batch).astype(np.float32)
        back = g.sample(0.5, uniforms=torch.from_numpy(u).cuda(), out=mine)
        assert back[0].data_ptr() == mine[0].data_ptr() and back[2].data_ptr() == mine[2][0].data_ptr()
        assert_sample_equal(back, c.sample(batch, 0.5, u), "out=")
        g.destroy()


def test_options_belong_to_one_buffer(mrb, orc):
    """Two prioritized buffers with the same contents, one forced onto the wide-row kernel with three
    workgroups per row, the other onto the LDS-top kernel with 5 staged levels: interleaved calls give the
    same bit-exact results, i.e. no option of one handle reaches the other."""
    shapes, dtypes = [(300,), (1,)], [np.float32, np.int32]  # a 1200-byte field: wide rows
    rng = np.random.default_rng(8)
    cap, batch = 3000, 64
    a, c = make_pair(mrb, orc, 0.6, cap, batch, seed=4, shapes=shapes, dtypes=dtypes)
    b = mrb.PER(0.6, cap, batch, shapes, torch_types(dtypes), seed0=4)
    a.set_option("sample_path", 1), a.set_option("row_split", 3)
    b.set_option("sample_path", 2), b.set_option("lds_levels", 5)
    with pytest.raises(ValueError):
        a.set_option("no_such_option", 1)
    with pytest.raises(ValueError):
        a.set_option("row_split", 1000)
    u = mrb.URB(8, 10, shapes, torch_types(dtypes))
    with pytest.raises(ValueError):
        u.set_option("sample_path", 1)  # an option of prioritized buffers
    u.set_option("row_split", 2)
    u.destroy()
    rows = random_rows(rng, cap, shapes, dtypes)
    a.insert(*to_dev(rows)), b.insert(*to_dev(rows)), c.push(rows, cap)
    for step in range(6):
        idx = rng.integers(0, cap, 500)
        pr = (rng.pareto(1.5, 500) + 1e-6).astype(np.float32)
        for buf in (a, b):
            buf.update_priorities(torch.from_numpy(idx).cuda(), torch.from_numpy(pr).cuda())
        c.update(idx, pr)
        un = rng.random(batch).astype(np.float32)
        want = c.sample(batch, 0.5, un)
        assert_sample_equal(a.sample(0.5, uniforms=torch.from_numpy(un).cuda()), want, "wide step %d" % step)
        assert_sample_equal(b.sample(0.5, uniforms=torch.from_numpy(un).cuda()), want, "lds step %d" % step)
    a.destroy(), b.destroy()


def test_uniform_primitive_attributes_used_by_reference_callers(mrb):
    """A subclass written like mindspore_rl/algorithm/mappo/mappo_replaybuffer.py:23-44 works unchanged,
    and buffer_sample.batch_size is readable (mindspore_rl/algorithm/gail/gail.py:163-164)."""

    class ConditionalBuffer(mrb.URB):
        def construct(self, exp, command):
            if command:
                self.buffer_append(self.buffer, exp, self.count, self.head)
            return self.buffer

    b = ConditionalBuffer(4, 10, [(2,)], [torch.float32])
    b.construct([torch.ones(2).cuda()], False)
    assert int(b.count) == 0
    out = b.construct([torch.ones(2).cuda() * 3], True)
    assert int(b.count) == 1 and float(out[0][0, 0]) == 3.0
    assert b.buffer_sample.batch_size == 4
    assert float(b.buffer_get(b.buffer, b.count, b.head, 0)[0][1]) == 3.0
    b.destroy()


def test_uniform_successive_samples_differ_and_errors(mrb):
    g = mrb.URB(32, 200, [(1,)], [torch.int32], seed=5)
    with pytest.raises(ValueError):
        g.sample()  # batch > count (empty)
    g.insert([torch.arange(200, dtype=torch.int32).reshape(200, 1).cuda()])
    a = t2n(g.sample()[0])
    b = t2n(g.sample()[0])
    assert not np.array_equal(a, b) and a.min() >= 0 and a.max() < 200  # rows hold their own slot number
    with pytest.raises(ValueError):
        g.get_item(200)
    g.sample(indices=torch.tensor([0, 500, -3]).cuda())
    with pytest.raises(IndexError):
        g.check()
    g.check()  # flags cleared by the failing check
    g.destroy()
    with pytest.raises(ValueError):
        g._state()  # destroyed handle
    with pytest.raises(ValueError):
        mrb.URB(1, 0, [(1,)], [torch.int32])


# ------------------------------------------------------------------ checkpoint
def test_state_dict_round_trip_continues_identically(mrb, tmp_path):
    """A buffer restored from state_dict() (through torch.save / torch.load(weights_only=True)) into a
    fresh buffer behaves exactly like the original from then on: same storage, same trees, same draws."""
    rng = np.random.default_rng(77)
    shapes, dtypes = [(5,), (1,)], [np.float32, np.int32]

    def reload(state):
        torch.save(state, tmp_path / "buf.pt")
        return torch.load(tmp_path / "buf.pt", weights_only=True)

    # prioritized: wrapped ring, updated priorities, generator advanced
    a = mrb.PER(0.6, 300, 16, shapes, torch_types(dtypes), seed0=5)
    a.insert(*to_dev(random_rows(rng, 450, shapes, dtypes)))
    a.update_priorities(torch.from_numpy(rng.integers(0, 300, 200)).cuda(),
                        torch.from_numpy(rng.pareto(1.5, 200).astype(np.float32) + 1e-6).cuda())
    a.sample(0.4)
    b = mrb.PER(0.6, 300, 16, shapes, torch_types(dtypes), seed0=999)
    b.load_state_dict(reload(a.state_dict()))
    for step in range(5):
        sa, sb = a.export_tree(), b.export_tree()
        assert np.array_equal(bits(sa[0][1:]), bits(sb[0][1:])) and np.array_equal(bits(sa[1][1:]), bits(sb[1][1:]))
        assert a.max_priority == b.max_priority and a._state()[:2] == b._state()[:2]
        oa, ob = a.sample(0.7), b.sample(0.7)
        for x, y in zip(oa, ob):
            assert torch.equal(x, y)
        rows = to_dev(random_rows(rng, 7, shapes, dtypes))
        a.insert(*rows), b.insert(*rows)
        a.update_priorities(oa[0], oa[1] + 0.5), b.update_priorities(ob[0], ob[1] + 0.5)
    a.destroy(), b.destroy()
    # an empty prioritized buffer round-trips too
    e = mrb.PER(0.6, 10, 2, shapes, torch_types(dtypes), seed0=1)
    f = mrb.PER(0.6, 10, 2, shapes, torch_types(dtypes), seed0=2)
    f.load_state_dict(reload(e.state_dict()))
    assert f.size() == 0
    e.destroy(), f.destroy()

    # uniform: wrapped ring
    u = mrb.URB(8, 50, shapes, torch_types(dtypes), seed=3)
    u.insert(to_dev(random_rows(rng, 70, shapes, dtypes)))
    u.sample()
    w = mrb.URB(8, 50, shapes, torch_types(dtypes), seed=4)
    w.load_state_dict(reload(u.state_dict()))
    assert (int(u.count), int(u.head)) == (int(w.count), int(w.head)) == (50, 20)
    for x, y in zip(u.sample(), w.sample()):
        assert torch.equal(x, y)
    for x, y in zip(u.get_item(0), w.get_item(0)):
        assert torch.equal(x, y)
    with pytest.raises(ValueError):
        mrb.URB(8, 51, shapes, torch_types(dtypes)).load_state_dict(u.state_dict())
    u.destroy(), w.destroy()

    # reservoir: past capacity
    r = mrb.RES(20, 8, shapes, torch_types(dtypes), seed1=6)
    r.push(*to_dev(random_rows(rng, 90, shapes, dtypes)))
    q = mrb.RES(20, 8, shapes, torch_types(dtypes), seed1=7)
    q.load_state_dict(reload(r.state_dict()))
    more = to_dev(random_rows(rng, 40, shapes, dtypes))
    r.push(*more), q.push(*more)
    for x, y in zip(r.storage(), q.storage()):
        assert torch.equal(x, y)
    for x, y in zip(r.sample(), q.sample()):
        assert torch.equal(x, y)
    r.destroy(), q.destroy()


def test_state_dict_cross_loads_with_the_oracle(mrb, orc):
    """The checkpoint path against the oracle, both ways: a state saved by the HIP buffer is loaded into
    an oracle buffer, a state saved by an oracle buffer into a fresh HIP buffer; each pair then continues
    with identical calls and must agree bit for bit (trees, running max, draws, rows, storage)."""
    rng = np.random.default_rng(2024)
    shapes, dtypes = [(5,), (1,), (40,)], [np.float32, np.int32, np.uint8]

    def per_pair_continues(g, c, what):
        for step in range(6):
            assert_tree_equal(g, c, "%s step %d" % (what, step))
            assert np.float32(g.max_priority) == np.float32(c.max_priority) and g.size() == c.size
            u = rng.random(16).astype(np.float32)
            out = g.sample(0.6, uniforms=torch.from_numpy(u).cuda())
            assert_sample_equal(out, c.sample(16, 0.6, u), "%s step %d" % (what, step))
            assert_sample_equal(g.sample(0.9), c.sample(16, 0.9), "%s step %d generator" % (what, step))
            rows = random_rows(rng, 9, shapes, dtypes)
            g.insert(*to_dev(rows)), c.push(rows, 9)
            idx = rng.integers(0, c.size, 50)
            pr = (rng.pareto(1.5, 50) + 1e-6).astype(np.float32)
            g.update_priorities(torch.from_numpy(idx).cuda(), torch.from_numpy(pr).cuda()), c.update(idx, pr)
        for f, view in enumerate(g.storage()):
            assert np.array_equal(t2n(view).view(np.uint8), c.field(f).view(np.uint8)), (what, f)

    for cap in (300, 1000):  # 300: wrapped ring; 1000: partly filled
        # HIP -> oracle
        g = mrb.PER(0.6, cap, 16, shapes, torch_types(dtypes), seed0=5)
        g.insert(*to_dev(random_rows(rng, 450, shapes, dtypes)))
        g.update_priorities(torch.from_numpy(rng.integers(0, min(cap, 450), 200)).cuda(),
                            torch.from_numpy(rng.pareto(1.5, 200).astype(np.float32) + 1e-6).cuda())
        g.sample(0.4)  # advances the generator
        c = orc.OraclePER(0.6, cap, shapes, dtypes, seed=12345)
        c.load_state_dict(g.state_dict())
        per_pair_continues(g, c, "hip->oracle cap %d" % cap)
        g.destroy()
        # oracle -> HIP
        c = orc.OraclePER(0.6, cap, shapes, dtypes, seed=8)
        c.push(random_rows(rng, 450, shapes, dtypes), 450)
        c.update(rng.integers(0, min(cap, 450), 200), rng.pareto(1.5, 200).astype(np.float32) + 1e-6)
        c.sample(16, 0.4)
        g = mrb.PER(0.6, cap, 16, shapes, torch_types(dtypes), seed0=999)
        g.load_state_dict(c.state_dict())
        per_pair_continues(g, c, "oracle->hip cap %d" % cap)
        with pytest.raises(ValueError):  # leaves are priorities ** alpha: another alpha must be refused
            mrb.PER(0.5, cap, 16, shapes, torch_types(dtypes)).load_state_dict(c.state_dict())
        g.destroy()

    # uniform ring, wrapped, both ways
    u = mrb.URB(8, 50, shapes, torch_types(dtypes), seed=3)
    u.insert(to_dev(random_rows(rng, 70, shapes, dtypes)))
    u.sample()
    cu = orc.OracleUniform(50, shapes, dtypes, seed=77)
    cu.load_state_dict(u.state_dict())
    cw = orc.OracleUniform(50, shapes, dtypes, seed=4)
    cw.append(random_rows(rng, 85, shapes, dtypes), 85)
    cw.sample(8)
    w = mrb.URB(8, 50, shapes, torch_types(dtypes), seed=5)
    w.load_state_dict(cw.state_dict())
    for gb, cb in ((u, cu), (w, cw)):
        for step in range(4):
            assert (int(gb.count), int(gb.head)) == (cb.count, cb.head)
            gi, gf = gb.sample_with_indices()
            ci, cf = cb.sample(8)
            assert np.array_equal(t2n(gi), ci)
            for a, b in zip(gf, cf):
                assert np.array_equal(t2n(a).view(np.uint8), b.view(np.uint8))
            rows = random_rows(rng, 13, shapes, dtypes)
            gb.insert(to_dev(rows)), cb.append(rows, 13)
            for a, b in zip(gb.get_item(-1), cb.get_item(-1)):
                assert np.array_equal(t2n(a).view(np.uint8), b.view(np.uint8))
        for f in range(len(shapes)):
            assert np.array_equal(t2n(gb.buffer[f]).view(np.uint8), cb.field(f).view(np.uint8))
        gb.destroy()

    # reservoir past its capacity, both ways
    r = mrb.RES(20, 8, shapes, torch_types(dtypes), seed1=6)
    r.push(*to_dev(random_rows(rng, 90, shapes, dtypes)))
    r.sample()
    cr = orc.OracleReservoir(20, shapes, dtypes, seed=1)
    cr.load_state_dict(r.state_dict())
    cq = orc.OracleReservoir(20, shapes, dtypes, seed=9)
    cq.push(random_rows(rng, 75, shapes, dtypes), 75)
    cq.sample(8)
    q = mrb.RES(20, 8, shapes, torch_types(dtypes), seed1=7)
    q.load_state_dict(cq.state_dict())
    for gb, cb in ((r, cr), (q, cq)):
        for step in range(4):
            rows = random_rows(rng, 40, shapes, dtypes)
            gb.push(*to_dev(rows)), cb.push(rows, 40)
            gi, gf = gb.sample(with_indices=True)
            ci, cf = cb.sample(8)
            assert np.array_equal(t2n(gi), ci)
            for a, b in zip(gf, cf):
                assert np.array_equal(t2n(a).view(np.uint8), b.view(np.uint8))
        for f, view in enumerate(gb.storage()):
            assert np.array_equal(t2n(view).view(np.uint8), cb.field(f).view(np.uint8))
        gb.destroy()


def test_zero_priority_gives_zero_weights_not_infinite_ones(mrb, orc):
    """A leaf updated to priority 0 makes the tree minimum 0: (0 / total * size)^-beta is +inf as with
    pow(), so every importance weight becomes 0 - on the oracle and on the GPU alike - and nothing is flagged."""
    shapes, dtypes = [(2,)], [np.float32]
    g, c = make_pair(mrb, orc, 0.6, 64, 8, seed=3, shapes=shapes, dtypes=dtypes)
    rng = np.random.default_rng(5)
    rows = random_rows(rng, 64, shapes, dtypes)
    g.insert(*to_dev(rows)), c.push(rows, 64)
    idx, pr = np.array([7, 30]), np.array([0.0, 2.5], np.float32)
    g.update_priorities(torch.from_numpy(idx).cuda(), torch.from_numpy(pr).cuda()), c.update(idx, pr)
    u = rng.random(8).astype(np.float32)
    for path in (1, 2):
        g.set_option("sample_path", path)
        gi, gw = g.sample(0.4, uniforms=torch.from_numpy(u).cuda())[:2]
        ci, cw, _ = c.sample(8, 0.4, u)
        assert np.array_equal(t2n(gi), ci) and 7 not in ci
        assert np.array_equal(bits(t2n(gw)), bits(cw)) and np.all(cw == 0.0)
    assert g.check() == 0
    g.destroy()


# --------------------------------------------------------- discounted return
def test_discounted_return_reference_vectors(mrb):
    """tests/st/test_discounted_return.py:39-53 on the HIP kernel."""
    from mindrl_amd.utils import DiscountedReturn
    net = DiscountedReturn(gamma=0.99)
    ret = net(torch.tensor([[1.], [1.], [1.], [1.]]), torch.tensor([[False], [False], [True], [False]]),
              torch.tensor([2.]))
    assert np.allclose(t2n(ret), np.array([[2.9701], [1.99], [1.], [2.98]], dtype=np.float32))
    ret = net(torch.tensor([1., 1., 1., 1.]), torch.tensor([False, True, False, True]), torch.tensor(2.))
    assert np.allclose(t2n(ret), np.array([1.99, 1, 1.99, 1.], dtype=np.float32))
    with pytest.raises(ValueError, match="range"):
        DiscountedReturn(gamma=1.5)


@pytest.mark.parametrize("shape", [(1, 1, 1), (5, 1, 1), (37, 3, 1), (100, 64, 5), (1000, 256, 1), (9, 1000, 17),
                                   (300, 65, 1), (257, 130, 3), (40, 70000, 1), (33, 9000, 8),
                                   # the tiled kernel's chunks of 60 steps (one, one and a step, as many as are kept
                                   # in flight, one more, ...) and grids that divide by eight (column groups are dealt
                                   # to the dies in another order then), up to the 256 workgroups of 16,384 columns
                                   (60, 512, 1), (61, 1024, 1), (120, 515, 1), (180, 1536, 1), (181, 100, 2),
                                   (240, 2048, 1), (241, 4096, 1), (59, 16384, 1), (130, 2047, 8)])
def test_discounted_return_bit_exact(mrb, orc, shape):
    from mindrl_amd.utils import DiscountedReturn
    t, b, inner = shape
    rng = np.random.default_rng(t * 7 + b)
    r = rng.normal(size=(t, b, inner)).astype(np.float32)
    d = rng.random((t, b)) < 0.05
    v = rng.normal(size=(b, inner)).astype(np.float32)
    for gamma in (0.0, 0.9, 0.99, 1.0):
        got = t2n(DiscountedReturn(gamma)(torch.from_numpy(r).cuda(), torch.from_numpy(d).cuda(),
                                          torch.from_numpy(v).cuda()))
        want = orc.discounted_return(r, d, v, gamma)
        assert got.shape == r.shape and np.array_equal(got.view(np.int32), want.view(np.int32)), gamma


def test_discounted_return_backward_matches_autograd_of_the_reference_loop(mrb):
    """need_bprop=True: gradients equal those torch's autograd gives for the reference's own loop
    (mindspore_rl/utils/discounted_return.py:84-92) evaluated with torch ops in float32."""
    from mindrl_amd.utils import DiscountedReturn
    torch.manual_seed(3)
    for t, b, inner in [(7, 1, 1), (50, 9, 1), (33, 5, 4)]:
        shape = (t, b) + ((inner,) if inner > 1 else ())
        r0 = torch.randn(shape, device="cuda")
        v0 = torch.randn(shape[1:], device="cuda")
        d = torch.rand(t, b, device="cuda") < 0.15
        w = torch.randn(shape, device="cuda")
        r1, v1 = r0.clone().requires_grad_(True), v0.clone().requires_grad_(True)
        out = DiscountedReturn(0.97, need_bprop=True)(r1, d, v1)
        (out * w).sum().backward()
        r2, v2 = r0.clone().requires_grad_(True), v0.clone().requires_grad_(True)
        last, rows = v2, [None] * t
        for step in range(t - 1, -1, -1):
            keep = (1 - d[step].float())
            keep = keep.reshape(keep.shape + (1,) * (last.dim() - keep.dim()))
            last = r2[step] + keep * 0.97 * last
            rows[step] = last
        ref = torch.stack(rows)
        (ref * w).sum().backward()
        assert torch.allclose(out, ref, rtol=1e-6, atol=1e-6)
        assert torch.allclose(r1.grad, r2.grad, rtol=1e-5, atol=1e-6)
        assert torch.allclose(v1.grad, v2.grad, rtol=1e-5, atol=1e-6)
    # without need_bprop the result carries no graph
    assert not DiscountedReturn(0.97)(r0.clone().requires_grad_(True), d, v0).requires_grad


# -------------------------------------------------------------- n-step buffer
class OracleNStep:
    """The reference's NStepBuffer, line for line, over two oracle ring buffers
    (mindspore_rl/utils/n_step_buffer.py:51-103)."""

    def __init__(self, orc, shapes, dtypes, td_step, buffer_size):
        self.buffer = orc.OracleUniform(buffer_size, shapes, dtypes)
        self.td_data = orc.OracleUniform(td_step, shapes, dtypes)
        self.td = td_step

    def push(self, rows):
        self.buffer.append(rows, 1)

    def get_data(self):
        check = self.buffer.count > self.td
        m = 0
        while m < self.td and check:
            keep = self.buffer.get_item(self.buffer.count - self.td + m)
            self.td_data.append([k[None] for k in keep], 1)
            m += 1
        return check

    def clear(self):
        self.buffer.reset()
        self.td_data.reset()


@pytest.mark.parametrize("td,size", [(1, 5), (3, 10), (5, 6), (4, 64)])
def test_n_step_buffer_matches_reference_loop(mrb, orc, td, size):
    from mindrl_amd.utils import NStepBuffer
    shapes, dtypes = [(4,), (1,)], [np.float32, np.int32]
    rng = np.random.default_rng(td * 100 + size)
    g = NStepBuffer(shapes, torch_types(dtypes), td, buffer_size=size)
    c = OracleNStep(orc, shapes, dtypes, td, size)
    for step in range(6 * size):
        rows = random_rows(rng, 1, shapes, dtypes)
        assert g.push([torch.from_numpy(r[0]).cuda() for r in rows]) is True
        c.push(rows)
        if step % 3 == 0:
            check, data = g.get_data()
            assert bool(check[0]) == c.get_data() and tuple(check.shape) == (1,)
            for f, view in enumerate(data):
                assert np.array_equal(t2n(view).view(np.uint8), c.td_data.field(f).view(np.uint8)), (step, f)
            assert int(g.td_data.count) == c.td_data.count and int(g.td_data.head) == c.td_data.head
        assert int(g.size()) == c.buffer.count
        if step == 4 * size:
            g.clear()
            c.clear()
    g.destroy()


def test_create_replay_buffer_builds_working_buffers(mrb):
    from mindrl_amd.core import create_replay_buffer
    cfg = {"number": 2, "type": mrb.URB, "capacity": 50, "sample_size": 4,
           "data_shape": [(4,), (1,)], "data_type": ["float32", "int32"]}
    bufs = create_replay_buffer(cfg)
    assert len(bufs) == 2
    bufs[0].insert([torch.ones(8, 4).cuda(), torch.arange(8, dtype=torch.int32).reshape(8, 1).cuda()])
    assert int(bufs[0].count) == 8 and int(bufs[1].count) == 0 and tuple(bufs[0].sample()[0].shape) == (4, 4)
    for b in bufs:
        b.destroy()


# ---------------------------------------------------------------- reservoir
@pytest.mark.parametrize("cap", [1, 10, 100, 5000])
def test_reservoir_random_pushes_bit_exact(mrb, orc, cap):
    """Batched and single pushes well past the capacity; storage compared slot by slot, then samples."""
    shapes, dtypes = [(17,), (6,), (1,)], [np.float32, np.int32, np.bool_]
    rng = np.random.default_rng(cap)
    g = mrb.RES(cap, 64, shapes, torch_types(dtypes), seed0=0, seed1=42)
    c = orc.OracleReservoir(cap, shapes, dtypes, seed=42)
    for step in range(30):
        n = 1 if step % 4 == 0 else int(rng.integers(1, 3 * cap + 5))
        rows = random_rows(rng, n, shapes, dtypes)
        g.push(*to_dev(rows)) if n > 1 else g.push(*[torch.from_numpy(r[0]).cuda() for r in rows])
        c.push(rows, n)
        assert (g.size(), g.total()) == (c.size, c.total)
        for f, view in enumerate(g.storage()):
            assert np.array_equal(t2n(view).view(np.uint8), c.field(f).view(np.uint8)), (step, f)
        gi, gf = g.sample(with_indices=True)
        ci, cf = c.sample(64)
        assert np.array_equal(t2n(gi), ci)
        for a, b in zip(gf, cf):
            assert np.array_equal(t2n(a).view(np.uint8), b.view(np.uint8))
    g.destroy()


def test_reservoir_reference_scenario(mrb):
    """tests/st/test_reservoir_replay_buffer.py:33-54 on the HIP buffer."""
    prb = mrb.RES(100, 256, ((17,), (6,)), (torch.float32, torch.int32), seed0=0, seed1=42)
    for i in range(100):
        prb.push(torch.ones(17) * i, (torch.ones(6) * i).to(torch.int32))
    states, actions = prb.sample()
    states, actions = t2n(states), t2n(actions)
    assert states.shape == (256, 17) and actions.shape == (256, 6)
    assert np.allclose(states, states[:, 0:1]) and np.allclose(actions, actions[:, 0:1])
    assert np.allclose(states[:, 0], actions[:, 0])
    h = prb.destroy()
    assert h.dtype == torch.int64 and tuple(h.shape) == (1,)
    with pytest.raises(ValueError):
        mrb.RES(4, 2, [(1,)], [torch.int32], seed0=1).sample()  # empty


# ---------------------------------------------------------------------- PER
PER_SHAPES = [(3,), (1,)]
PER_DTYPES = [np.float32, np.int32]


def id_rows(n, start=0):
    ids = np.arange(start, start + n)
    return [np.repeat(ids[:, None], 3, 1).astype(np.float32), ids.astype(np.int32)[:, None]]


def make_pair(mrb, orc, alpha, cap, batch, seed=9, shapes=PER_SHAPES, dtypes=PER_DTYPES):
    g = mrb.PER(alpha, cap, batch, shapes, torch_types(dtypes), seed0=seed)
    c = orc.OraclePER(alpha, cap, shapes, dtypes, seed=seed)
    return g, c


@pytest.mark.parametrize("fused", [1, 0])
@pytest.mark.parametrize("path", [1, 2])
@pytest.mark.parametrize("cap", [1, 2, 5, 100, 200, 4096, 5000, 10000, 70000, 300000])
def test_per_random_ops_bit_exact(mrb, orc, cap, path, fused):
    """Random pushes (plain / with priorities / larger than capacity), updates with
    duplicates and samples; after every step both trees, indices, rows, size, head and
    running max are compared. Capacities cover tree depths 0..17, i.e. the top kernel
    alone (<= 4096 leaves) and one rebuild round."""
    rng = np.random.default_rng(cap + path)
    batch = 32
    g, c = make_pair(mrb, orc, 0.6, cap, batch)
    g.set_option("sample_path", path)
    g.set_option("fused_rebuild", fused)  # small updates and pushes in one launch, or a launch per round
    serial, exact_w = 0, 0
    for step in range(12):
        n = int(rng.integers(1, min(2 * cap + 3, 3000)))
        if step % 4 == 1:
            n = int(rng.integers(1, 40))  # a push of a few rows
        rows = id_rows(n, serial)
        serial += n
        if step % 3 == 2:
            pr = (np.abs(rng.normal(size=n)) + 1e-6).astype(np.float32)
            g.insert(*to_dev(rows), priorities=torch.from_numpy(pr).cuda())
            c.push(rows, n, pr)
        else:
            g.insert(*to_dev(rows))
            c.push(rows, n)
        k = int(rng.integers(1, min(2 * cap + 2, 2500)))
        if step % 2 == 0:
            k = int(rng.integers(1, 1025))  # few enough entries for the launch driven by entries
        idx = rng.integers(0, cap, k)
        if step % 3 == 0:
            idx[: k // 2] = idx[0] // 256 * 256 + rng.integers(0, 256, k // 2)  # many entries in one leaf tile
            idx = np.minimum(idx, cap - 1)
        pr = rng.pareto(1.5, k).astype(np.float32) + np.float32(1e-6)
        g.update_priorities(torch.from_numpy(idx).cuda(), torch.from_numpy(pr).cuda())
        c.update(idx, pr)
        assert_tree_equal(g, c, "cap %d step %d" % (cap, step))
        assert g.size() == c.size and g._state()[1] == c.head
        assert np.float32(g.max_priority) == np.float32(c.max_priority)
        u = rng.random(batch).astype(np.float32)
        beta = float(rng.uniform(0, 1))
        exact_w += assert_sample_equal(g.sample(beta, uniforms=torch.from_numpy(u).cuda()), c.sample(batch, beta, u),
                                       "cap %d step %d" % (cap, step))
        # generator-driven draw: both sides advance the same counter-based stream
        exact_w += assert_sample_equal(g.sample(beta), c.sample(batch, beta), "cap %d step %d rng" % (cap, step))
        for f, (a, b) in enumerate(zip(g.storage(), [c.field(0), c.field(1)])):
            assert np.array_equal(t2n(a).view(np.uint8), b.view(np.uint8)), (step, f)
    assert g.check() in (0, 8)
    assert exact_w == 24, "importance weights not bit-identical in %d of 24 draws" % (24 - exact_w)
    g.destroy()


@pytest.mark.parametrize("alpha", [0.0, 0.4, 0.6, 1.0, 1.7])
def test_device_powf_bit_exact(mrb, orc, alpha):
    """priorities ** alpha computed on the device equals the oracle's deterministic powf bit for bit."""
    n = 1 << 16
    rng = np.random.default_rng(int(alpha * 10))
    pr = np.exp(rng.uniform(-60, 40, n)).astype(np.float32)
    pr[:8] = [0.0, 1.0, 1e-38, 1e-45, 3e38, 2.0, 0.5, 1e-7]
    g = mrb.PER(alpha, n, 4, [(1,)], [torch.int32], seed0=1)
    g.insert(torch.zeros(n, 1, dtype=torch.int32).cuda())
    g.update_priorities(torch.arange(n).cuda(), torch.from_numpy(pr).cuda())
    s, _ = g.export_tree()
    want = orc.powf_array(pr, alpha)
    bad = np.nonzero(bits(s[n:]) != bits(want))[0]
    assert bad.size == 0, (pr[bad[:5]], s[n:][bad[:5]], want[bad[:5]])
    g.destroy()


def test_reference_scenario(mrb):
    """tests/st/test_priority_replay_buffer.py:34-66 on the HIP buffer, through the
    method names that test uses (push / sample / update_priorities)."""
    capacity, batch_size = 200, 32
    prb = mrb.PER(1., capacity, batch_size, ((17,), (6,)), (torch.float32, torch.int32), seed0=0, seed1=42)
    for i in range(100):
        prb.push(torch.ones(17) * i, (torch.ones(6) * i).to(torch.int32))
    indices, weights, states, actions = prb.sample(1.)
    ind = t2n(indices)
    assert np.all(ind < 100) and weights.shape == (32,) and weights.dtype == torch.float32
    assert np.allclose(t2n(states), np.broadcast_to(ind.reshape(-1, 1), states.shape))
    assert np.allclose(t2n(actions), np.broadcast_to(ind.reshape(-1, 1), actions.shape))
    prb.update_priorities(indices, torch.ones(32) * 1e-7)
    indices_new, _, states_new, actions_new = prb.sample(1.)
    ind2 = t2n(indices_new)
    assert np.all(ind2 < 100) and np.all(ind != ind2)
    assert np.allclose(t2n(states_new), np.broadcast_to(ind2.reshape(-1, 1), states_new.shape))
    assert np.allclose(t2n(actions_new), np.broadcast_to(ind2.reshape(-1, 1), actions_new.shape))
    assert bool(prb.full()) is False
    with pytest.raises(ValueError):
        prb.reset()
    h = prb.destroy()
    assert h.dtype == torch.int64 and tuple(h.shape) == (1,)


@pytest.mark.parametrize("cap", [10_000, 300_000, 5_000_000])
@pytest.mark.parametrize("n", [40, 300, 700, 2000])
def test_updates_with_invalid_entries_among_many(mrb, orc, cap, n):
    """Invalid entries (index outside the ring; negative, NaN or infinite priority) inside calls of 40 .. 2000
    entries - one wave per entry, two waves per entry, the stamp pass and, on the 23-level tree, the
    entry-driven lowest round - are skipped and flagged while every valid entry lands as if the invalid ones
    were not there: also where the LAST entry aimed at a leaf is the invalid one (the valid one before it
    wins) and where an invalid entry shares its tile with valid ones."""
    rng = np.random.default_rng(7000 + n + cap % 97)
    shapes, dtypes = [(1,)], [np.int32]
    g = mrb.PER(0.6, cap, 16, shapes, torch_types(dtypes), seed0=5)
    c = orc.OraclePER(0.6, cap, shapes, dtypes, seed=5)
    for start in range(0, cap, 1 << 18):
        m = min(1 << 18, cap - start)
        rows = [np.zeros((m, 1), np.int32)]
        g.insert(*to_dev(rows))
        c.push(rows, m)
    for rep in range(3):
        idx = rng.integers(0, cap, n)
        idx[n // 2:] = np.minimum(idx[n // 2] // 256 * 256 + rng.integers(0, 256, n - n // 2), cap - 1)  # one crowded tile
        pr = (rng.pareto(1.5, n) + 1e-6).astype(np.float32)
        bad_idx = rng.choice(n, max(2, n // 10), replace=False)
        idx[bad_idx[0::2]] = cap + rng.integers(0, 1000, len(bad_idx[0::2]))
        idx[bad_idx[1::2]] = -1 - rng.integers(0, 1000, len(bad_idx[1::2]))
        bad_pr = rng.choice(n, max(3, n // 10), replace=False)
        pr[bad_pr] = np.resize(np.array([-1.0, np.nan, np.inf], np.float32), len(bad_pr))
        # a leaf whose last entry is invalid: the valid entry before it must win
        idx[n - 1] = idx[1] = int(rng.integers(0, cap))
        pr[1], pr[n - 1] = 3.25, np.nan
        ok = (idx >= 0) & (idx < cap) & np.isfinite(pr) & (pr >= 0)
        assert ok[1] and not ok[n - 1] and ok.sum() < n
        g.update_priorities(torch.from_numpy(idx).cuda(), torch.from_numpy(pr).cuda())
        c.update(idx[ok], pr[ok])
        flags = C.c_uint32(0)
        assert mrb.lib.lib().mrb_per_check(g._h, C.byref(flags), None) == 0
        assert flags.value & mrb.lib.DERR_INDEX and flags.value & mrb.lib.DERR_PRIORITY, flags.value
        assert_tree_equal(g, c, "cap %d n %d rep %d" % (cap, n, rep))
        assert np.float32(g.max_priority) == np.float32(c.max_priority)
        u = rng.random(16).astype(np.float32)
        assert_sample_equal(g.sample(0.5, uniforms=torch.from_numpy(u).cuda()), c.sample(16, 0.5, u), "after rep %d" % rep)
    g.destroy()


@pytest.mark.parametrize("cap", [4, 37, 1000, 2048, 4096, 5000, 10_000, 16_384])
def test_updates_of_a_few_hundred_entries_on_small_trees(mrb, orc, cap):
    """update_priorities of 1 .. 384 entries on trees of 2 .. 14 levels (one launch of one workgroup that walks
    the entries' paths: the tree's top in LDS, the nodes below it in LDS hash tables, two levels per step): random
    indices, consecutive slots (neighbouring paths meet at every level), a handful of leaves hit by every entry
    (the latest entry wins each) and invalid entries among valid ones - trees, running max and flags as the
    oracle's after every call; with the one-launch option off the same calls give the same bits."""
    rng = np.random.default_rng(8100 + cap)
    shapes, dtypes = [(2,)], [np.float32]
    g = mrb.PER(0.7, cap, 8, shapes, torch_types(dtypes), seed0=3)
    g2 = mrb.PER(0.7, cap, 8, shapes, torch_types(dtypes), seed0=3)
    g2.set_option("fused_rebuild", 0)
    c = orc.OraclePER(0.7, cap, shapes, dtypes, seed=3)
    fill = cap - cap // 5  # some leaves stay unfilled: their minimum is FLT_MAX until an update reaches them
    rows = [rng.normal(size=(fill, 2)).astype(np.float32)]
    g.insert(*to_dev(rows))
    g2.insert(*to_dev(rows))
    c.push(rows, fill)
    for n in (1, 2, 17, 64, 65, 100, 128, 255, 256, 321, 384):
        for mode in ("random", "consecutive", "crowded", "invalid"):
            if mode == "invalid" and n < 17:
                continue
            if mode == "random":
                idx = rng.integers(0, cap, n)
            elif mode == "consecutive":
                idx = (rng.integers(0, cap) + np.arange(n)) % cap
            elif mode == "crowded":
                idx = rng.integers(0, min(cap, 7), n) + rng.integers(0, max(1, cap - 7))
            else:
                idx = rng.integers(0, cap, n)
                idx[rng.choice(n, 5, replace=False)] = cap + rng.integers(0, 100, 5)
                idx[rng.choice(n, 3, replace=False)] = -1 - rng.integers(0, 100, 3)
            pr = (rng.pareto(1.5, n) + 1e-6).astype(np.float32)
            if mode == "invalid":
                pr[rng.choice(n, 6, replace=False)] = np.array([-1.0, np.nan, np.inf, -np.inf, -0.5, np.nan], np.float32)
                idx[n - 1] = idx[2] = int(rng.integers(0, cap))  # the last entry aimed at a leaf is invalid:
                pr[2], pr[n - 1] = 1.75, np.nan                   # the valid one before it wins
            ok = (idx >= 0) & (idx < cap) & np.isfinite(pr) & (pr >= 0)
            for buf in (g, g2):
                buf.update_priorities(torch.from_numpy(idx).cuda(), torch.from_numpy(pr).cuda())
            c.update(idx[ok], pr[ok])
            what = "cap %d n %d %s" % (cap, n, mode)
            for buf in (g, g2):
                flags = C.c_uint32(0)
                assert mrb.lib.lib().mrb_per_check(buf._h, C.byref(flags), None) == 0
                want = (mrb.lib.DERR_INDEX | mrb.lib.DERR_PRIORITY) if mode == "invalid" else 0
                assert flags.value == want, (what, flags.value)
                assert_tree_equal(buf, c, what)
                assert bits(np.float32(buf.max_priority)) == bits(np.float32(c.max_priority)), what
    u = rng.random(8).astype(np.float32)
    assert_sample_equal(g.sample(0.5, uniforms=torch.from_numpy(u).cuda()), c.sample(8, 0.5, u), "cap %d" % cap)
    g.destroy()
    g2.destroy()


def test_per_error_paths(mrb):
    L = mrb.lib.lib()
    assert L.mrb_backend() == 1
    g = mrb.PER(0.6, 16, 4, [(1,)], [torch.int32], seed0=3)
    with pytest.raises(ValueError):
        g.sample(0.4)  # empty
    g.insert(torch.zeros(16, 1, dtype=torch.int32).cuda())
    g.update_priorities(torch.tensor([3, 99, -1]).cuda(), torch.tensor([2.0, 1.0, 1.0]).cuda())
    with pytest.raises(IndexError):
        g.check()
    g.update_priorities(torch.tensor([3, 4, 5]).cuda(), torch.tensor([-2.0, float("nan"), float("inf")]).cuda())
    with pytest.raises(ValueError):
        g.check()
    s, _ = g.export_tree()
    assert abs(s[16 + 3] - 2.0 ** 0.6) < 1e-6
    assert s[16 + 4] == 1.0 and s[16 + 5] == 1.0  # invalid entries skipped
    assert L.mrb_per_update(C.c_int64(987654), None, None, 1, None) == mrb.lib.MRB_EHANDLE
    assert L.mrb_per_update(C.c_int64(g._h), None, None, 1, None) == mrb.lib.MRB_EINVAL
    assert b"NULL" in L.mrb_last_error()
    g.destroy()
    with pytest.raises(ValueError):
        g.size()
    with pytest.raises(ValueError):
        mrb.PER(0.6, -5, 4, [(1,)], [torch.int32])


@pytest.mark.parametrize("seed", range(12))
def test_randomised_differential(mrb, orc, seed):
    """Random buffer shapes, capacities (trees of 0..18 levels), alphas and operation mixes,
    the HIP buffer and the oracle fed the same calls; everything observable compared after each."""
    rng = np.random.default_rng(9000 + seed)
    cap = int(rng.choice([1, 2, 3, 7, 64, 65, 1000, 4097, 9999, 40000, 150000]))
    nf = int(rng.integers(1, 5))
    pool = [((1,), np.uint8), ((3,), np.int16), ((2, 2), np.float32), ((5,), np.float64), ((64,), np.float32),
            ((300,), np.uint8), ((1,), np.bool_), ((1,), np.int64)]
    picks = [pool[i] for i in rng.integers(0, len(pool), nf)]
    shapes, dtypes = [p[0] for p in picks], [p[1] for p in picks]
    alpha = float(rng.choice([0.0, 0.3, 0.6, 1.0]))
    batch = int(rng.choice([1, 5, 64, 300]))
    path, split = int(rng.integers(0, 3)), int(rng.choice([0, 0, 1, 3]))
    g, c = make_pair(mrb, orc, alpha, cap, batch, seed=seed + 1, shapes=shapes, dtypes=dtypes)
    g.set_option("sample_path", path)
    g.set_option("row_split", split)
    for step in range(25):
        op = rng.integers(0, 4) if c.size else 0
        if op == 0:
            n = int(rng.integers(1, min(2 * cap + 2, 5000)))
            rows = random_rows(rng, n, shapes, dtypes)
            if rng.random() < 0.4:
                pr = (rng.pareto(1.2, n) + 1e-6).astype(np.float32)
                g.insert(*to_dev(rows), priorities=torch.from_numpy(pr).cuda())
                c.push(rows, n, pr)
            else:
                g.insert(*to_dev(rows))
                c.push(rows, n)
        elif op == 1:
            n = int(rng.integers(1, min(3 * cap + 2, 6000)))
            idx = rng.integers(0, cap, n)
            pr = np.where(rng.random(n) < 0.05, 0.0, rng.lognormal(0, 2, n)).astype(np.float32)
            g.update_priorities(torch.from_numpy(idx).cuda(), torch.from_numpy(pr).cuda())
            c.update(idx, pr)
        elif c.export_tree()[0][1] > 0:
            beta = float(rng.uniform(0, 1))
            if op == 2:
                u = rng.random(batch).astype(np.float32)
                assert_sample_equal(g.sample(beta, uniforms=torch.from_numpy(u).cuda()), c.sample(batch, beta, u),
                                    "seed %d step %d" % (seed, step))
            else:
                assert_sample_equal(g.sample(beta), c.sample(batch, beta), "seed %d step %d rng" % (seed, step))
        assert_tree_equal(g, c, "seed %d step %d" % (seed, step))
        assert g.size() == c.size and np.float32(g.max_priority) == np.float32(c.max_priority)
    for f, view in enumerate(g.storage()):
        assert np.array_equal(t2n(view).view(np.uint8), c.field(f).view(np.uint8)), f
    g.check()
    g.destroy()


@pytest.mark.parametrize("path", [1, 2])
def test_sixteen_fields_of_odd_sizes(mrb, orc, path, sizes=(1, 2, 3, 4, 6, 8, 12, 16, 20, 24, 48, 100, 1000, 4096, 4100, 7)):
    """The maximum of 16 fields, row sizes 1..4100 bytes covering every copy granule (1, 2, 4, 8,
    16 bytes) and rows that need several passes per workgroup; all three buffer kinds."""
    sizes = list(sizes)
    shapes, dtypes = [(n,) for n in sizes], [np.uint8] * len(sizes)
    shapes[7], dtypes[7] = (4,), np.float32   # 16 bytes
    shapes[9], dtypes[9] = (3,), np.int64     # 24 bytes
    rng = np.random.default_rng(16)
    cap, batch = 300, 40
    g, c = make_pair(mrb, orc, 0.7, cap, batch, seed=2, shapes=shapes, dtypes=dtypes)
    g.set_option("sample_path", path)
    u = mrb.URB(batch, cap, shapes, torch_types(dtypes), seed=8)
    cu = orc.OracleUniform(cap, shapes, dtypes, seed=8)
    r = mrb.RES(cap, batch, shapes, torch_types(dtypes), seed1=8)
    cr = orc.OracleReservoir(cap, shapes, dtypes, seed=8)
    for step in range(6):
        n = int(rng.integers(1, 250))
        rows = random_rows(rng, n, shapes, dtypes)
        dev = to_dev(rows)
        g.insert(*dev), c.push(rows, n)
        u.insert(dev), cu.append(rows, n)
        r.push(*dev), cr.push(rows, n)
        draws = rng.random(batch).astype(np.float32)
        assert_sample_equal(g.sample(0.5, uniforms=torch.from_numpy(draws).cuda()), c.sample(batch, 0.5, draws),
                            "step %d" % step)
        ui, uf = u.sample_with_indices()
        ci, cf = cu.sample(batch)
        assert np.array_equal(t2n(ui), ci)
        ri, rf = r.sample(with_indices=True)
        ki, kf = cr.sample(batch)
        assert np.array_equal(t2n(ri), ki)
        for f in range(len(sizes)):
            assert np.array_equal(t2n(uf[f]).view(np.uint8), cf[f].view(np.uint8)), (step, f)
            assert np.array_equal(t2n(rf[f]).view(np.uint8), kf[f].view(np.uint8)), (step, f)
            assert np.array_equal(t2n(u.buffer[f]).view(np.uint8), cu.field(f).view(np.uint8)), (step, f)
    for b in (g, u, r):
        b.destroy()


@pytest.mark.parametrize("path", [1, 2])
def test_out_of_domain_inputs_are_clamped_and_flagged(mrb, orc, path):
    """Draws outside [0, 1), NaN draws, and slots far outside the buffer: the oracle defines what comes
    back (the descent has no clamp), the row copies stay inside the storage, and flags are raised."""
    shapes, dtypes = [(600,), (1,)], [np.float32, np.int32]  # one wide and one narrow field
    rng = np.random.default_rng(4)
    cap = 1500
    g, c = make_pair(mrb, orc, 0.6, cap, 8, seed=5, shapes=shapes, dtypes=dtypes)
    g.set_option("sample_path", path)
    rows = random_rows(rng, cap, shapes, dtypes)
    g.insert(*to_dev(rows)), c.push(rows, cap)
    u = np.array([0.0, 0.999, 1.0, 7.5, -3.0, np.nan, np.inf, 1e30], np.float32)
    assert_sample_equal(g.sample(0.5, uniforms=torch.from_numpy(u).cuda()), c.sample(8, 0.5, u), "odd draws")
    assert g.check() & 8  # the descent ended past the filled leaves at least once
    wild = torch.tensor([0, cap - 1, cap, 10 ** 12, -1, -2 ** 62, 2 ** 62, 5], dtype=torch.int64).cuda()
    got = g.gather(wild)
    want = np.clip(t2n(wild), 0, cap - 1)
    assert np.array_equal(t2n(got[1])[:, 0], c.field(1)[want, 0])
    assert np.array_equal(t2n(got[0]), c.field(0)[want])
    with pytest.raises(IndexError):
        g.check()
    g.destroy()


def test_gather_of_more_granules_than_one_grid_row_holds(mrb):
    """A gather of narrow rows whose widest field needs more workgroups than a launch's row of them may have
    (16,384 x 256 threads, a thread per 16-byte granule): the threads go round more than once; fields of other
    sizes end earlier. Checked against torch's own indexing of the storage."""
    from mindrl_amd.core import PriorityReplayBuffer
    cap, n = 3000, 170_000
    shapes, types = [(120,), (1,), (3,)], [torch.float32, torch.int32, torch.uint8]  # 30 granules, one, three bytes
    g = PriorityReplayBuffer(0.6, cap, 4, shapes, types, seed0=1)
    gen = torch.Generator(device="cuda").manual_seed(5)
    rows = [torch.randn(cap, 120, device="cuda", generator=gen), torch.arange(cap, dtype=torch.int32, device="cuda")[:, None],
            torch.randint(0, 255, (cap, 3), dtype=torch.uint8, device="cuda", generator=gen)]
    g.insert(*rows)
    idx = torch.randint(0, cap, (n,), device="cuda", generator=gen)
    got = g.gather(idx)
    for f in range(3):
        assert torch.equal(got[f], rows[f][idx]), f
    g.check()
    g.destroy()


# ----------------------------------------------- the five benchmark configurations
def test_config1_dqn_per_cartpole_full_loop(mrb, orc):
    """Config 1: capacity 10 000, alpha .6, beta .4, eps 1e-6; fill, then 1000 x
    {sample 64, update with |N(0,1)|+eps, insert 1}. Every step compared."""
    shapes = [(4,), (1,), (1,), (4,), (1,)]
    dtypes = [np.float32, np.int32, np.float32, np.float32, np.bool_]
    rng = np.random.default_rng(1001)
    cap, batch = 10_000, 64
    g, c = make_pair(mrb, orc, 0.6, cap, batch, seed=1001, shapes=shapes, dtypes=dtypes)

    def transitions(n):
        return [rng.uniform(-2.4, 2.4, (n, 4)).astype(np.float32), rng.integers(0, 2, (n, 1)).astype(np.int32),
                np.ones((n, 1), np.float32), rng.uniform(-2.4, 2.4, (n, 4)).astype(np.float32),
                rng.random((n, 1)) < 0.05]

    rows = transitions(cap)
    g.insert(*to_dev(rows))
    c.push(rows, cap)
    exact = 0
    for step in range(1000):
        u = rng.random(batch).astype(np.float32)
        out = g.sample(0.4, uniforms=torch.from_numpy(u).cuda())
        ref = c.sample(batch, 0.4, u)
        exact += assert_sample_equal(out, ref, "step %d" % step)
        td = (np.abs(rng.normal(size=batch)) + 1e-6).astype(np.float32)
        g.update_priorities(out[0], torch.from_numpy(td).cuda())
        c.update(ref[0], td)
        one = transitions(1)
        g.insert(*[torch.from_numpy(r[0]).cuda() for r in one])
        c.push(one, 1)
        if step % 50 == 0 or step == 999:
            assert_tree_equal(g, c, "step %d" % step)
    assert exact == 1000
    assert g.check() == 0
    g.destroy()


def test_config4_apex_high_churn(mrb, orc):
    """Config 4 at its real shape: capacity 2^21, 521-byte rows, per step insert 4096
    with actor priorities, update 2048 (~10% duplicates, Pareto(1.5)), sample 1024."""
    shapes = [(64,), (1,), (1,), (64,), (1,)]
    dtypes = [np.float32, np.int32, np.float32, np.float32, np.bool_]
    rng = np.random.default_rng(1004)
    cap, batch = 1 << 21, 1024
    g, c = make_pair(mrb, orc, 0.6, cap, batch, seed=1004, shapes=shapes, dtypes=dtypes)
    for step in range(6):
        n = 4096 if step else 65536
        rows = random_rows(rng, n, shapes, dtypes)
        pr = (np.abs(rng.normal(size=n)) + 1e-6).astype(np.float32)
        g.insert(*to_dev(rows), priorities=torch.from_numpy(pr).cuda())
        c.push(rows, n, pr)
        idx = rng.integers(0, c.size, 2048)
        idx[rng.integers(0, 2048, 205)] = idx[rng.integers(0, 2048, 205)]
        up = rng.pareto(1.5, 2048).astype(np.float32) + np.float32(1e-6)
        g.update_priorities(torch.from_numpy(idx).cuda(), torch.from_numpy(up).cuda())
        c.update(idx, up)
        u = rng.random(batch).astype(np.float32)
        for path in (1, 2):
            g.set_option("sample_path", path)
            assert_sample_equal(g.sample(0.5, uniforms=torch.from_numpy(u).cuda()), c.sample(batch, 0.5, u),
                                "step %d path %d" % (step, path))
        g.set_option("sample_path", 0)
    assert_tree_equal(g, c, "config 4")
    assert g.check() == 0
    g.destroy()


def test_config5_tree_descent_stress(mrb, orc):
    """Config 5 at full size: 2^24 leaves, 8-byte rows, heavy-tailed priorities,
    batch 65 536 stratified, update 65 536 random indices per step."""
    shapes, dtypes = [(1,), (1,)], [np.int32, np.float32]
    rng = np.random.default_rng(1005)
    cap, batch = 1 << 24, 65536
    g, c = make_pair(mrb, orc, 0.6, cap, batch, seed=1005, shapes=shapes, dtypes=dtypes)
    rows = [np.arange(cap, dtype=np.int32)[:, None], rng.normal(size=(cap, 1)).astype(np.float32)]
    pr = np.where(rng.random(cap) < 0.99, rng.uniform(0, 1e-3, cap), rng.uniform(1, 100, cap)).astype(np.float32)
    g.insert(*to_dev(rows), priorities=torch.from_numpy(pr).cuda())
    c.push(rows, cap)
    c.update(np.arange(cap), pr)
    for step in range(3):
        idx = rng.integers(0, cap, batch)
        up = np.where(rng.random(batch) < 0.99, rng.uniform(0, 1e-3, batch), rng.uniform(1, 100, batch)).astype(np.float32)
        g.update_priorities(torch.from_numpy(idx).cuda(), torch.from_numpy(up).cuda())
        c.update(idx, up)
        u = rng.random(batch).astype(np.float32)
        for path in (2, 1):
            g.set_option("sample_path", path)
            out = g.sample(0.7, uniforms=torch.from_numpy(u).cuda())
            assert_sample_equal(out, c.sample(batch, 0.7, u), "step %d path %d" % (step, path))
            assert np.array_equal(t2n(out[2])[:, 0], t2n(out[0]))  # row k holds its own slot number
        g.set_option("sample_path", 0)
    assert_tree_equal(g, c, "config 5")
    assert g.check() == 0
    g.destroy()


@pytest.mark.parametrize("cap", [3_000_000, 20_000_000])
def test_sparse_updates_on_very_large_trees(mrb, orc, cap):
    """Trees of 22 and 25 levels: updates of up to 1024 entries elect among themselves (sizes 1, 7, 1000 with
    10 % duplicates), larger ones with few entries for the tree take the entry-driven lowest round (60,000:
    groups of 4 and 8 lanes per entry)."""
    shapes, dtypes = [(1,)], [np.uint8]
    rng = np.random.default_rng(cap % 1000)
    g, c = make_pair(mrb, orc, 0.6, cap, 256, seed=3, shapes=shapes, dtypes=dtypes)
    rows = [np.zeros((cap, 1), np.uint8)]
    pr = rng.lognormal(0, 1, cap).astype(np.float32)
    g.insert(*to_dev(rows), priorities=torch.from_numpy(pr).cuda())
    c.push(rows, cap)
    c.update(np.arange(cap), pr)
    for n in (1, 1000, 60000, 7):
        idx = rng.integers(0, cap, n)
        if n >= 1000:
            idx[rng.integers(0, n, n // 10)] = idx[rng.integers(0, n, n // 10)]
        up = rng.pareto(1.5, n).astype(np.float32) + np.float32(1e-6)
        g.update_priorities(torch.from_numpy(idx).cuda(), torch.from_numpy(up).cuda())
        c.update(idx, up)
        u = rng.random(256).astype(np.float32)
        assert_sample_equal(g.sample(0.5, uniforms=torch.from_numpy(u).cuda()), c.sample(256, 0.5, u), "n %d" % n)
    assert_tree_equal(g, c, "cap %d" % cap)
    assert np.float32(g.max_priority) == np.float32(c.max_priority)
    # pushes with priorities on the full ring: 5000 rows (the leaf-level waves collect the call's largest
    # p^alpha for the top workgroup), one of them above the running max; then 300 rows
    for n in (5000, 300):
        more = [np.ones((n, 1), np.uint8)]
        mp = (rng.pareto(1.5, n) + 1e-6).astype(np.float32)
        mp[n // 2] = np.float32(c.max_priority) * 3 + 1
        g.insert(*to_dev(more), priorities=torch.from_numpy(mp).cuda())
        c.push(more, n, mp)
        assert_tree_equal(g, c, "cap %d push %d with priorities" % (cap, n))
        assert np.float32(g.max_priority) == np.float32(c.max_priority)
    # invalid entries are skipped and flagged, valid ones in the same call still land
    g.update_priorities(torch.tensor([5, cap + 3, -1, 9]).cuda(), torch.tensor([2.0, 1.0, 1.0, float("nan")]).cuda())
    c.update([5], [2.0])
    with pytest.raises(IndexError):
        g.check()
    assert_tree_equal(g, c, "cap %d after invalid entries" % cap)
    g.destroy()


@pytest.mark.parametrize("cap,obs_shape,extra", [(5000, (84, 84, 4), False), (70_000, (36, 1000), True),
                                                 (2_500_000, (1024,), False), (300, (16,), True)])
def test_sample_with_next_equals_sample_then_gather(mrb, orc, cap, obs_shape, extra):
    """mrb_per_sample_next - the sample and, in the same launch, the observation at the slot each sampled row
    names - against the oracle's sample plus numpy's take of the observations, and against mrb_per_sample followed by mrb_per_gather:
    a 28,224-byte image row, a 36,000-byte row (two workgroups per row in the second layer), a 22-level tree
    (the copy waves share the descent's top group) and 16-byte rows; with a second wide field in the row
    (`extra`) the general addressing path runs. Slot numbers outside [0, size) are clamped and flagged."""
    rng = np.random.default_rng(4400 + cap % 1000)
    shapes = [obs_shape, (1,), (1,)] + ([(8,)] if extra else [])
    dtypes = [np.uint8, np.int64, np.float32] + ([np.float32] if extra else [])
    batch = 96
    g = mrb.PER(0.6, cap, batch, shapes, torch_types(dtypes), seed0=9)
    c = orc.OraclePER(0.6, cap, shapes, dtypes, seed=9)
    fill = cap - cap // 7
    mirror = np.zeros((fill + 4,) + obs_shape, np.uint8)  # the observation field by slot (the ring does not wrap here)
    for start in range(0, fill, 50_000):
        m = min(50_000, fill - start)
        rows = [rng.integers(0, 256, (m,) + obs_shape, dtype=np.uint8),
                rng.integers(0, fill, (m, 1)).astype(np.int64), rng.normal(size=(m, 1)).astype(np.float32)]
        if extra:
            rows.append(rng.normal(size=(m, 8)).astype(np.float32))
        pr = rng.lognormal(0, 1, m).astype(np.float32)
        g.insert(*to_dev(rows), priorities=torch.from_numpy(pr).cuda())
        c.push(rows, m, pr)
        mirror[start:start + m] = rows[0]
    for rep in range(3):
        u = rng.random(batch).astype(np.float32)
        ud = torch.from_numpy(u).cuda()
        out = g.sample_with_next(0.5, 1, 0, uniforms=ud)
        ci, cw, cf = c.sample(batch, 0.5, u)
        assert_sample_equal(out[:-1], (ci, cw, cf), "sample part, rep %d" % rep)
        want = np.take(mirror, cf[1].reshape(-1), axis=0)
        assert np.array_equal(t2n(out[-1]), want), "next rows differ from numpy's take, rep %d" % rep
        two = g.sample(0.5, uniforms=ud)
        assert torch.equal(g.gather(two[3].reshape(-1))[0], out[-1])
        g.check()
    # slot numbers outside the stored rows: clamped like mrb_per_gather's, and flagged
    bad = [rng.integers(0, 256, (4,) + obs_shape, dtype=np.uint8), np.array([[-5], [fill + 4], [cap + 9], [3]], np.int64),
           np.zeros((4, 1), np.float32)] + ([np.zeros((4, 8), np.float32)] if extra else [])
    huge = np.full(4, 1e9, np.float32)  # the four rows take nearly all of the mass
    g.insert(*to_dev(bad), priorities=torch.from_numpy(huge).cuda())
    c.push(bad, 4, huge)
    mirror[fill:] = bad[0]
    u = rng.random(batch).astype(np.float32)
    out = g.sample_with_next(0.5, 1, 0, uniforms=torch.from_numpy(u).cuda())
    ci, cw, cf = c.sample(batch, 0.5, u)
    assert_sample_equal(out[:-1], (ci, cw, cf), "sample part with wild slot numbers")
    slots = cf[1].reshape(-1)
    assert ((slots < 0) | (slots >= fill + 4)).any()
    want = np.take(mirror, np.clip(slots, 0, fill + 4 - 1), axis=0)
    assert np.array_equal(t2n(out[-1]), want)
    flags = C.c_uint32(0)
    assert mrb.lib.lib().mrb_per_check(g._h, C.byref(flags), None) == 0
    assert flags.value == mrb.lib.DERR_INDEX, flags.value
    # argument checks: the slot field must be 8 bytes wide, the gathered field made of 16-byte granules
    with pytest.raises(ValueError):
        g.sample_with_next(0.5, 2, 0)
    with pytest.raises(ValueError):
        g.sample_with_next(0.5, 1, 2)
    g.destroy()


def test_tree_of_27_levels(mrb, orc):
    """Capacity 2^26 + 11 (a tree of 27 levels, 2^27 leaves: three node groups of nine levels per descent; deeper
    than the path kernels take, so small updates elect among themselves in the tile kernels): the full ring
    pushed with priorities, updates of 50, 1000 (10 % duplicates) and 200,000 entries (the entry-driven lowest
    round), a push that wraps the ring, samples through the wide-row kernel and through the LDS-top kernel -
    indices, rows, weights, both trees and the running max as the oracle's."""
    cap = (1 << 26) + 11
    shapes, dtypes = [(1,)], [np.uint8]
    rng = np.random.default_rng(2627)
    g, c = make_pair(mrb, orc, 0.5, cap, 256, seed=3, shapes=shapes, dtypes=dtypes)
    rows = [(np.arange(cap, dtype=np.int64) % 251).astype(np.uint8)[:, None]]
    pr = rng.lognormal(0, 1, cap).astype(np.float32)
    g.insert(*to_dev(rows), priorities=torch.from_numpy(pr).cuda())
    c.push(rows, cap)
    c.update(np.arange(cap), pr)
    del pr
    for n in (50, 1000, 200_000):
        idx = rng.integers(0, cap, n)
        if n >= 1000:
            idx[rng.integers(0, n, n // 10)] = idx[rng.integers(0, n, n // 10)]
        up = rng.pareto(1.5, n).astype(np.float32) + np.float32(1e-6)
        g.update_priorities(torch.from_numpy(idx).cuda(), torch.from_numpy(up).cuda())
        c.update(idx, up)
        u = rng.random(256).astype(np.float32)
        assert_sample_equal(g.sample(0.5, uniforms=torch.from_numpy(u).cuda()), c.sample(256, 0.5, u), "n %d" % n)
    more = [np.full((300, 1), 7, np.uint8)]
    g.insert(*to_dev(more))
    c.push(more, 300)
    assert_tree_equal(g, c, "27 levels")
    assert np.float32(g.max_priority) == np.float32(c.max_priority)
    g.check()
    # the same strata through the LDS-top kernel (9 levels staged, the 18 below them walked five per load)
    g.set_option("sample_path", 2)
    for beta in (0.4, 1.0):
        u = rng.random(256).astype(np.float32)
        assert_sample_equal(g.sample(beta, uniforms=torch.from_numpy(u).cuda()), c.sample(256, beta, u), "LDS-top kernel")
    g.check()
    g.destroy()


@pytest.mark.parametrize("cap", [1 << 17, 1_000_000])
def test_config3_atari_shape_properties(mrb, orc, cap):
    """Config 3's rows (u8[84,84,4] + next_idx i64 + action i32 + reward f32 + done bool =
    28 241 stored bytes), batch 512, at capacity 2^17 and at the full 10^6 (28.2 GB in HBM).
    The tree logic does not depend on row content, so indices, weights, the small fields and
    both trees are compared with an oracle that holds only the four small fields, and the
    image field is checked against torch's own index_select of the storage."""
    shapes = [(84, 84, 4), (1,), (1,), (1,), (1,)]
    dtypes = [np.uint8, np.int64, np.int32, np.float32, np.bool_]
    rng = np.random.default_rng(1003)
    batch = 512
    g = mrb.PER(0.6, cap, batch, shapes, torch_types(dtypes), seed0=1003)
    c = orc.OraclePER(0.6, cap, shapes[1:], dtypes[1:], seed=1003)
    gen = torch.Generator(device="cuda").manual_seed(1003)
    for start in range(0, cap, 4096):
        chunk = min(4096, cap - start)
        small = [np.arange(start + 1, start + chunk + 1, dtype=np.int64)[:, None] % cap,
                 rng.integers(0, 18, (chunk, 1)).astype(np.int32),
                 rng.integers(-1, 2, (chunk, 1)).astype(np.float32), rng.random((chunk, 1)) < 0.01]
        obs = torch.randint(0, 256, (chunk, 84, 84, 4), dtype=torch.uint8, device="cuda", generator=gen)
        g.insert(obs, *to_dev(small))
        c.push(small, chunk)
    pr = rng.lognormal(0, 1, cap).astype(np.float32)
    g.update_priorities(torch.arange(cap).cuda(), torch.from_numpy(pr).cuda())
    c.update(np.arange(cap), pr)
    store = g.storage()
    for step in range(8):
        beta = 0.4 + 0.6 * step / 7
        u = rng.random(batch).astype(np.float32)
        out = g.sample(beta, uniforms=torch.from_numpy(u).cuda())
        ci, cw, cf = c.sample(batch, beta, u)
        assert_sample_equal((out[0], out[1]) + tuple(out[3:]), (ci, cw, cf), "step %d" % step)
        assert torch.equal(out[2], store[0].index_select(0, out[0]))
        # dereference of the frame-shared next_obs index: rows gathered at the sampled next_idx values
        nxt = g.gather(out[3].reshape(-1))
        assert torch.equal(nxt[0], store[0].index_select(0, out[3].reshape(-1)))
        assert np.array_equal(t2n(nxt[1]), c.field(0)[cf[0].reshape(-1)])
        td = (np.abs(rng.normal(size=batch)) + 1e-6).astype(np.float32)
        g.update_priorities(out[0], torch.from_numpy(td).cuda())
        c.update(ci, td)
        four = [np.arange(4, dtype=np.int64)[:, None], rng.integers(0, 18, (4, 1)).astype(np.int32),
                rng.integers(-1, 2, (4, 1)).astype(np.float32), rng.random((4, 1)) < 0.01]
        obs4 = torch.randint(0, 256, (4, 84, 84, 4), dtype=torch.uint8, device="cuda", generator=gen)
        head = g._state()[1]
        g.insert(obs4, *to_dev(four))
        c.push(four, 4)
        assert torch.equal(store[0][head:head + 4], obs4)
    assert_tree_equal(g, c, "config 3 shape")
    assert g.check() == 0
    g.destroy()


FUZZ_LAYOUTS = [([(3,), (1,)], [np.float32, np.int32]), ([(300,), (1,), (3,)], [np.float32, np.int32, np.uint8]),
                ([(1,), (2,)], [np.int32, np.float32]),
                ([(64,), (1,), (1,), (64,), (1,)], [np.float32, np.int32, np.float32, np.float32, np.bool_])]
FUZZ_CAPS = [1, 3, 200, 257, 4096, 5000, 9000, 16384, 40000, 70000, 131072, 300000, 1 << 20, (1 << 20) + 7, 2_500_000,
             5_000_000]


@pytest.mark.parametrize("block", range(6))
def test_random_configurations_and_operation_sequences(mrb, orc, block):
    """Ten seeded random cases per block: capacity (trees of 0 to 23 levels), row layout, alpha, batch, sample
    kernel, fused or per-round rebuilds, workgroups per row, counters on the host or on the device - then a random
    sequence of pushes (with and without priorities, from 1 row to more than the capacity), updates (sizes on both
    sides of every threshold, duplicates, many entries in one leaf tile, zero priorities), samples with given
    draws, with the generator, several batches per launch. Trees, size, head, running max and every sample are
    compared with the oracle after every operation."""
    for case in range(10):
        seed = 7000 + 10 * block + case
        rng = np.random.default_rng(seed)
        cap = int(FUZZ_CAPS[rng.integers(0, len(FUZZ_CAPS))])
        shapes, dtypes = FUZZ_LAYOUTS[rng.integers(0, len(FUZZ_LAYOUTS))] if cap < 400000 else FUZZ_LAYOUTS[2]
        alpha = float(rng.choice([0.0, 0.4, 0.6, 1.0, 1.5]))
        batch = int(rng.choice([1, 8, 33, 64, 256]))
        g, c = make_pair(mrb, orc, alpha, cap, batch, seed=seed + 1, shapes=shapes, dtypes=dtypes)
        g.set_option("sample_path", int(rng.integers(0, 3)))
        g.set_option("fused_rebuild", int(rng.integers(0, 2)))
        g.set_option("row_split", int(rng.choice([0, 0, 2, 3])))
        dev = bool(rng.integers(0, 2))
        g.set_option("device_counters", int(dev))
        tag = "seed %d cap %d alpha %.1f batch %d dev %d" % (seed, cap, alpha, batch, dev)
        fill, done = int(rng.choice([cap, cap, max(1, cap // 2), max(1, cap - 5)])), 0
        while done < fill:
            n = min(fill - done, 1 << 18)
            rows = random_rows(rng, n, shapes, dtypes)
            pr = (rng.pareto(1.5, n) + 1e-6).astype(np.float32) if rng.integers(0, 2) else None
            g.insert(*to_dev(rows), priorities=torch.from_numpy(pr).cuda() if pr is not None else None)
            c.push(rows, n, pr) if pr is not None else c.push(rows, n)
            done += n
        assert_tree_equal(g, c, tag + " prefill")
        for step in range(int(rng.integers(6, 14))):
            op = int(rng.integers(0, 5))
            what = "%s step %d op %d" % (tag, step, op)
            if op == 0:
                hi = min(cap, 6000) if dev else min(2 * cap + 2, 6000)
                n = max(1, min(int(rng.choice([1, 3, int(rng.integers(1, 300)), int(rng.integers(1, hi + 1))])), hi))
                rows = random_rows(rng, n, shapes, dtypes)
                pr = None
                if rng.integers(0, 2):
                    pr = (rng.pareto(1.5, n) + 1e-6).astype(np.float32)
                    if rng.integers(0, 3) == 0:
                        pr[rng.integers(0, n)] = np.float32(c.max_priority) * 2 + 1
                g.insert(*to_dev(rows), priorities=torch.from_numpy(pr).cuda() if pr is not None else None)
                c.push(rows, n, pr) if pr is not None else c.push(rows, n)
            elif op == 1:
                hi = 1024 if dev else 3000
                n = int(rng.choice([1, 7, 16, 17, 64, int(rng.integers(1, hi + 1)), hi]))
                idx = rng.integers(0, cap, n)
                if n > 4 and rng.integers(0, 2):
                    idx[: n // 3] = idx[0]
                if n > 4 and rng.integers(0, 2):
                    idx[n // 2:] = np.minimum(idx[n // 2] // 256 * 256 + rng.integers(0, 256, n - n // 2), cap - 1)
                pr = (rng.pareto(1.5, n) + 1e-6).astype(np.float32)
                if cap > 100 and rng.integers(0, 4) == 0:
                    pr[rng.integers(0, n)] = 0.0
                g.update_priorities(torch.from_numpy(idx).cuda(), torch.from_numpy(pr).cuda()), c.update(idx, pr)
            elif op == 2:
                u, beta = rng.random(batch).astype(np.float32), float(rng.uniform(0, 1))
                assert_sample_equal(g.sample(beta, uniforms=torch.from_numpy(u).cuda()), c.sample(batch, beta, u), what)
            elif op == 3:
                beta = float(rng.uniform(0, 1))
                assert_sample_equal(g.sample(beta), c.sample(batch, beta), what)
            else:
                nb, beta = int(rng.integers(1, 5)), float(rng.uniform(0, 1))
                got = g.sample_many(nb, beta)
                for i in range(nb):
                    assert_sample_equal([x[i] for x in got], c.sample(batch, beta), what + " batch %d" % i)
            assert_tree_equal(g, c, what)
            assert g.size() == c.size and g._state()[1] == c.head, what
            assert np.float32(g.max_priority) == np.float32(c.max_priority), what
        g.destroy()


class _Foreign:
    """An array of another framework as far as this package can tell: it is no torch tensor and no numpy array,
    it only speaks DLPack (and has a shape). Its memory is a device tensor's."""

    def __init__(self, t):
        self._t = t
        self.shape = tuple(t.shape)
        self.exports = 0

    def __dlpack__(self, *args, **kwargs):
        self.exports += 1
        return self._t.__dlpack__(*args, **kwargs)

    def __dlpack_device__(self):
        return self._t.__dlpack_device__()


def test_dlpack_producers_are_taken_without_a_copy(mrb, orc):
    """insert / update_priorities / sample(uniforms=) accept objects that only speak DLPack; a device-resident
    producer of the right type is used where it lies (same address, nothing passes through the host), and the
    results equal the oracle's."""
    from mindrl_amd.core._rows import as_tensor, flat_on_device
    rng = np.random.default_rng(21)
    cap, batch, n = 1000, 32, 300
    g, c = make_pair(mrb, orc, 0.6, cap, batch, seed=3)
    rows = id_rows(n)
    dev_rows = to_dev(rows)
    foreign = [_Foreign(t) for t in dev_rows]
    for f, t in zip(foreign, dev_rows):
        seen = as_tensor(f)
        assert seen.data_ptr() == t.data_ptr() and seen.is_cuda  # shared memory, no copy
    lay = g._layout
    assert lay.batch_of(foreign) == n
    on_dev = lay.to_device(foreign, g._dev)
    assert [o.data_ptr() for o in on_dev] == [t.data_ptr() for t in dev_rows]
    g.insert(*foreign), c.push(rows, n)
    assert all(f.exports >= 1 for f in foreign)
    idx = rng.integers(0, n, 50)
    pr = (rng.pareto(1.5, 50) + 1e-6).astype(np.float32)
    d_idx, d_pr = torch.from_numpy(idx).cuda(), torch.from_numpy(pr).cuda()
    assert flat_on_device(_Foreign(d_pr), torch.float32, g._dev).data_ptr() == d_pr.data_ptr()
    g.update_priorities(_Foreign(d_idx), _Foreign(d_pr)), c.update(idx, pr)
    u = rng.random(batch).astype(np.float32)
    d_u = torch.from_numpy(u).cuda()
    assert_sample_equal(g.sample(0.5, uniforms=_Foreign(d_u)), c.sample(batch, 0.5, u), "dlpack uniforms")
    assert_tree_equal(g, c, "dlpack")
    g.destroy()


def test_large_updates_refuse_stream_capture(mrb):
    """An update of more than 1024 entries elects its entries with tags the host counts; recorded into a HIP graph
    it would replay against stale tags, so it is refused while the stream is capturing (both entry points), and
    the capture itself stays usable: a small update recorded right after it replays correctly."""
    import ctypes as C
    cap, n = 50_000, 3000
    shapes, types = [(3,), (1,)], [torch.float32, torch.int32]
    g = mrb.PER(0.6, cap, 32, shapes, types, seed0=5)
    g.insert(torch.randn(cap, 3, device="cuda"), torch.arange(cap, dtype=torch.int32, device="cuda").reshape(cap, 1))
    idx = torch.randint(0, cap, (n,), device="cuda")
    pr = torch.rand(n, device="cuda") + 0.1
    L = mrb.lib.lib()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        sp = C.c_void_p(side.cuda_stream)
        graph.capture_begin()
        assert L.mrb_per_update(g._h, idx.data_ptr(), pr.data_ptr(), n, sp) == mrb.lib.MRB_ESTATE
        assert b"1024" in L.mrb_last_error()
        assert L.mrb_per_update_noalloc(g._h, idx.data_ptr(), pr.data_ptr(), n, sp) == mrb.lib.MRB_ESTATE
        mrb.lib.check(L.mrb_per_update_noalloc(g._h, idx.data_ptr(), pr.data_ptr(), 1024, sp))  # the limit itself records
        graph.capture_end()
    torch.cuda.synchronize()
    before = g.export_tree()[0].copy()
    graph.replay()
    torch.cuda.synchronize()
    after = g.export_tree()[0]
    leaves = after.size // 2
    touched = np.unique(t2n(idx[:1024]))
    assert np.any(before[leaves + touched] != after[leaves + touched])
    mrb.lib.check(L.mrb_per_update(g._h, idx.data_ptr(), pr.data_ptr(), n, C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    assert g.check() == 0
    del graph
    g.destroy()


@pytest.mark.parametrize("cap", [1, 2, 3, 100, 3000, 10_000, 16_384, 20_000, 70_000, 300_000, 1_000_000, 2_200_000, 5_000_000])
def test_update_push_equals_update_then_push(mrb, orc, cap):
    """mrb_per_update_push against the oracle's update followed by its push, on trees of 0 to 23 levels: one
    pushed row or a few, with and without priorities for the pushed rows, duplicate, invalid and out-of-range
    entries, entries aimed at the very slots the push overwrites, across the ring's wrap; 1 to 1100 entries (the
    one-workgroup, one-wave, two-launch and two-call paths). Both trees, the running max, size, head, rows and a
    sample are compared after every call."""
    rng = np.random.default_rng(cap + 77)
    batch = 16
    g, c = make_pair(mrb, orc, 0.6, cap, batch, seed=2)
    fill = max(1, cap - 7)  # the pushes below run across the end of the ring
    chunk = 200_000
    serial = 0
    while serial < fill:
        n = min(chunk, fill - serial)
        rows = id_rows(n, serial)
        g.insert(*to_dev(rows)), c.push(rows, n)
        serial += n
    exp_flags = 0
    for step, (k, nrows) in enumerate([(1, 1), (64, 1), (17, 1), (300, 1), (512, 4), (40, 3), (1000, 7), (1100, 2),
                                       (512, 1), (64, 1), (200, 300), (5, 20), (384, 1), (65, 1), (100, 1), (128, 1), (129, 1)]):
        idx = rng.integers(0, cap, k)
        if step % 3 == 0 and k > 4:
            idx[: k // 3] = idx[0]  # duplicates: the last entry wins
        head = c.head
        if step % 2 == 1 and k > 2:
            idx[-1] = head  # the slot the push overwrites next: the push's value must win
            idx[0] = (head + nrows - 1) % cap
        pr = (rng.pareto(1.5, k) + 1e-6).astype(np.float32)
        if step % 4 == 2 and k > 8:
            pr[3] = -1.0
            idx[5] = cap + 9
            exp_flags |= 3
        if step == 6:
            pr[k // 2] = np.float32(1e6)  # a new running max that the pushed rows must take
        rows = id_rows(nrows, serial)
        serial += nrows
        ipr = None
        if step % 5 == 4:
            ipr = (np.abs(rng.normal(size=nrows)) + 1e-6).astype(np.float32)
        g.update_priorities_and_insert(torch.from_numpy(idx).cuda(), torch.from_numpy(pr).cuda(), *to_dev(rows),
                                       insert_priorities=None if ipr is None else torch.from_numpy(ipr).cuda())
        ok = (idx >= 0) & (idx < cap) & np.isfinite(pr) & (pr >= 0)  # the device skips and flags the others
        c.update(idx[ok], pr[ok])
        c.push(rows, nrows, ipr)
        what = "cap %d step %d (%d entries, %d rows)" % (cap, step, k, nrows)
        assert_tree_equal(g, c, what)
        assert g.size() == c.size and g._state()[1] == c.head, what
        assert np.float32(g.max_priority) == np.float32(c.max_priority), what
        u = rng.random(batch).astype(np.float32)
        assert_sample_equal(g.sample(0.5, uniforms=torch.from_numpy(u).cuda()), c.sample(batch, 0.5, u), what)
    for f, (a, b) in enumerate(zip(g.storage(), [c.field(0), c.field(1)])):
        assert np.array_equal(t2n(a).view(np.uint8), b.view(np.uint8)), f
    flags = C.c_uint32(0)
    assert mrb.lib.lib().mrb_per_check(g._h, C.byref(flags), None) == 0
    assert (flags.value & 3) == exp_flags, flags.value
    g.destroy()


@pytest.mark.parametrize("gen", [False, True])
@pytest.mark.parametrize("cap,batch", [(2, 2), (3, 5), (100, 64), (3000, 48), (4096, 512), (5000, 33), (10_000, 64), (16_384, 200),
                                       (16_385, 64), (70_000, 64), (10_000, 600)])
def test_update_push_sample_equals_the_three_calls(mrb, orc, cap, batch, gen):
    """mrb_per_update_push_sample against the oracle's update, push and sample, one after the other: the learner's
    step as one call, which is one launch of one workgroup on trees of 2 to 14 levels (here 1 to 14: capacities 2 to
    16,384) and the separate calls beyond (capacity 16,385 and 70,000, batches over 512, more than 384 entries, several
    rows). Duplicate, invalid and out-of-range entries, entries aimed at the slot the push overwrites, a pushed
    row that takes a new running max or a priority of its own - so large that nearly every stratum samples the
    row pushed by the same call -, across the ring's wrap, with the caller's draws and with the buffer's generator.
    Indices, weights, rows, both trees, the running max, size and head are compared after every call."""
    rng = np.random.default_rng(cap * 7 + batch + gen)
    shapes, dtypes = [(3,), (1,), (5,)], [np.float32, np.int32, np.uint8]
    g, c = make_pair(mrb, orc, 0.6, cap, batch, seed=5, shapes=shapes, dtypes=dtypes)

    def rows_of(n, start):
        ids = np.arange(start, start + n)
        return [np.repeat(ids[:, None], 3, 1).astype(np.float32), ids.astype(np.int32)[:, None],
                (ids[:, None] + np.arange(5)[None, :]).astype(np.uint8)]

    fill = max(1, cap - 5)
    rows = rows_of(fill, 0)
    g.insert(*to_dev(rows)), c.push(rows, fill)
    serial = fill
    exp_flags = 0
    for step, (k, nrows) in enumerate([(1, 1), (64, 1), (17, 1), (300, 1), (384, 1), (385, 1), (40, 3), (64, 1), (2, 1),
                                       (200, 1), (64, 1), (33, 1), (64, 2), (64, 1), (65, 1), (100, 1), (128, 1), (129, 1)]):
        idx = rng.integers(0, min(cap, serial), k)
        if step % 3 == 0 and k > 4:
            idx[: k // 3] = idx[0]  # duplicates: the last entry wins
        head = c.head
        if step % 2 == 1 and k > 2:
            idx[-1] = head  # the slot the push overwrites next: the push's value must win
        pr = (rng.pareto(1.5, k) + 1e-6).astype(np.float32)
        if step % 4 == 2 and k > 8:
            pr[3] = -1.0
            idx[5] = cap + 9
            exp_flags |= 3
        if step == 7:
            pr[k // 2] = np.float32(1e5)  # a new running max that the pushed row takes, and the sample sees
        rows = rows_of(nrows, serial)
        serial += nrows
        ipr = None
        if step % 5 == 4:
            ipr = (np.abs(rng.normal(size=nrows)) + 1e-6).astype(np.float32)
        if step == 10:
            ipr = np.full(nrows, 1e12, np.float32)  # the pushed row outweighs all the others together
        u = None if gen else rng.random(batch).astype(np.float32)
        out = None
        if k == batch:  # the sampled indices go where the update's indices come from (a loop's own buffer)
            out = (torch.from_numpy(idx).cuda(), torch.empty(batch, dtype=torch.float32, device="cuda"),
                   g._layout.empty(batch, g._dev))
        got = g.update_priorities_insert_and_sample(
            out[0] if out else torch.from_numpy(idx).cuda(), torch.from_numpy(pr).cuda(), *to_dev(rows), beta=0.4 + 0.05 * step,
            insert_priorities=None if ipr is None else torch.from_numpy(ipr).cuda(),
            uniforms=None if gen else torch.from_numpy(u).cuda(), out=out)
        ok = (idx >= 0) & (idx < cap) & np.isfinite(pr) & (pr >= 0)  # the device skips and flags the others
        c.update(idx[ok], pr[ok])
        pushed_at = c.head
        c.push(rows, nrows, ipr)
        want = c.sample(batch, 0.4 + 0.05 * step, u)
        what = "cap %d batch %d step %d (%d entries, %d rows)" % (cap, batch, step, k, nrows)
        assert_sample_equal(got, want, what)
        if step == 10 and cap > 8:
            assert np.mean(want[0] == pushed_at) > 0.5, what  # the sample did pick the row of this very call
        assert_tree_equal(g, c, what)
        assert g.size() == c.size and g._state()[1] == c.head, what
        assert np.float32(g.max_priority) == np.float32(c.max_priority), what
        if step % 4 == 3:  # the separate calls go on from the same state (the generator's counter included)
            u2 = None if gen else rng.random(batch).astype(np.float32)
            assert_sample_equal(g.sample(0.5, uniforms=None if gen else torch.from_numpy(u2).cuda()), c.sample(batch, 0.5, u2), what)
    for f, (a, b) in enumerate(zip(g.storage(), [c.field(0), c.field(1), c.field(2)])):
        assert np.array_equal(t2n(a).view(np.uint8), b.view(np.uint8)), f
    flags = C.c_uint32(0)
    assert mrb.lib.lib().mrb_per_check(g._h, C.byref(flags), None) == 0
    assert (flags.value & 3) == exp_flags, flags.value
    g.destroy()


@pytest.mark.parametrize("gen", [True, False])
@pytest.mark.parametrize("cap,batch,steps", [(3000, 48, 3), (10_000, 64, 5), (16_384, 300, 2), (100, 64, 4), (70_000, 64, 2)])
def test_hip_graph_replays_the_whole_step_with_device_counters(mrb, orc, cap, batch, steps, gen):
    """`steps` calls of mrb_per_update_push_sample, each updating the rows the call before sampled (in place: one
    index buffer), recorded ONCE into a HIP graph with device_counters and replayed 8 times: the one-workgroup kernel
    takes the ring position, the row count and the generator's call counter from the device and moves them on
    itself; the buffer fills during the replays, then the ring wraps. After every replay the last sample, both trees,
    size, head and running max equal the oracle's; eager calls in between use the same counters. (Capacity 70,000
    lies outside the one-launch kernel: the same call as its two-call fallback.)"""
    rng = np.random.default_rng(cap + batch + gen)
    shapes, dtypes = [(4,), (1,), (1,), (4,), (1,)], [np.float32, np.int32, np.float32, np.float32, np.bool_]
    g, c = make_pair(mrb, orc, 0.6, cap, batch, seed=23, shapes=shapes, dtypes=dtypes)
    fill = cap - 3 * steps - 1  # not full: the row count changes during the replays, then the ring wraps
    rows = random_rows(rng, fill, shapes, dtypes)
    pr0 = (rng.pareto(1.5, fill) + 1e-6).astype(np.float32)
    g.insert(*to_dev(rows), priorities=torch.from_numpy(pr0).cuda()), c.push(rows, fill, pr0)
    g.set_option("device_counters", 1)
    new_rows = [[torch.zeros((1,) + tuple(s), dtype=t).cuda() for s, t in zip(shapes, torch_types(dtypes))] for _ in range(steps)]
    pr_dev = torch.ones((steps, batch), dtype=torch.float32, device="cuda")
    u_dev = torch.zeros((steps, batch), dtype=torch.float32, device="cuda")
    out = (torch.empty(batch, dtype=torch.int64, device="cuda"), torch.empty(batch, dtype=torch.float32, device="cuda"),
           g._layout.empty(batch, g._dev))
    first = rng.integers(0, fill, batch)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        graph.capture_begin()
        for k in range(steps):
            g.update_priorities_insert_and_sample(out[0], pr_dev[k], *new_rows[k], beta=0.5, uniforms=None if gen else u_dev[k], out=out)
        graph.capture_end()
    torch.cuda.synchronize()
    prev = first
    for rep in range(8):
        fresh = [random_rows(rng, 1, shapes, dtypes) for _ in range(steps)]
        pr = (rng.pareto(1.5, (steps, batch)) + 1e-6).astype(np.float32)
        u = rng.random((steps, batch)).astype(np.float32)
        for k in range(steps):
            for dst, src in zip(new_rows[k], fresh[k]):
                dst.copy_(torch.from_numpy(src))
        pr_dev.copy_(torch.from_numpy(pr))
        u_dev.copy_(torch.from_numpy(u))
        out[0].copy_(torch.from_numpy(prev))
        graph.replay()
        torch.cuda.synchronize()
        for k in range(steps):
            ok = (prev >= 0) & (prev < cap)
            c.update(prev[ok], pr[k][ok])
            c.push(fresh[k], 1)
            want = c.sample(batch, 0.5, None if gen else u[k])
            prev = want[0]
        what = "cap %d replay %d" % (cap, rep)
        assert_sample_equal((out[0], out[1]) + tuple(out[2]), want, what)
        assert_tree_equal(g, c, what)
        assert g.size() == c.size and g._state()[1] == c.head, what
        assert np.float32(g.max_priority) == np.float32(c.max_priority)
        if rep % 3 == 1:  # eager calls in between
            extra = random_rows(rng, 2, shapes, dtypes)
            g.insert(*to_dev(extra)), c.push(extra, 2)
            got = g.update_priorities_insert_and_sample(torch.from_numpy(prev).cuda(), torch.from_numpy(pr[0]).cuda(),
                                                        *to_dev(fresh[0]), beta=0.7)
            ok = (prev >= 0) & (prev < cap)
            c.update(prev[ok], pr[0][ok]), c.push(fresh[0], 1)
            want = c.sample(batch, 0.7)
            assert_sample_equal(got, want, "eager after replay %d" % rep)
            prev = want[0]
    for f, (a, b) in enumerate(zip(g.storage(), [c.field(i) for i in range(len(shapes))])):
        assert np.array_equal(t2n(a).view(np.uint8), b.view(np.uint8)), f
    g.set_option("device_counters", 0)
    assert g.size() == c.size
    mrb.lib.lib().mrb_per_check(g._h, C.byref(C.c_uint32(0)), None)
    del graph
    g.destroy()


@pytest.mark.parametrize("seed", range(40))
def test_whole_step_calls_in_bursts_without_a_wait(mrb, orc, seed):
    """Seeded random configurations of mrb_per_update_push_sample - capacities 3 to 40,000, batches 1 to 600, rows of
    7 bytes to over 2 KB, one array per field and packed - called in bursts of up to 24 calls with no wait in between,
    in half of the bursts every call updating the rows the call before sampled (its indices read from that call's
    output on the device). Every call's sample, then trees, size, head and running max, against the oracle."""
    rng = np.random.default_rng(7000 + seed)
    layouts = [([(3,), (1,)], [np.float32, np.int32]), ([(300,), (1,), (3,)], [np.float32, np.int32, np.uint8]),
               ([(4,), (1,), (1,), (4,), (1,)], [np.float32, np.int32, np.float32, np.float32, np.bool_]),
               ([(512,), (1,)], [np.float32, np.int32]), ([(520,), (5,)], [np.float32, np.uint8]), ([(7,)], [np.uint8])]
    cap = int(rng.choice([3, 4, 5, 64, 200, 257, 1000, 2048, 2049, 4096, 5000, 9000, 10000, 16384, 16385, 40000]))
    shapes, dtypes = layouts[rng.integers(0, len(layouts))]
    alpha = float(rng.choice([0.0, 0.4, 0.6, 1.0]))
    batch = int(rng.choice([1, 2, 8, 33, 64, 64, 200, 384, 448, 449, 512, 600]))
    g = mrb.PER(alpha, cap, batch, shapes, torch_types(dtypes), seed0=seed + 1, packed_rows=bool(rng.integers(0, 3) == 0))
    c = orc.OraclePER(alpha, cap, shapes, dtypes, seed=seed + 1)
    gen = bool(rng.integers(0, 3) == 0)
    fill = int(rng.choice([cap, cap, max(1, cap // 2), max(1, cap - 5)]))
    rows = random_rows(rng, fill, shapes, dtypes)
    pr = (rng.pareto(1.5, fill) + 1e-6).astype(np.float32)
    g.insert(*to_dev(rows), priorities=torch.from_numpy(pr).cuda()), c.push(rows, fill, pr)
    for burst in range(3):
        nb = int(rng.integers(1, 25))
        follow = bool(rng.integers(0, 2))
        first = rng.integers(0, min(cap, c.size), batch)
        steps = []
        for k in range(nb):
            n = batch if follow else int(rng.choice([1, 7, 64, 65, 128, int(rng.integers(1, 385)), 384, 385]))
            ent = rng.integers(0, min(cap, c.size), n)
            if n > 4 and rng.integers(0, 3) == 0:
                ent[: n // 3] = ent[0]
            if n > 2 and rng.integers(0, 3) == 0:
                ent[-1] = (c.head + k) % cap  # the slot this call's push overwrites
            p = (rng.pareto(1.5, n) + 1e-6).astype(np.float32)
            if n > 8 and rng.integers(0, 6) == 0:
                p[3] = -1.0
            m = 1 if rng.integers(0, 8) else int(rng.integers(2, 5))
            kind = rng.integers(0, 4)
            ipr = (rng.pareto(1.5, m) + 1e-6).astype(np.float32) if kind == 0 else np.full(m, 1e9, np.float32) if kind == 1 else None
            steps.append(dict(ent=ent, p=p, row=random_rows(rng, m, shapes, dtypes), m=m, ipr=ipr,
                              u=None if gen else rng.random(batch).astype(np.float32), beta=float(rng.uniform(0, 1))))
        dev_in = [dict(ent=torch.from_numpy(s["ent"]).cuda(), p=torch.from_numpy(s["p"]).cuda(), row=to_dev(s["row"]),
                       ipr=None if s["ipr"] is None else torch.from_numpy(s["ipr"]).cuda(),
                       u=None if s["u"] is None else torch.from_numpy(s["u"]).cuda()) for s in steps]
        outs = [(torch.empty(batch, dtype=torch.int64, device="cuda"), torch.empty(batch, dtype=torch.float32, device="cuda"),
                 g._layout.empty(batch, g._dev)) for _ in range(nb)]
        torch.cuda.synchronize()
        prev = torch.from_numpy(first).cuda()
        for k in range(nb):
            d = dev_in[k]
            g.update_priorities_insert_and_sample(prev if follow else d["ent"], d["p"], *d["row"], beta=steps[k]["beta"],
                                                  insert_priorities=d["ipr"], uniforms=d["u"], out=outs[k])
            prev = outs[k][0]
        torch.cuda.synchronize()
        cprev = first
        for k, s in enumerate(steps):
            ent = cprev if follow else s["ent"]
            ok = (ent >= 0) & (ent < cap) & np.isfinite(s["p"]) & (s["p"] >= 0)
            c.update(ent[ok], s["p"][ok])
            c.push(s["row"], s["m"], s["ipr"])
            want = c.sample(batch, s["beta"], s["u"])
            what = "seed %d burst %d call %d of %d (follow %d, %d entries, %d rows)" % (seed, burst, k, nb, follow, len(ent), s["m"])
            assert_sample_equal((outs[k][0], outs[k][1]) + tuple(outs[k][2]), want, what)
            cprev = want[0]
        assert_tree_equal(g, c, "seed %d burst %d" % (seed, burst))
        assert g.size() == c.size and g._state()[1] == c.head
        assert np.float32(g.max_priority) == np.float32(c.max_priority)
    mrb.lib.lib().mrb_per_check(g._h, C.byref(C.c_uint32(0)), None)  # (flags of the invalid entries: not this test's subject)
    g.destroy()


@pytest.mark.parametrize("cap,npush,batch", [(3000, 1, 48), (10_000, 1, 64), (70_000, 1, 48), (70_000, 3, 300), (1_000_000, 4, 512),
                                             (3_000_000, 1, 40), (3_000_000, 2, 100)])
def test_hip_graph_replays_sample_then_update_push_with_device_counters(mrb, orc, cap, npush, batch):
    """The learner's step as two calls - a generator-driven sample, then update_priorities of the sampled rows and
    the push of new ones as ONE call (mrb_per_update_push) - recorded once with device_counters and replayed 10
    times: the push's own last launch moves the ring position on (no separate launch), the buffer fills, the ring
    wraps. Every replay equals the oracle's sample, update, push; eager calls in between use the same counters."""
    rng = np.random.default_rng(cap + npush)
    shapes, dtypes = ([(300,), (1,), (2,)], [np.float32, np.int32, np.uint8]) if cap < 10 ** 5 else ([(2,), (1,)], [np.float32, np.int32])
    g, c = make_pair(mrb, orc, 0.6, cap, batch, seed=17, shapes=shapes, dtypes=dtypes)
    fill = cap - 5 * npush - 2  # not full: the row count changes during the replays, then the ring wraps
    done = 0
    while done < fill:
        n = min(500_000, fill - done)
        rows = random_rows(rng, n, shapes, dtypes)
        g.insert(*to_dev(rows)), c.push(rows, n)
        done += n
    g.set_option("device_counters", 1)
    new_rows = [torch.zeros((npush,) + tuple(s), dtype=t).cuda() for s, t in zip(shapes, torch_types(dtypes))]
    pr_dev = torch.ones(batch, dtype=torch.float32, device="cuda")
    out = (torch.empty(batch, dtype=torch.int64, device="cuda"), torch.empty(batch, dtype=torch.float32, device="cuda"),
           g._layout.empty(batch, g._dev))
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        graph.capture_begin()
        g.sample(0.5, out=out)
        g.update_priorities_and_insert(out[0], pr_dev, *new_rows)
        graph.capture_end()
    torch.cuda.synchronize()
    for rep in range(10):
        fresh = random_rows(rng, npush, shapes, dtypes)
        pr = (rng.pareto(1.5, batch) + 1e-6).astype(np.float32)
        for dst, src in zip(new_rows, fresh):
            dst.copy_(torch.from_numpy(src))
        pr_dev.copy_(torch.from_numpy(pr))
        graph.replay()
        torch.cuda.synchronize()
        want = c.sample(batch, 0.5)
        assert_sample_equal((out[0], out[1]) + tuple(out[2]), want, "cap %d replay %d" % (cap, rep))
        c.update(want[0], pr)
        c.push(fresh, npush)
        assert_tree_equal(g, c, "cap %d replay %d" % (cap, rep))
        assert g.size() == c.size and g._state()[1] == c.head, "cap %d replay %d" % (cap, rep)
        assert np.float32(g.max_priority) == np.float32(c.max_priority)
        if rep % 4 == 2:  # eager calls in between
            extra = random_rows(rng, 3, shapes, dtypes)
            g.insert(*to_dev(extra)), c.push(extra, 3)
            one = random_rows(rng, 1, shapes, dtypes)
            g.insert(*to_dev(one)), c.push(one, 1)
            assert_sample_equal(g.sample(0.9), c.sample(batch, 0.9), "eager after replay %d" % rep)
    for f, (a, b) in enumerate(zip(g.storage(), [c.field(i) for i in range(len(shapes))])):
        assert np.array_equal(t2n(a).view(np.uint8), b.view(np.uint8)), f
    g.set_option("device_counters", 0)
    assert g.size() == c.size
    del graph
    g.destroy()
