"""Pins the CPU oracle (oracle/mrb_oracle.c) with checks that do not retype its
formulas: hand-computed known answers, brute force on tiny inputs, numpy
library routines, closed forms and the invariants asserted by the reference's
own (disabled) buffer tests.

Reference invariants used:
  I1 indices < number of pushed rows      tests/st/test_priority_replay_buffer.py:50,61
  I2 gathered row == row pushed at index  tests/st/test_priority_replay_buffer.py:51-54,63-66
  I3 a minimised priority is not redrawn  tests/st/test_priority_replay_buffer.py:57-62
  I4 successive uniform samples differ    tests/st/test_uniform_replay_buffer.py:83-85
"""
import numpy as np
import pytest


# ---------------------------------------------------------------- powf / rng
def test_powf_matches_libm_pow_within_one_ulp(orc):
    rng = np.random.default_rng(1)
    x = np.exp(rng.uniform(-40, 20, 400_000)).astype(np.float32)
    for a in (0.6, 0.4, 0.5, 0.7, 1.5, -0.4, -0.6, -1.0):
        got = orc.powf_array(x, a)
        want = np.power(x.astype(np.float64), np.float64(np.float32(a))).astype(np.float32)
        ulps = np.abs(got.view(np.int32).astype(np.int64) - want.view(np.int32).astype(np.int64))
        assert ulps.max() <= 1, a
        assert (ulps != 0).mean() < 1e-3, a


def test_powf_exact_cases(orc):
    assert orc.powf(0.0, 0.6) == 0.0
    assert orc.powf(123.25, 0.0) == 1.0
    assert orc.powf(1.0, -0.37) == 1.0
    for v in (1e-7, 0.3, 7.0, 1e30):
        assert np.float32(orc.powf(v, 1.0)) == np.float32(v)
    for r in (2.0, 3.0, 12.0, 1024.0, 0.5, 0.125):
        assert orc.powf(r * r, 0.5) == r
    assert orc.powf(3.0, 2.0) == 9.0
    assert orc.powf(2.0, -1.0) == 0.5
    assert orc.powf(1e30, 2.0) == np.inf
    assert orc.powf(1e-30, 2.0) == 0.0
    # zero base, as libm pow(): 0^a is 0 for a > 0 and +inf for a < 0 (a zero minimum priority then
    # gives importance weights r / inf = 0, not r / 0 = inf)
    for a in (-0.4, -1.0, -2.5):
        assert orc.powf(0.0, a) == np.inf
    with np.errstate(divide="ignore"):
        assert np.power(np.float64(0.0), -0.4) == np.inf  # what numpy's pow (libm) gives for the same case
    # monotone in x for a > 0
    x = np.linspace(0.001, 10, 5000).astype(np.float32)
    assert np.all(np.diff(orc.powf_array(x, 0.6)) >= 0)


def test_rng_range_and_streams(orc):
    u0 = orc.rng_uniform(42, 0, 4096)
    u1 = orc.rng_uniform(42, 1, 4096)
    assert u0.dtype == np.float32 and np.all(u0 >= 0) and np.all(u0 < 1)
    assert abs(u0.mean() - 0.5) < 0.03 and not np.array_equal(u0, u1)
    L = orc.lib()
    b = np.array([L.orc_rng_below(7, 3, k, 1000) for k in range(5000)])
    assert b.min() >= 0 and b.max() < 1000 and len(np.unique(b)) > 900


# ------------------------------------------------------------- uniform ring
class ListRing:
    """Brute-force model: a Python list of rows, oldest first."""

    def __init__(self, cap):
        self.cap, self.rows = cap, []

    def append(self, rows):
        self.rows.extend(rows)
        self.rows = self.rows[-self.cap:]


@pytest.mark.parametrize("cap", [1, 3, 4, 7])
def test_ring_matches_list_model(orc, cap):
    rng = np.random.default_rng(cap)
    shapes, dtypes = [(2,), (1,)], [np.float32, np.int32]
    buf = orc.OracleUniform(cap, shapes, dtypes)
    model = ListRing(cap)
    serial = 0
    for step in range(60):
        n = int(rng.integers(1, 2 * cap + 3))
        ids = np.arange(serial, serial + n)
        serial += n
        buf.append([np.stack([ids, -ids], 1).astype(np.float32), ids.astype(np.int32)], n)
        model.append(list(ids))
        assert buf.count == len(model.rows) == min(serial, cap)
        # logical order: get_item(j) is the j-th oldest row; negative from the newest
        for j in range(buf.count):
            f0, f1 = buf.get_item(j)
            assert f1[0] == model.rows[j] and f0[0] == model.rows[j] and f0[1] == -model.rows[j]
            assert buf.get_item(j - buf.count)[1][0] == model.rows[j]
        with pytest.raises(IndexError):
            buf.get_item(buf.count)
        # head is the slot of the oldest row once full
        if buf.count == cap:
            assert buf.field(1)[buf.head, 0] == model.rows[0]
        else:
            assert buf.head == 0
        # physical layout before wrapping: slot i holds the i-th row
        if serial <= cap:
            assert list(buf.field(1)[:serial, 0]) == model.rows


def test_ring_closed_form_and_reset(orc):
    cap, m = 5, 13
    buf = orc.OracleUniform(cap, [(1,)], [np.int64])
    for r in range(m):
        buf.append([np.array([r])], 1)
    # after m rows: logical item j is row max(0, m-cap)+j
    assert [int(buf.get_item(j)[0][0]) for j in range(cap)] == [m - cap + j for j in range(cap)]
    assert buf.head == m % cap
    # reset: count 0, head kept (mindspore_rl/core/uniform_replay_buffer.py:149)
    h = buf.head
    buf.reset()
    assert buf.count == 0 and buf.head == h
    buf.append([np.array([100, 101])], 2)
    assert buf.count == 2 and buf.head == (h + 2) % cap


def test_gather_equals_numpy_take(orc):
    rng = np.random.default_rng(5)
    cap = 50
    shapes, dtypes = [(3, 2), (1,), (5,)], [np.float32, np.bool_, np.uint8]
    buf = orc.OracleUniform(cap, shapes, dtypes)
    a = rng.normal(size=(cap, 3, 2)).astype(np.float32)
    b = rng.random((cap, 1)) < 0.5
    c = rng.integers(0, 256, (cap, 5)).astype(np.uint8)
    buf.append([a, b, c], cap)
    idx = rng.integers(0, cap, 200)
    g = buf.gather(idx)
    assert np.array_equal(g[0], a[idx]) and np.array_equal(g[1], b[idx]) and np.array_equal(g[2], c[idx])
    with pytest.raises(IndexError):
        buf.gather([cap])


def test_uniform_sample_successive_calls_differ(orc):  # I4
    buf = orc.OracleUniform(200, [(1,)], [np.int32], seed=3)
    buf.append([np.arange(200, dtype=np.int32)], 200)
    i0, r0 = buf.sample(32)
    i1, r1 = buf.sample(32)
    assert not np.array_equal(i0, i1)
    assert np.array_equal(r0[0][:, 0], i0) and np.array_equal(r1[0][:, 0], i1)
    assert i0.min() >= 0 and i0.max() < 200
    with pytest.raises(ValueError):
        orc.OracleUniform(10, [(1,)], [np.int32]).sample(1)  # batch > count


# --------------------------------------------------------------- PER trees
def pairwise_levels(leaf_sum, leaf_min):
    """Segment tree from its leaves by repeated pairwise reduction of whole levels
    (numpy float32 adds) -> heap arrays."""
    n = leaf_sum.size
    s = np.zeros(2 * n, np.float32)
    m = np.zeros(2 * n, np.float32)
    s[n:], m[n:] = leaf_sum, leaf_min
    ls, lm = leaf_sum.astype(np.float32), leaf_min.astype(np.float32)
    while ls.size > 1:
        ls = (ls[0::2] + ls[1::2]).astype(np.float32)
        lm = np.minimum(lm[0::2], lm[1::2])
        s[ls.size:2 * ls.size], m[lm.size:2 * lm.size] = ls, lm
    return s, m


def rows_for(n, start=0):
    ids = np.arange(start, start + n)
    return [np.repeat(ids[:, None], 3, 1).astype(np.float32), ids.astype(np.int32)[:, None]]


def new_per(orc, alpha, cap, seed=1):
    return orc.OraclePER(alpha, cap, [(3,), (1,)], [np.float32, np.int32], seed=seed)


def test_known_answer_tiny_tree(orc):
    """Hand-computed. Priorities 1,2,3,4 (alpha 1): sums [10; 3,7; 1,2,3,4].
    B=4, u=.5: seg=2.5, masses 1.25, 3.75, 6.25, 8.75.
      1.25: <=3 L; >1 -> .25, R -> leaf 1     3.75: >3 -> .75, R; <=3 L -> leaf 2
      6.25: >3 -> 3.25, R; >3 -> .25 R -> 3   8.75: >3 -> 5.75; >3 -> 2.75 -> leaf 3
    weights beta=1: (p/pmin)^-1 = 1/2, 1/3, 1/4, 1/4."""
    per = new_per(orc, 1.0, 4)
    per.push(rows_for(4), 4)
    per.update([0, 1, 2, 3], [1, 2, 3, 4])
    s, m = per.export_tree()
    assert list(s[1:]) == [10, 3, 7, 1, 2, 3, 4] and list(m[1:]) == [1, 1, 3, 1, 2, 3, 4]
    idx, w, rows = per.sample(4, 1.0, uniforms=[0.5] * 4)
    assert list(idx) == [1, 2, 3, 3]
    np.testing.assert_allclose(w, [1 / 2, 1 / 3, 1 / 4, 1 / 4], rtol=1e-6)
    assert list(rows[1][:, 0]) == [1, 2, 3, 3]
    # tie-break: mass exactly equal to the left sum goes left (decision, unpinned by the reference)
    idx, _, _ = per.sample(1, 1.0, uniforms=[0.3])  # mass 3.0 == sum[2] -> left subtree; then 3 > 1 -> leaf 1
    assert list(idx) == [1]
    assert per.max_priority == 4.0


@pytest.mark.parametrize("cap", [1, 2, 5, 8, 37, 64, 100])
def test_tree_equals_pairwise_rebuild_after_random_ops(orc, cap):
    rng = np.random.default_rng(cap)
    per = new_per(orc, 0.6, cap)
    leaves = per.leaves
    assert leaves >= cap and leaves & (leaves - 1) == 0 and leaves < 2 * max(cap, 1) + 1
    leaf = np.zeros(leaves, np.float32)
    leafmin = np.full(leaves, np.finfo(np.float32).max, np.float32)
    maxp, pushes, serial = np.float32(1.0), 0, 0
    for step in range(40):
        n = int(rng.integers(1, cap + 3))
        per.push(rows_for(n, serial), n)
        serial += n
        for j in range(n):
            leaf[pushes % cap] = leafmin[pushes % cap] = maxp  # new rows: running max, not raised to alpha
            pushes += 1
        k = int(rng.integers(1, 2 * cap + 2))
        idx = rng.integers(0, cap, k)
        pr = np.abs(rng.normal(size=k)).astype(np.float32) * 3 + np.float32(1e-6)
        per.update(idx, pr)
        q = orc.powf_array(pr, 0.6)
        for i, v in zip(idx, q):  # duplicates: last write wins
            leaf[i] = leafmin[i] = v
        maxp = max(maxp, q.max())  # over all entries, overwritten ones included
        s, m = per.export_tree()
        es, em = pairwise_levels(leaf, leafmin)
        assert np.array_equal(s[1:].view(np.int32), es[1:].view(np.int32))
        assert np.array_equal(m[1:].view(np.int32), em[1:].view(np.int32))
        assert per.max_priority == maxp
        assert per.size == min(pushes, cap) and per.head == pushes % cap


def test_load_state_rebuilds_the_same_tree_and_continues_identically(orc):
    """orc_per_load_state (leaves in, every internal node recomputed bottom-up) against numpy's pairwise
    reduction of the same leaves, and against the buffer the state came from, which then takes the same
    calls; the same for the uniform ring and the reservoir."""
    rng = np.random.default_rng(31)
    for cap in (5, 64, 100):
        a = new_per(orc, 0.6, cap)
        a.push(rows_for(cap + 3, 0), cap + 3)
        a.update(rng.integers(0, cap, 40), np.abs(rng.normal(size=40)).astype(np.float32) + np.float32(1e-6))
        a.sample(4, 0.5)
        state = a.state_dict()
        b = new_per(orc, 0.6, cap)
        b.load_state_dict(state)
        leaves = a.leaves
        leaf = np.zeros(leaves, np.float32)
        leafmin = np.full(leaves, np.finfo(np.float32).max, np.float32)
        leaf[:a.size] = leafmin[:a.size] = state["leaves"]
        es, em = pairwise_levels(leaf, leafmin)
        s, m = b.export_tree()
        assert np.array_equal(s[1:].view(np.int32), es[1:].view(np.int32))
        assert np.array_equal(m[1:].view(np.int32), em[1:].view(np.int32))
        for step in range(5):
            ia, wa, ra = a.sample(4, 0.7)
            ib, wb, rb = b.sample(4, 0.7)
            assert np.array_equal(ia, ib) and np.array_equal(wa.view(np.int32), wb.view(np.int32))
            assert all(np.array_equal(x, y) for x, y in zip(ra, rb))
            a.push(rows_for(3, 1000 + step), 3), b.push(rows_for(3, 1000 + step), 3)
            a.update(ia, wa + np.float32(0.5)), b.update(ib, wb + np.float32(0.5))
            assert a.max_priority == b.max_priority and (a.size, a.head) == (b.size, b.head)
            assert np.array_equal(a.export_tree()[0][1:].view(np.int32), b.export_tree()[0][1:].view(np.int32))
    shapes, dtypes = [(2,)], [np.int32]
    u = orc.OracleUniform(7, shapes, dtypes, seed=3)
    u.append([np.arange(24).reshape(12, 2)], 12)
    u.sample(3)
    w = orc.OracleUniform(7, shapes, dtypes, seed=99)
    w.load_state_dict(u.state_dict())
    assert (w.count, w.head) == (u.count, u.head) == (7, 5)
    assert np.array_equal(u.sample(3)[0], w.sample(3)[0]) and np.array_equal(u.get_item(0)[0], w.get_item(0)[0])
    r = orc.OracleReservoir(6, shapes, dtypes, seed=4)
    r.push([np.arange(60).reshape(30, 2)], 30)
    q = orc.OracleReservoir(6, shapes, dtypes, seed=5)
    q.load_state_dict(r.state_dict())
    more = [np.arange(100, 140).reshape(20, 2)]
    r.push(more, 20), q.push(more, 20)
    assert np.array_equal(r.field(0), q.field(0)) and (r.size, r.total) == (q.size, q.total) == (6, 50)
    assert np.array_equal(r.sample(4)[0], q.sample(4)[0])


def test_root_is_pairwise_not_sequential_sum(orc):
    per = new_per(orc, 1.0, 1024)
    rng = np.random.default_rng(0)
    pr = (rng.random(1024) * 10 + 0.01).astype(np.float32)
    per.push(rows_for(1024), 1024)
    per.update(np.arange(1024), pr)
    s, _ = per.export_tree()
    x = pr.copy()
    while x.size > 1:
        x = x[0::2] + x[1::2]
    seq = np.float32(0)
    for v in pr:
        seq = np.float32(seq + v)
    assert s[1] == x[0]
    assert seq != x[0]  # this input separates the two orders


def test_update_duplicates_last_write_wins_and_untouched_nodes(orc):
    per = new_per(orc, 1.0, 16)
    per.push(rows_for(16), 16)
    before_s, _ = per.export_tree()
    per.update([3, 3, 3, 9, 3], [5.0, 7.0, 100.0, 2.0, 0.25])
    s, m = per.export_tree()
    assert s[16 + 3] == 0.25 and s[16 + 9] == 2.0
    assert per.max_priority == 100.0  # overwritten duplicate still raises the max
    touched = set()
    for leaf in (3, 9):
        i = 16 + leaf
        while i >= 1:
            touched.add(i)
            i //= 2
    for i in range(1, 32):
        if i not in touched:
            assert s[i] == before_s[i]
    # new pushes take the running max
    per.push(rows_for(1, 16), 1)
    s, _ = per.export_tree()
    assert s[16 + 0] == 100.0


# ------------------------------------------------------------ PER sampling
def test_descent_equals_prefix_sum_search_when_arithmetic_is_exact(orc):
    """Integer priorities, power-of-two batch and dyadic uniforms make every float
    operation exact, so the tree descent must equal a search over the cumulative
    sums: the first leaf whose inclusive prefix sum reaches the mass."""
    rng = np.random.default_rng(11)
    for cap in (4, 16, 50, 128):
        per = new_per(orc, 1.0, cap)
        per.push(rows_for(cap), cap)
        pr = rng.integers(0, 9, cap).astype(np.float32)  # zeros included
        pr[rng.integers(0, cap)] = 8
        total = pr.sum()
        per.update(np.arange(cap), pr)
        for batch in (1, 4, 32):
            u = (rng.integers(0, 256, batch) / 256).astype(np.float32)
            idx, _, _ = per.sample(batch, 0.5, uniforms=u, gather=False)
            mass = (u.astype(np.float64) + np.arange(batch)) * (float(total) / batch)
            want = np.searchsorted(np.cumsum(pr.astype(np.float64)), mass, side="left")
            assert np.array_equal(idx, want), (cap, batch)


def test_stratified_indices_monotone_and_filled(orc):  # I1
    rng = np.random.default_rng(2)
    per = new_per(orc, 0.6, 200)  # 256 leaves, 100 filled
    per.push(rows_for(100), 100)
    per.update(np.arange(100), rng.lognormal(size=100).astype(np.float32))
    for t in range(50):
        u = rng.random(32).astype(np.float32)
        idx, w, rows = per.sample(32, 0.4, uniforms=u)
        assert np.all(idx < 100) and np.all(idx >= 0)
        assert np.all(np.diff(idx) >= 0)
        assert np.array_equal(rows[1][:, 0], idx) and np.array_equal(rows[0], np.repeat(idx[:, None], 3, 1))  # I2
        assert np.all(w > 0) and np.all(w <= 1.0 + 1e-6)
    # smallest draws stay inside the filled leaves
    idx, _, _ = per.sample(32, 0.4, uniforms=np.zeros(32, np.float32), gather=False)
    assert np.all(idx < 100)
    # The largest draw of the LAST stratum can round to a mass above the total; the
    # descent applies no clamp (as the reference's algorithm applies none), so that one
    # stratum may end on an unfilled leaf. Every other stratum stays inside.
    idx, _, _ = per.sample(32, 0.4, uniforms=np.full(32, np.float32(1) - np.float32(2 ** -24)), gather=False)
    assert np.all(idx[:-1] < 100) and 0 <= idx[-1] < per.leaves


def test_one_hot_and_equal_priorities(orc):
    per = new_per(orc, 1.0, 64)
    per.push(rows_for(64), 64)
    pr = np.zeros(64, np.float32)
    pr[37] = 2.5
    per.update(np.arange(64), pr)
    idx, _, _ = per.sample(16, 1.0, uniforms=np.random.default_rng(0).random(16), gather=False)
    assert np.all(idx == 37)
    # equal priorities (power of two count): stratum k of B=64 lands on leaf k, weights all 1
    per.update(np.arange(64), np.full(64, 0.5, np.float32))
    idx, w, _ = per.sample(64, 0.7, uniforms=np.full(64, 0.5, np.float32), gather=False)
    assert np.array_equal(idx, np.arange(64)) and np.all(w == 1.0)


def test_is_weights_closed_form(orc):
    rng = np.random.default_rng(3)
    per = new_per(orc, 0.6, 1000)
    per.push(rows_for(1000), 1000)
    pr = rng.lognormal(size=1000).astype(np.float32)
    per.update(np.arange(1000), pr)
    s, m = per.export_tree()
    leaves = per.leaves
    for beta in (0.0, 0.4, 0.7, 1.0):
        idx, w, _ = per.sample(128, beta, uniforms=rng.random(128).astype(np.float32), gather=False)
        p = s[leaves + idx].astype(np.float64)
        want = (p / np.float64(m[1])) ** (-beta)  # (p/total*N)^-b / (pmin/total*N)^-b == (p/pmin)^-b
        np.testing.assert_allclose(w, want, rtol=1e-6)
        if beta == 0.0:
            assert np.all(w == 1.0)
    # the minimum-priority row has weight exactly 1 and nothing exceeds it
    amin = int(np.argmin(s[leaves:leaves + 1000]))
    assert m[1] == s[leaves + amin]


def test_reference_scenario_minimised_priorities_not_redrawn(orc):  # I1, I2, I3
    """tests/st/test_priority_replay_buffer.py:34-66 replayed on the oracle:
    capacity 200, batch 32, alpha 1, push 100 rows whose values equal their row
    number, sample, set those priorities to 1e-7, sample again."""
    per = orc.OraclePER(1.0, 200, [(17,), (6,)], [np.float32, np.int32], seed=42)
    for i in range(100):
        per.push([np.ones(17, np.float32) * i, np.ones(6, np.int32) * i], 1)
    idx, w, (states, actions) = per.sample(32, 1.0)
    assert np.all(idx < 100) and w.shape == (32,) and w.dtype == np.float32
    assert np.allclose(states, np.broadcast_to(idx.reshape(-1, 1), states.shape))
    assert np.allclose(actions, np.broadcast_to(idx.reshape(-1, 1), actions.shape))
    per.update(idx, np.ones(32, np.float32) * 1e-7)
    idx2, _, (states2, actions2) = per.sample(32, 1.0)
    assert np.all(idx2 < 100) and np.all(idx != idx2)
    assert np.allclose(states2, np.broadcast_to(idx2.reshape(-1, 1), states2.shape))
    assert np.allclose(actions2, np.broadcast_to(idx2.reshape(-1, 1), actions2.shape))


def test_push_wraps_and_explicit_priorities(orc):
    per = new_per(orc, 0.5, 6)
    per.push(rows_for(4), 4)
    per.push(rows_for(5, 4), 5, priorities=[4.0, 9.0, 16.0, 25.0, 36.0])  # slots 4,5,0,1,2
    s, _ = per.export_tree()
    assert list(s[8:14]) == [4.0, 5.0, 6.0, 1.0, 2.0, 3.0]
    assert per.size == 6 and per.head == 3 and per.max_priority == 6.0
    assert list(per.field(1)[:, 0]) == [6, 7, 8, 3, 4, 5]
    # more rows than slots in one call: the last `capacity` survive
    per.push(rows_for(14, 100), 14)
    assert per.head == (9 + 14) % 6
    order = [int(v) for v in per.field(1)[:, 0]]
    assert sorted(order) == list(range(108, 114)) and order[(per.head - 1) % 6] == 113


def test_errors(orc):
    per = new_per(orc, 0.6, 8)
    with pytest.raises(ValueError):
        per.sample(4, 0.4, uniforms=[0.1] * 4)  # empty
    per.push(rows_for(8), 8)
    with pytest.raises(ValueError):
        per.update([8], [1.0])
    with pytest.raises(ValueError):
        per.update([0], [-1.0])
    with pytest.raises(ValueError):
        per.update([0], [np.nan])


# ---------------------------------------------------------------- reservoir
def test_reservoir_keeps_every_row_with_equal_probability(orc):
    """Defining property of reservoir sampling: after N rows, each is held with probability capacity / N."""
    cap, n, trials = 8, 40, 6000
    kept = np.zeros(n)
    for t in range(trials):
        b = orc.OracleReservoir(cap, [(1,)], [np.int32], seed=5000 + t)
        if t % 2:
            b.push([np.arange(n, dtype=np.int32)[:, None]], n)  # one batch
        else:
            for i in range(n):  # row by row: same policy
                b.push([np.array([[i]], np.int32)], 1)
        held = b.field(0)[:, 0]
        assert len(set(held)) == cap and b.size == cap and b.total == n
        kept[held] += 1
    p = kept / trials
    sigma = np.sqrt(0.2 * 0.8 / trials)
    assert np.all(np.abs(p - cap / n) < 5 * sigma), p


def test_reservoir_fill_phase_and_batch_equals_sequential(orc):
    a = orc.OracleReservoir(10, [(2,), (1,)], [np.float32, np.int32], seed=9)
    b = orc.OracleReservoir(10, [(2,), (1,)], [np.float32, np.int32], seed=9)
    ids = np.arange(37)
    rows = [np.stack([ids, -ids], 1).astype(np.float32), ids.astype(np.int32)[:, None]]
    a.push([r[:6] for r in rows], 6)
    assert a.size == 6 and list(a.field(1)[:6, 0]) == [0, 1, 2, 3, 4, 5]  # slots fill in order
    a.push([r[6:] for r in rows], 31)
    for i in range(37):
        b.push([r[i:i + 1] for r in rows], 1)
    assert np.array_equal(a.field(0), b.field(0)) and np.array_equal(a.field(1), b.field(1))
    assert a.total == b.total == 37 and a.size == 10


def test_reservoir_reference_scenario(orc):
    """tests/st/test_reservoir_replay_buffer.py:33-54: capacity 100, sample 256 rows after 100 pushes
    whose values equal their row number; every sampled row is internally consistent."""
    buf = orc.OracleReservoir(100, [(17,), (6,)], [np.float32, np.int32], seed=42)
    for i in range(100):
        buf.push([np.ones((1, 17), np.float32) * i, np.ones((1, 6), np.int32) * i], 1)
    idx, (states, actions) = buf.sample(256)
    assert np.allclose(states, states[:, 0:1]) and np.allclose(actions, actions[:, 0:1])
    assert np.allclose(states[:, 0], actions[:, 0]) and np.array_equal(states[:, 0], idx)
    idx2, _ = buf.sample(256)
    assert not np.array_equal(idx, idx2) and idx.min() >= 0 and idx.max() < 100
    with pytest.raises(ValueError):
        orc.OracleReservoir(4, [(1,)], [np.int32]).sample(2)  # empty


# --------------------------------------------------------- discounted return
def test_discounted_return_reference_known_answers(orc):
    """The reference's own vectors (tests/st/test_discounted_return.py:39-53)."""
    ret = orc.discounted_return(np.ones((4, 1), np.float32), [[False], [False], [True], [False]], [2.0], 0.99)
    assert np.allclose(ret, np.array([[2.9701], [1.99], [1.0], [2.98]], np.float32))
    ret = orc.discounted_return(np.ones(4, np.float32), np.array([False, True, False, True])[:, None], [2.0], 0.99)
    assert np.allclose(ret, np.array([1.99, 1.0, 1.99, 1.0], np.float32))


def test_discounted_return_closed_forms(orc):
    rng = np.random.default_rng(4)
    t, b, inner = 50, 7, 3
    r = rng.normal(size=(t, b, inner)).astype(np.float32)
    v = rng.normal(size=(b, inner)).astype(np.float32)
    none = np.zeros((t, b), bool)
    # gamma 0: the return is the reward; gamma 1 without episode ends: reversed running sum plus the bootstrap
    assert np.array_equal(orc.discounted_return(r, none, v, 0.0), r)
    want = np.cumsum(r[::-1].astype(np.float64), 0)[::-1] + v
    np.testing.assert_allclose(orc.discounted_return(r, none, v, 1.0), want, rtol=1e-5, atol=1e-5)
    # general: float64 evaluation of the definition, episode ends cutting the bootstrap
    d = rng.random((t, b)) < 0.1
    g = 0.97
    want = np.zeros((t, b, inner))
    last = v.astype(np.float64)
    for step in range(t - 1, -1, -1):
        last = r[step] + (1 - d[step])[:, None] * g * last
        want[step] = last
    np.testing.assert_allclose(orc.discounted_return(r, d, v, g), want, rtol=1e-5, atol=1e-5)
    # a done at step s makes everything at or before s independent of what follows
    d2 = none.copy()
    d2[20] = True
    a1 = orc.discounted_return(r, d2, v, g)
    r2 = r.copy()
    r2[21:] += 5.0
    a2 = orc.discounted_return(r2, d2, v * 3, g)
    assert np.array_equal(a1[:21], a2[:21]) and not np.array_equal(a1[21:], a2[21:])


def test_all_cores_mode_of_the_timing_baseline_changes_nothing(orc):
    """The OpenMP mode used for the "all host cores" baseline only shares out the row copies."""
    rng = np.random.default_rng(8)
    per = orc.OraclePER(0.6, 500, [(33,), (1,)], [np.float32, np.int32], seed=2)
    per.push([rng.normal(size=(500, 33)).astype(np.float32), np.arange(500, dtype=np.int32)[:, None]], 500)
    per.update(np.arange(500), rng.lognormal(size=500).astype(np.float32))
    u = rng.random(64).astype(np.float32)
    one = per.sample(64, 0.5, u)
    orc.set_threads(4)
    try:
        many = per.sample(64, 0.5, u)
    finally:
        orc.set_threads(1)
    assert np.array_equal(one[0], many[0]) and np.array_equal(one[1], many[1])
    assert all(np.array_equal(a, b) for a, b in zip(one[2], many[2]))
