"""Writes the golden fixtures in this directory.

The reference holds no vectors for this path (its buffer tests are disabled and
assert only invariants), and its arithmetic lives in MindSpore, which is not
available. These fixtures therefore freeze THIS repository's contract: they are
produced by the CPU oracle (oracle/mrb_oracle.c) after tests/test_oracle_pins.py
has pinned it, and both the oracle and the HIP library must reproduce them bit
for bit. Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import orc  # noqa: E402


def per_scenario():
    """Config-1-shaped loop at capacity 100 (128 leaves): fill, then 40 x {sample 16, update, insert 1}."""
    rng = np.random.default_rng(20250101)
    cap, batch, alpha, beta, steps = 100, 16, 0.6, 0.4, 40
    shapes, dtypes = [(4,), (1,), (1,), (4,), (1,)], [np.float32, np.int32, np.float32, np.float32, np.bool_]
    per = orc.OraclePER(alpha, cap, shapes, dtypes, seed=11)

    def rows(n):
        return [rng.uniform(-2.4, 2.4, (n, 4)).astype(np.float32), rng.integers(0, 2, (n, 1)).astype(np.int32),
                np.ones((n, 1), np.float32), rng.uniform(-2.4, 2.4, (n, 4)).astype(np.float32),
                rng.random((n, 1)) < 0.05]

    fill = rows(cap)
    per.push(fill, cap)
    out = {"cap": cap, "batch": batch, "alpha": np.float32(alpha), "beta": np.float32(beta), "steps": steps}
    for f, a in enumerate(fill):
        out["fill_%d" % f] = a
    U, TD, IDX, W, NEW = [], [], [], [], [[] for _ in shapes]
    G = [[] for _ in shapes]
    for _ in range(steps):
        u = rng.random(batch).astype(np.float32)
        idx, w, got = per.sample(batch, beta, u)
        td = (np.abs(rng.normal(size=batch)) + 1e-6).astype(np.float32)
        per.update(idx, td)
        one = rows(1)
        per.push(one, 1)
        U.append(u), TD.append(td), IDX.append(idx), W.append(w)
        for f in range(len(shapes)):
            NEW[f].append(one[f][0])
            G[f].append(got[f])
    s, m = per.export_tree()
    out.update(uniforms=np.stack(U), td=np.stack(TD), indices=np.stack(IDX), weights=np.stack(W), sum_heap=s,
               min_heap=m, max_priority=np.float32(per.max_priority))
    for f in range(len(shapes)):
        out["new_%d" % f] = np.stack(NEW[f])
        out["gathered_%d" % f] = np.stack(G[f])
    np.savez_compressed(os.path.join(HERE, "per_config1_small.npz"), **out)


def urb_scenario():
    """Uniform ring at capacity 37: appends of varying size (one larger than the capacity), a reset, gathers."""
    rng = np.random.default_rng(20250102)
    cap = 37
    shapes, dtypes = [(17,), (6,), (1,)], [np.float32, np.float32, np.bool_]
    buf = orc.OracleUniform(cap, shapes, dtypes, seed=5)
    sizes = [1, 5, 20, 30, 1, 50, 3, 0, 12, 40, 7]  # 0 marks the reset
    out = {"cap": cap, "sizes": np.array(sizes)}
    for step, n in enumerate(sizes):
        if n == 0:
            buf.reset()
        else:
            r = [rng.normal(size=(n, 17)).astype(np.float32), rng.uniform(-1, 1, (n, 6)).astype(np.float32),
                 rng.random((n, 1)) < 0.01]
            for f, a in enumerate(r):
                out["rows_%d_%d" % (step, f)] = a
            buf.append(r, n)
        out["count_%d" % step] = buf.count
        out["head_%d" % step] = buf.head
        if buf.count:
            idx = rng.integers(0, buf.count, 9)
            out["idx_%d" % step] = idx
            for f, a in enumerate(buf.gather(idx)):
                out["gather_%d_%d" % (step, f)] = a
            for f, a in enumerate(buf.get_item(-1)):
                out["newest_%d_%d" % (step, f)] = a
    for f in range(len(shapes)):
        out["storage_%d" % f] = buf.field(f)
    np.savez_compressed(os.path.join(HERE, "urb_ring_small.npz"), **out)


def powf_vectors():
    rng = np.random.default_rng(20250103)
    x = np.exp(rng.uniform(-30, 20, 4096)).astype(np.float32)
    out = {"x": x}
    for a in (0.4, 0.6, 1.0, -0.4, -1.0):
        out["pow_%s" % a] = orc.powf_array(x, a)
    np.savez_compressed(os.path.join(HERE, "powf_vectors.npz"), **out)


if __name__ == "__main__":
    per_scenario()
    urb_scenario()
    powf_vectors()
    print("wrote fixtures to", HERE)
