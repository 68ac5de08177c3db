"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py):
the oracle must reproduce them on the CPU, the HIP library on the GPU, bit for bit."""
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
PER_SHAPES = [(4,), (1,), (1,), (4,), (1,)]
PER_DTYPES = [np.float32, np.int32, np.float32, np.float32, np.bool_]
URB_SHAPES = [(17,), (6,), (1,)]
URB_DTYPES = [np.float32, np.float32, np.bool_]


def same_bits(a, b):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    return a.shape == b.shape and a.dtype == b.dtype and np.array_equal(a.view(np.uint8), b.view(np.uint8))


class OracleSide:
    def __init__(self, orc):
        self.orc = orc

    def per(self, alpha, cap, batch):
        return self.orc.OraclePER(alpha, cap, PER_SHAPES, PER_DTYPES, seed=11)

    def urb(self, cap):
        return self.orc.OracleUniform(cap, URB_SHAPES, URB_DTYPES, seed=5)

    def push(self, b, rows, n):
        b.push(rows, n)

    def sample(self, b, batch, beta, u):
        i, w, f = b.sample(batch, beta, u)
        return i, w, f

    def update(self, b, idx, td):
        b.update(idx, td)

    def tree(self, b):
        return b.export_tree() + (np.float32(b.max_priority),)

    def append(self, b, rows, n):
        b.append(rows, n)

    def state(self, b):
        return b.count, b.head

    def gather(self, b, idx):
        return b.gather(idx)

    def newest(self, b):
        return b.get_item(-1)

    def storage(self, b, f):
        return b.field(f)


class HipSide:
    def __init__(self):
        import torch
        from gpu_util import torch_types
        from mindrl_amd.core import PriorityReplayBuffer, UniformReplayBuffer
        self.torch, self.tt, self.P, self.U = torch, torch_types, PriorityReplayBuffer, UniformReplayBuffer

    def dev(self, arrays):
        return [self.torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in arrays]

    def per(self, alpha, cap, batch):
        return self.P(alpha, cap, batch, PER_SHAPES, self.tt(PER_DTYPES), seed0=11)

    def urb(self, cap):
        return self.U(9, cap, URB_SHAPES, self.tt(URB_DTYPES), seed=5)

    def push(self, b, rows, n):
        b.insert(*self.dev(rows))

    def sample(self, b, batch, beta, u):
        out = b.sample(beta, uniforms=self.torch.from_numpy(u).cuda())
        return out[0].cpu().numpy(), out[1].cpu().numpy(), [f.cpu().numpy() for f in out[2:]]

    def update(self, b, idx, td):
        b.update_priorities(self.torch.from_numpy(idx).cuda(), self.torch.from_numpy(td).cuda())

    def tree(self, b):
        return b.export_tree() + (np.float32(b.max_priority),)

    def append(self, b, rows, n):
        b.insert(self.dev(rows))

    def state(self, b):
        return int(b.count), int(b.head)

    def gather(self, b, idx):
        return [f.cpu().numpy() for f in b.sample(indices=self.torch.from_numpy(idx).cuda())]

    def newest(self, b):
        return [f.cpu().numpy() for f in b.get_item(-1)]

    def storage(self, b, f):
        return b.buffer[f].cpu().numpy()


def run_per_fixture(side):
    g = np.load(os.path.join(GOLD, "per_config1_small.npz"))
    cap, batch, steps = int(g["cap"]), int(g["batch"]), int(g["steps"])
    b = side.per(float(g["alpha"]), cap, batch)
    side.push(b, [g["fill_%d" % f] for f in range(5)], cap)
    for t in range(steps):
        idx, w, rows = side.sample(b, batch, float(g["beta"]), g["uniforms"][t])
        assert np.array_equal(idx, g["indices"][t]), t
        assert same_bits(w, g["weights"][t]), t
        for f in range(5):
            assert same_bits(rows[f], g["gathered_%d" % f][t]), (t, f)
        side.update(b, g["indices"][t], g["td"][t])
        side.push(b, [g["new_%d" % f][t][None] for f in range(5)], 1)
    s, m, mp = side.tree(b)
    assert same_bits(s[1:], g["sum_heap"][1:]) and same_bits(m[1:], g["min_heap"][1:])
    assert mp == g["max_priority"]


def run_urb_fixture(side):
    g = np.load(os.path.join(GOLD, "urb_ring_small.npz"))
    b = side.urb(int(g["cap"]))
    for step, n in enumerate(g["sizes"]):
        if n == 0:
            b.reset()
        else:
            side.append(b, [g["rows_%d_%d" % (step, f)] for f in range(3)], int(n))
        assert side.state(b) == (int(g["count_%d" % step]), int(g["head_%d" % step])), step
        if ("idx_%d" % step) in g:
            for f, a in enumerate(side.gather(b, g["idx_%d" % step])):
                assert same_bits(a, g["gather_%d_%d" % (step, f)]), (step, f)
            for f, a in enumerate(side.newest(b)):
                assert same_bits(a, g["newest_%d_%d" % (step, f)]), (step, f)
    for f in range(3):
        assert same_bits(side.storage(b, f), g["storage_%d" % f])


def test_oracle_reproduces_per_fixture(orc):
    run_per_fixture(OracleSide(orc))


def test_oracle_reproduces_urb_fixture(orc):
    run_urb_fixture(OracleSide(orc))


def test_oracle_reproduces_powf_vectors(orc):
    g = np.load(os.path.join(GOLD, "powf_vectors.npz"))
    for key in g.files:
        if key.startswith("pow_"):
            assert same_bits(orc.powf_array(g["x"], float(key[4:])), g[key]), key


@pytest.mark.gpu
def test_hip_reproduces_per_fixture():
    run_per_fixture(HipSide())


@pytest.mark.gpu
def test_hip_reproduces_urb_fixture():
    run_urb_fixture(HipSide())
