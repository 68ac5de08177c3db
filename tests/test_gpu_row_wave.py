"""The wave-per-row sample kernel (k_per_sample_rows: one wave walks the tree, copies its row and takes the
importance weight) against the oracle: it is chosen for launches of at least 2048 rows of up to a few kilobytes;
here the buffer option "row_wave" = 1 forces it at every size, and the parity scenarios of test_gpu_parity.py are
rerun with it, plus launches large enough to take it on their own."""
import numpy as np
import pytest
import torch

import test_gpu_parity as tg
from gpu_util import assert_sample_equal, random_rows, to_dev, torch_types

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mrb_rows():
    if not torch.cuda.is_available():
        pytest.fail("no HIP device: the GPU parity tests cannot run (there is no CPU fallback)")
    from mindrl_amd import _lib
    from mindrl_amd.core import PriorityReplayBuffer, ReservoirReplayBuffer, UniformReplayBuffer
    _lib.lib()

    def per(*args, **kwargs):
        b = PriorityReplayBuffer(*args, **kwargs)
        b.set_option("row_wave", 1)
        return b

    class NS:
        pass

    ns = NS()
    ns.lib, ns.PER, ns.URB, ns.RES = _lib, per, UniformReplayBuffer, ReservoirReplayBuffer
    yield ns


@pytest.mark.parametrize("fused", [1])
@pytest.mark.parametrize("cap", [1, 2, 5, 100, 4096, 5000, 70000, 300000])
def test_row_wave_per_random_ops_bit_exact(mrb_rows, orc, cap, fused):
    tg.test_per_random_ops_bit_exact(mrb_rows, orc, cap, 1, fused)


def test_row_wave_sixteen_narrow_fields(mrb_rows, orc):
    """sixteen fields of 1 .. 100 bytes: more than four narrow fields, more than 128 narrow bytes"""
    tg.test_sixteen_fields_of_odd_sizes(mrb_rows, orc, 1, sizes=[1, 2, 3, 4, 6, 8, 12, 16, 20, 24, 48, 100, 5, 9, 10, 7])


@pytest.mark.parametrize("shape", range(3))
def test_row_wave_sample_many(mrb_rows, orc, shape):
    tg.test_sample_many_equals_successive_samples(mrb_rows, orc, shape)


def test_row_wave_config1_loop(mrb_rows, orc):
    tg.test_config1_dqn_per_cartpole_full_loop(mrb_rows, orc)


def test_row_wave_config4(mrb_rows, orc):
    tg.test_config4_apex_high_churn(mrb_rows, orc)


def test_row_wave_graph_replay(mrb_rows, orc):
    tg.test_hip_graph_replays_a_whole_loop_with_device_counters(mrb_rows, orc, 70000, 1)
    tg.test_hip_graph_replays_update_and_sample(mrb_rows, orc, 1)


def test_row_wave_out_of_domain(mrb_rows, orc):
    tg.test_out_of_domain_inputs_are_clamped_and_flagged(mrb_rows, orc, 1)


@pytest.mark.parametrize("cap,shapes,dtypes", [
    (3000, [(4,), (1,), (1,), (4,), (1,)], [np.float32, np.int32, np.float32, np.float32, np.bool_]),  # 12 levels, 41 B rows
    (1_000_000, [(17,), (6,), (1,), (17,), (1,)], [np.float32, np.float32, np.float32, np.float32, np.bool_]),  # 20 levels
    (1 << 21, [(64,), (1,), (1,), (64,), (1,)], [np.float32, np.int32, np.float32, np.float32, np.bool_]),  # 21 levels, 521 B
    (5_000_000, [(256,), (3,)], [np.float32, np.uint8]),  # 23 levels, one 1 KB field
])
def test_large_launches_take_the_row_wave_kernel_on_their_own(orc, cap, shapes, dtypes):
    """No option set: one batch of 2500 rows and eight batches of 300 in one launch (2400 rows) go to the
    wave-per-row kernel, a batch of 300 to the workgroup kernel; all equal the oracle's samples."""
    from mindrl_amd.core import PriorityReplayBuffer
    rng = np.random.default_rng(cap % 1000)
    fill = min(cap, 200_000)
    big = PriorityReplayBuffer(0.6, cap, 2500, shapes, torch_types(dtypes), seed0=4)
    small = PriorityReplayBuffer(0.6, cap, 300, shapes, torch_types(dtypes), seed0=4)
    cb = orc.OraclePER(0.6, cap, shapes, dtypes, seed=4)
    cs = orc.OraclePER(0.6, cap, shapes, dtypes, seed=4)
    rows = random_rows(rng, fill, shapes, dtypes)
    pr = (rng.pareto(1.5, fill) + 1e-6).astype(np.float32)
    dev = to_dev(rows)
    for g, c in ((big, cb), (small, cs)):
        g.insert(*dev, priorities=torch.from_numpy(pr).cuda()), c.push(rows, fill, pr)
    for rep in range(2):
        u = rng.random(2500).astype(np.float32)
        assert_sample_equal(big.sample(0.5, uniforms=torch.from_numpy(u).cuda()), cb.sample(2500, 0.5, u), "2500 rows, given draws")
        assert_sample_equal(big.sample(0.5), cb.sample(2500, 0.5), "2500 rows, generator")
        um = rng.random((8, 300)).astype(np.float32)
        got = small.sample_many(8, 0.7, uniforms=torch.from_numpy(um).cuda())
        for i in range(8):
            assert_sample_equal([x[i] for x in got], cs.sample(300, 0.7, um[i]), "batch %d of 8" % i)
        assert_sample_equal(small.sample(0.7), cs.sample(300, 0.7), "300 rows")
    assert big.check() in (0, 8) and small.check() in (0, 8)
    big.destroy(), small.destroy()
