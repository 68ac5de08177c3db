"""CPU-only checks of the product's host side: the C-ABI library loads and
exports every symbol include/mrb.h declares, argument validation that needs no
device, and the Python-side layout logic. No kernel is launched here."""
import ctypes as C
import os
import re

import numpy as np
import pytest
import torch

from mindrl_amd import _lib
from mindrl_amd.core._rows import FieldLayout
from mindrl_amd.dtype import as_torch_dtype

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "mrb.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mrb_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_symbols()
    assert len(names) == 47
    L = _lib.lib()
    for n in names:
        assert hasattr(L, n), "libmrb.so does not export %s" % n
    assert set(_lib.SIGNATURES) | {"mrb_last_error"} == set(names)
    assert L.mrb_backend() == 1 and L.mrb_version() == _lib.ABI_VERSION == 4


def test_status_codes_without_a_device():
    L = _lib.lib()
    assert L.mrb_urb_state(123456, None, None) == _lib.MRB_EHANDLE
    assert b"123456" in L.mrb_last_error()
    assert L.mrb_per_destroy(42) == _lib.MRB_EHANDLE
    assert L.mrb_set_option(42, b"row_split", 0) == _lib.MRB_EHANDLE  # options belong to a buffer
    h = C.c_int64(0)
    fb = (C.c_int64 * 1)(4)
    assert L.mrb_urb_create(0, 1, fb, C.byref(h)) == _lib.MRB_EINVAL
    assert L.mrb_urb_create(10, 0, fb, C.byref(h)) == _lib.MRB_EINVAL
    assert L.mrb_urb_create(10, 17, fb, C.byref(h)) == _lib.MRB_EINVAL
    assert L.mrb_per_create(10, C.c_float(-1.0), 1, fb, 0, C.byref(h)) == _lib.MRB_EINVAL
    with pytest.raises(ValueError):
        _lib.check(_lib.MRB_EINVAL)


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the no-device failure mode")
def test_buffers_fail_loudly_without_a_device():
    from mindrl_amd.core import PriorityReplayBuffer, UniformReplayBuffer
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        UniformReplayBuffer(4, 10, [(1,)], [torch.float32])
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        PriorityReplayBuffer(0.6, 10, 4, [(1,)], [torch.float32])


def test_missing_library_is_an_error(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libmrb.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.lib()


def test_field_layout():
    lay = FieldLayout([(84, 84, 4), (1,), 1, (1,), (1,)], [np.uint8, "int64", torch.int32, "mindspore.float32", bool])
    assert lay.bytes == [28224, 8, 4, 4, 1] and sum(lay.bytes) == 28241
    assert lay.dtypes == [torch.uint8, torch.int64, torch.int32, torch.float32, torch.bool]
    assert lay.batch_of([torch.zeros(84, 84, 4), torch.zeros(1), torch.zeros(1), torch.zeros(1), torch.zeros(1)]) == 1
    assert lay.batch_of([torch.zeros(5, 84, 84, 4)] + [torch.zeros(5, 1)] * 4) == 5
    with pytest.raises(ValueError):
        lay.batch_of([torch.zeros(5, 84, 84, 4)] + [torch.zeros(4, 1)] * 4)
    with pytest.raises(ValueError):
        lay.batch_of([torch.zeros(1)])
    with pytest.raises(ValueError):
        FieldLayout([(1,)] * 17, [np.float32] * 17)
    with pytest.raises(TypeError):
        as_torch_dtype("complex64")


def test_kernels_use_no_scratch_memory(tmp_path):
    """Register arrays that the compiler cannot keep in registers end up in scratch
    (or LDS) and slow the sample kernel by 2x; the device assembly's metadata must show
    private_segment_fixed_size 0 for every kernel and the expected LDS sizes."""
    import subprocess
    from mindrl_amd import build
    out = tmp_path / "mrb.s"
    flags = [f for f in build.HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    res = subprocess.run(["/opt/rocm/bin/hipcc"] + flags + ["--cuda-device-only", "-S", "-o", str(out),
                          os.path.join(build.CSRC, "mrb.hip")], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                         text=True)
    assert res.returncode == 0, res.stdout
    text = out.read_text()
    kernels = {}
    for block in text.split("  - .agpr_count:")[1:]:
        name = re.search(r"\.name:\s+(\S+)", block).group(1)
        kernels[name] = (int(re.search(r"\.private_segment_fixed_size:\s+(\d+)", block).group(1)),
                         int(re.search(r"\.group_segment_fixed_size:\s+(\d+)", block).group(1)),
                         int(re.search(r"\.vgpr_count:\s+(\d+)", block).group(1)))
    assert sum("k_per_sample_wide" in k for k in kernels) == 8 and sum("k_rows_gather_wide" in k for k in kernels) == 4
    assert len(kernels) == 55, sorted(kernels)
    for name, (scratch, lds, vgprs) in kernels.items():
        assert scratch == 0, "%s uses %d bytes of scratch per lane" % (name, scratch)
        assert vgprs <= 128, (name, vgprs)
        if "k_per_sample_wide" in name or "k_rows_gather_wide" in name:
            assert lds <= 256, (name, lds)  # a private array turned into LDS would show here
        if "k_tree_update" in name:
            assert lds == 8192, (name, lds)  # the election words (256 x 8 B per wave) and nothing else
        if "k_tree_wg" in name:
            # the staged top of both trees, three hash tables (+ the position word of the device-counter variant)
            base = 2 * 4096 * 4 + 3 * 2048 * 12
            if "push_sample" in name:
                # the whole-step kernel: also a slot per thread (512 or 1024), two field tables, a few words handed over
                threads = 1024 if "Li1024E" in name else 512
                assert threads * 8 + 2 * 648 <= lds - base <= threads * 8 + 2 * 648 + 128, (name, lds)
            else:
                assert lds == base + (8 if "pushILb1E" in name else 0), (name, lds)
    # The whole-step kernel reads the kernel-argument segment with vector loads only (a scalar read in flight would
    # hold up its barriers' waits for LDS): past the loads that stand in for the preloaded arguments on firmware
    # without preloading - they end with a branch to the kernel proper - its code holds no scalar load.
    steps = re.findall(r"^(_ZN3mrb21k_tree_wg_push_sample\w+):[^\n]*\n(.*?)^\.Lfunc_end", text, re.S | re.M)
    assert len(steps) == 4, "the four instantiations of k_tree_wg_push_sample in the assembly"
    for name, body in steps:
        code = [l.strip() for l in body.splitlines() if l.startswith("\t") and not l.strip().startswith((".", ";"))]
        first_branch = next(i for i, l in enumerate(code) if l.startswith("s_branch"))
        assert first_branch < 8 and all(l.startswith(("s_load", "s_waitcnt")) for l in code[:first_branch]), (name, code[:8])
        late = [l for l in code[first_branch:] if l.startswith(("s_load", "s_buffer_load"))]
        assert not late, (name, late[:4])


def test_only_the_documented_entry_points_wait_or_allocate():
    """include/mrb.h promises that only create / destroy / state / check / export_tree wait for the device and
    that only create allocates (mrb_per_update may enlarge its scratch, never free it). Checked on the source:
    the body of every other extern "C" function, and of the helpers they share, names no such call."""
    src = open(os.path.join(ROOT, "mindrl_amd", "csrc", "mrb.hip")).read()
    bodies = {}
    for m in re.finditer(r"^(?:static )?(?:int|void|uint32_t|int64_t|const char\*) (\w+)\([^;{]*\)\s*\{\n(.*?)^\}", src, re.M | re.S):
        bodies[m.group(1)] = m.group(2)
    one_liners = {"mrb_last_error", "mrb_backend", "mrb_version"}  # return a constant
    assert {n for n in bodies if n.startswith("mrb_")} == set(declared_symbols()) - one_liners, sorted(bodies)
    waits = re.compile(r"hipDeviceSynchronize|hipStreamSynchronize|hipEventSynchronize|hipMemcpy\(")
    allocs = re.compile(r"hipMalloc|hipFree|hipHostMalloc")
    may_wait = {"mrb_urb_create", "mrb_per_create", "mrb_res_create", "mrb_urb_destroy", "mrb_per_destroy",
                "mrb_res_destroy", "mrb_per_state", "mrb_per_export_tree", "read_and_clear_flags", "rows_alloc",
                "counters_to_device", "counters_from_device"}
    may_alloc = {"mrb_urb_create", "mrb_per_create", "mrb_res_create", "rows_alloc", "mrb_per_update"}  # (mrb_per_update_push calls it)
    for name, body in bodies.items():
        if name not in may_wait:
            assert not waits.search(body), "%s waits for the device" % name
        if name not in may_alloc:
            assert not allocs.search(body), "%s allocates or frees device memory" % name
    assert "hipFree" not in bodies["mrb_per_update"]
    # the check functions wait through this helper and nothing else does
    users = [n for n, b in bodies.items() if "read_and_clear_flags(" in b]
    assert sorted(users) == ["mrb_per_check", "mrb_urb_check"]
    # device-resident counters are copied (with a wait) only where the header says so: switching the option,
    # state queries and the checkpoint calls - never by push, sample or update
    users = {n for n, b in bodies.items() if re.search(r"counters_(to|from)_device\(", b)}
    assert users == {"mrb_set_option", "mrb_per_state", "mrb_per_get_counters", "mrb_per_set_counters", "mrb_urb_state",
                     "mrb_urb_reset", "mrb_urb_seed", "mrb_urb_get_counters", "mrb_urb_set_counters"}, users
    # the allocation-free entry point and the core it shares with mrb_per_update
    for name in ("mrb_per_update_noalloc", "per_update", "tree_rebuild", "next_epoch", "static_scratch"):
        assert not allocs.search(bodies[name]) and not waits.search(bodies[name]), name


def test_create_replay_buffer_follows_the_reference_config_entry():
    """mindspore_rl/core/msrl.py:270-300: type / number / params-or-(sample_size, capacity) + data_shape / data_type."""
    from mindrl_amd.core import create_replay_buffer

    class Fake:
        def __init__(self, sample_size, capacity, shapes, types):
            self.args = (sample_size, capacity, shapes, types)

    cfg = {"number": 1, "type": Fake, "capacity": 100000, "sample_size": 64,
           "data_shape": [(4,), (1,)], "data_type": ["float32", "int32"]}
    one = create_replay_buffer(cfg)
    assert one.args == (64, 100000, ((4,), (1,)), ("float32", "int32"))
    many = create_replay_buffer(dict(cfg, number=3))
    assert len(many) == 3 and all(isinstance(m, Fake) for m in many)
    with_params = create_replay_buffer({"type": Fake, "params": {"sample_size": 2, "capacity": 5},
                                        "data_shape": [(1,)], "data_type": ["float32"]})
    assert with_params.args == (2, 5, ((1,),), ("float32",))
    default_size = create_replay_buffer({"type": Fake, "capacity": 7, "data_shape": [(1,)], "data_type": ["int32"]})
    assert default_size.args[0] == 1
    params = {"sample_size": 2, "capacity": 5}
    create_replay_buffer({"type": Fake, "params": params, "data_shape": [(1,)], "data_type": ["float32"]})
    assert params == {"sample_size": 2, "capacity": 5}  # the caller's dict is not written to
    for bad in ({"capacity": 7, "data_shape": [(1,)], "data_type": ["int32"]},               # no type
                {"type": Fake, "capacity": 7, "data_type": ["int32"]},                        # no data_shape
                {"type": Fake, "capacity": 7, "data_shape": [(1,)], "data_type": ["int32"], "sampel_size": 3}):
        with pytest.raises(KeyError):
            create_replay_buffer(bad)
    with pytest.raises(ValueError):
        create_replay_buffer(dict(cfg, number=0))


def test_replay_buffer_set_binds_the_handlers_msrl_binds():
    """mindspore_rl/core/msrl.py:407-421: one buffer -> replay_buffer_sample/insert/full/reset bound to it;
    `number` > 1 -> a list and nothing bound; `multi_type_replaybuffer` -> a dict of named buffers."""
    from mindrl_amd.core import ReplayBufferSet

    class Fake:
        def __init__(self, sample_size, capacity, shapes, types):
            self.capacity, self.rows = capacity, []

        def insert(self, row):
            self.rows.append(row)

        def sample(self):
            return self.rows[-1]

        def full(self):
            return len(self.rows) >= self.capacity

        def reset(self):
            self.rows = []

    entry = {"number": 1, "type": Fake, "capacity": 2, "sample_size": 1, "data_shape": [(1,)], "data_type": ["int32"]}
    one = ReplayBufferSet(entry)
    one.replay_buffer_insert(5), one.replay_buffer_insert(6)
    assert one.replay_buffer_sample() == 6 and one.replay_buffer_full() and isinstance(one.buffers, Fake)
    one.replay_buffer_reset()
    assert one.buffers.rows == []
    assert isinstance(ReplayBufferSet({k: v for k, v in entry.items() if k != "number"}).buffers, Fake)  # number defaults to 1
    several = ReplayBufferSet(dict(entry, number=2))
    assert isinstance(several.buffers, list) and len(several.buffers) == 2 and not hasattr(several, "replay_buffer_sample")
    named = ReplayBufferSet({"multi_type_replaybuffer": True, "policy": entry, "expert": dict(entry, capacity=9)})
    assert set(named.buffers) == {"policy", "expert"} and named.buffers["expert"].capacity == 9
    assert not hasattr(named, "replay_buffer_insert")
    with pytest.raises(TypeError):
        ReplayBufferSet([entry])


def test_bench_refuses_more_than_one_gpu():
    """Every box has one GPU: `bench.py --gpus N` with N > 1 exits non-zero with a message, before touching a device."""
    import subprocess
    import sys
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE,
                         stderr=subprocess.PIPE, text=True, timeout=120)
    assert res.returncode != 0 and "one GPU" in res.stderr and res.stdout.strip() == ""
