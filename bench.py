#!/usr/bin/env python3
"""Replay-buffer hot-path benchmark on one MI355X.

A step is one pass of the hot path over one batch. The default workload is the benchmark's config 3:
PriorityReplayBuffer.sample (stratified sum-tree descent + importance weights + row gather) on the
Atari-shaped buffer of capacity 1,000,000 (28,241 stored bytes per row, batch 512), one C-ABI call
per step on one stream, every call ordered after the one before it. Inputs are synthetic and resident
in HBM before the timed region; the sampling uniforms are drawn on the host beforehand, one set per step.

Prints ONE JSON line. `roofline` prices the dominant kernel's algorithmic bytes against the HBM peak with
the launch duration measured by HIP events over the timed region; `cpu_baseline` is the CPU oracle
(a sequential C restatement of the reference path) timed on this machine's host cores on a bounded
sample of the same workload. Other workloads: c1 (DQN-PER loop), c2 (uniform buffer gather), c4, c5
(prioritized, narrow rows), res (reservoir), dr (discounted return).
"""
import argparse
import ctypes as C
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

PER_WORKLOADS = {
    # name: (capacity, batch, shapes, numpy dtypes, update n, insert n, description)
    "c1": (10_000, 64, [(4,), (1,), (1,), (4,), (1,)], ["float32", "int32", "float32", "float32", "bool"], 64, 1,
           "config 1: DQN-PER CartPole-shaped PriorityReplayBuffer, capacity 10,000, 41 B rows; step = sample 64 + "
           "update_priorities 64 + insert 1"),
    "c3": (1_000_000, 512, [(84, 84, 4), (1,), (1,), (1,), (1,)], ["uint8", "int64", "int32", "float32", "bool"],
           512, 4, "config 3: Atari-shaped PriorityReplayBuffer, capacity 1,000,000, 28,241 B stored rows "
                   "(obs u8[84,84,4] + next_idx i64 + action i32 + reward f32 + done bool), batch 512"),
    "c4": (1 << 21, 1024, [(64,), (1,), (1,), (64,), (1,)], ["float32", "int32", "float32", "float32", "bool"],
           2048, 4096, "config 4: Ape-X PriorityReplayBuffer, capacity 2,097,152, 521 B rows, batch 1024"),
    "c5": (1 << 24, 65536, [(1,), (1,)], ["int32", "float32"], 65536, 4096,
           "config 5: tree-descent stress, capacity 16,777,216, 8 B rows, batch 65,536"),
}
WORKLOAD_CAP = {k: v[0] for k, v in PER_WORKLOADS.items()}
# the rocprofv3 summary that holds the tracked figures of a workload's dominant kernel
PROFILE_OF = {
    "c3": "k_per_sample_wide_config3_atari_cap1M_batch512.md",
    "c5": "k_per_sample_lds_and_tree_update_config5_2pow24_batch65536.md",
}


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=2000)
    p.add_argument("--warmup", type=int, default=200)
    p.add_argument("--workload", default="c3", choices=sorted(PER_WORKLOADS) + ["c2", "res", "dr"])
    p.add_argument("--capacity", type=int, default=0, help="override the workload's capacity (for quick trials)")
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--graph", action="store_true", help="replay the timed steps as one captured HIP graph")
    p.add_argument("--row-split", type=int, default=0, help="workgroups per sampled row (0 = library default)")
    p.add_argument("--sample-path", type=int, default=0, help="0 auto, 1 wide-row kernel, 2 LDS-top kernel")
    p.add_argument("--packed-rows", type=int, default=0,
                   help="keep rows of at most this many bytes packed in one array (library option packed_rows; 0 = "
                        "one array per field, the reference's layout)")
    p.add_argument("--no-extras", action="store_true",
                   help="skip the untimed side figures (update, insert, loop, graph replay, several streams)")
    p.add_argument("--settle-ms", type=float, default=300.0,
                   help="untimed calls of the step for this long before the warm-up steps, so that a short timed "
                        "region is not measured on a GPU that is still raising its clocks after the host-side set-up")
    return p.parse_args()


def kernel_sources_sha16():
    """First 16 hex digits of the SHA-256 of the library's kernel sources: names the build a profile was taken of."""
    import hashlib
    h = hashlib.sha256()
    for name in ("mrb_device.h", "mrb_kernels.h", "mrb.hip"):
        with open(os.path.join(ROOT, "mindrl_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def profile_figures(workload):
    """Figures of the committed rocprofv3 summary of this workload's dominant kernel (lines `key: value`
    in its "figures" block), or {} if the summary is not there or was taken of other kernel sources than the
    ones in this tree (its `kernel_sources_sha16` line): a stale profile prices nothing."""
    name = PROFILE_OF.get(workload)
    path = os.path.join(ROOT, "profiles", name) if name else None
    if not path or not os.path.exists(path):
        return {}, name
    text = open(path).read()
    sha = re.search(r"^\s*kernel_sources_sha16:\s*([0-9a-f]{16})\s*$", text, re.M)
    if not sha or sha.group(1) != kernel_sources_sha16():
        return {"stale": True}, name
    out = {}
    for key, val in re.findall(r"^\s*(rocprof_avg_ns|traffic_bytes_per_launch):\s*([0-9.eE+]+)\s*$", text, re.M):
        out[key] = float(val)
    return out, name


def roofline(kernel, algo_bytes, kern_s, wall_s_per_step, workload, formula, defaults=True):
    """achieved = algorithmic bytes per launch / average launch duration (HIP events over the timed
    region); frac_wall prices the same bytes with the host's wall clock per step. The rocprofv3 average
    and the counter-measured HBM traffic cannot be measured inside this process: they are read from the
    committed summary of this very command, and left out (null) when the run is not the default one."""
    fig, name = profile_figures(workload) if defaults else ({}, PROFILE_OF.get(workload))
    achieved = algo_bytes / kern_s / 1e9
    r = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
         "traffic": fig.get("traffic_bytes_per_launch"), "kernel": kernel, "algorithmic_bytes_per_launch": algo_bytes,
         "algorithmic_bytes": formula, "avg_launch_us": kern_s * 1e6,
         "frac_wall": algo_bytes / wall_s_per_step / 1e9 / HBM_PEAK_GBS, "profile": name}
    if fig.get("stale"):
        r["profile_note"] = "the committed profile was taken of other kernel sources: traffic and profiler figures left out"
    if "rocprof_avg_ns" in fig:
        r["rocprof_avg_us"] = fig["rocprof_avg_ns"] * 1e-3
        r["frac_kernel_rocprof"] = algo_bytes / (fig["rocprof_avg_ns"] * 1e-9) / 1e9 / HBM_PEAK_GBS
    return r


def fill_per(buf, torch, capacity, shapes, np_dtypes, seed, lognormal=True):
    """Prefill to capacity in chunks (rows generated on the device), then set the priorities."""
    gen = torch.Generator(device="cuda").manual_seed(seed)
    row_bytes = sum(int(np.prod(s)) * np.dtype(d).itemsize for s, d in zip(shapes, np_dtypes))
    chunk = max(1, min(capacity, (256 << 20) // row_bytes))
    done = 0
    while done < capacity:
        n = min(chunk, capacity - done)
        fields = []
        for s, d in zip(shapes, np_dtypes):
            d = np.dtype(d)
            if d == np.uint8:
                fields.append(torch.randint(0, 256, (n,) + tuple(s), dtype=torch.uint8, device="cuda", generator=gen))
            elif d == np.bool_:
                fields.append(torch.rand((n,) + tuple(s), device="cuda", generator=gen) < 0.01)
            elif d.kind == "f":
                fields.append(torch.randn((n,) + tuple(s), device="cuda", generator=gen))
            elif d == np.int64:
                fields.append(((torch.arange(done, done + n, device="cuda") + 1) % capacity).reshape((n,) + tuple(s)))
            else:
                fields.append(torch.randint(0, 18, (n,) + tuple(s), dtype=torch.int32, device="cuda", generator=gen))
        buf.insert(*fields)
        done += n
    if lognormal:
        rng = np.random.default_rng(seed)
        pr = rng.lognormal(0.0, 1.0, capacity).astype(np.float32)
        buf.update_priorities(torch.arange(capacity, device="cuda"), torch.from_numpy(pr).cuda())
    torch.cuda.synchronize()


def host_mem_available():
    """MemAvailable of /proc/meminfo in bytes (0 if it cannot be read)."""
    try:
        for line in open("/proc/meminfo"):
            if line.startswith("MemAvailable:"):
                return int(line.split()[1]) * 1024
    except OSError:
        pass
    return 0


def oracle_per(workload, shapes, np_dtypes, seed, lognormal=True):
    """The CPU oracle filled like the GPU buffer, at the workload's full capacity when the host has the memory
    for it (config 3: 10^6 rows of 28 KB are 28 GB of host rows, taken when three times that is available),
    else cut to 131,072 rows (17 tree levels instead of 20, which favours the CPU; the cut is stated in the
    result)."""
    from oracle import orc
    cap = WORKLOAD_CAP[workload]
    row_bytes = sum(int(np.prod(s)) * np.dtype(d).itemsize for s, d in zip(shapes, np_dtypes))
    if cap * row_bytes > (1 << 30) and host_mem_available() < 3 * cap * row_bytes:
        cap = min(cap, 1 << 17)
    rng = np.random.default_rng(seed)
    per = orc.OraclePER(0.6, cap, shapes, np_dtypes, seed=seed)
    chunk = min(cap, 2048)
    rows = []
    for s, d in zip(shapes, np_dtypes):
        d = np.dtype(d)
        if d == np.uint8:
            rows.append(rng.integers(0, 256, (chunk,) + tuple(s), dtype=np.uint8))
        elif d == np.bool_:
            rows.append(rng.random((chunk,) + tuple(s)) < 0.01)
        else:
            rows.append(rng.integers(0, 3, (chunk,) + tuple(s)).astype(d))
    for start in range(0, cap, chunk):
        n = min(chunk, cap - start)
        per.push([r[:n] for r in rows], n)
    if lognormal:
        for start in range(0, cap, 1 << 20):
            n = min(1 << 20, cap - start)
            per.update(np.arange(start, start + n), rng.lognormal(0, 1, n).astype(np.float32))
    return per, cap, rows


def cpu_baseline_sample(workload, shapes, np_dtypes, batch, seed):
    """orc_per_sample (descent + weights + row copies) on one thread, and with the row copies on all cores."""
    from oracle import orc
    per, cap, _ = oracle_per(workload, shapes, np_dtypes, seed)
    rng = np.random.default_rng(seed + 7)
    L = orc.lib()
    idx = np.empty(batch, np.int64)
    w = np.empty(batch, np.float32)
    dst = per._dst(batch)
    dptr = orc._ptr_array(dst)
    u_all = rng.random((64, batch)).astype(np.float32)

    def timed(seconds):
        calls, t_end = 0, time.perf_counter() + seconds
        t0 = time.perf_counter()
        while time.perf_counter() < t_end:
            u = u_all[calls % 64]
            rc = L.orc_per_sample(per.h, batch, 0.4, u.ctypes.data, idx.ctypes.data, w.ctypes.data, dptr)
            assert rc == 0
            calls += 1
        return calls, time.perf_counter() - t0

    calls, dt = timed(10.0)
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = max(1, min(cores, 16))
    orc.set_threads(cores)
    calls_mt, dt_mt = timed(4.0)
    orc.set_threads(1)
    cut = " (cut from %d: the host lacks the memory for the rows)" % WORKLOAD_CAP[workload] if cap != WORKLOAD_CAP[workload] else ""
    return {
        "value": calls * batch / dt, "unit": "transitions/s", "cores": 1, "kind": "port",
        "sample": "%d sample calls (batch %d, same row shape) in %.1f s on a capacity-%d buffer%s, 1 thread" % (
            calls, batch, dt, cap, cut),
        "all_cores": {"value": calls_mt * batch / dt_mt, "cores": cores,
                      "sample": "%d calls in %.1f s, row copies on %d OpenMP threads" % (calls_mt, dt_mt, cores)},
    }


def cpu_baseline_loop(workload, shapes, np_dtypes, batch, upd_n, ins_n, seed):
    """The same sample + update_priorities + insert loop on the oracle, one thread."""
    from oracle import orc
    per, cap, rows = oracle_per(workload, shapes, np_dtypes, seed, lognormal=False)
    rng = np.random.default_rng(seed + 7)
    L = orc.lib()
    idx = np.empty(batch, np.int64)
    w = np.empty(batch, np.float32)
    dst = per._dst(batch)
    dptr = orc._ptr_array(dst)
    u_all = rng.random((64, batch)).astype(np.float32)
    upd = min(upd_n, batch)
    pr_all = (np.abs(rng.normal(size=(64, upd_n))) + 1e-6).astype(np.float32)
    src = [np.ascontiguousarray(r[:ins_n]) for r in rows]
    sptr = orc._ptr_array(src)
    steps, t_end = 0, time.perf_counter() + 10.0
    t0 = time.perf_counter()
    while time.perf_counter() < t_end:
        for _ in range(64):
            i = steps % 64
            L.orc_per_sample(per.h, batch, 0.4, u_all[i].ctypes.data, idx.ctypes.data, w.ctypes.data, dptr)
            L.orc_per_update(per.h, idx.ctypes.data, pr_all[i].ctypes.data, upd)
            L.orc_per_push(per.h, sptr, ins_n, None)
            steps += 1
    dt = time.perf_counter() - t0
    return {"value": steps / dt, "unit": "steps/s", "cores": 1, "kind": "port",
            "sample": "%d steps of sample %d + update %d + insert %d in %.1f s on a capacity-%d buffer, 1 thread" % (
                steps, batch, upd, ins_n, dt, cap)}


def events(torch):
    return torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)


class PerRun:
    """One prioritized buffer filled for a workload, with the C-ABI calls of its step bound to device buffers."""

    def __init__(self, a, torch):
        from mindrl_amd import _lib
        from mindrl_amd.core import PriorityReplayBuffer
        from mindrl_amd.core._rows import pointers

        self.torch, self._lib, self.pointers = torch, _lib, pointers
        self.capacity, self.batch, self.shapes, self.np_dtypes, self.upd_n, self.ins_n, self.desc = PER_WORKLOADS[a.workload]
        if a.capacity:
            self.capacity = a.capacity
            self.desc += " [capacity overridden to %d]" % a.capacity
        self.loop_step = a.workload == "c1"  # config 1's step is the whole loop, the others time sample()
        self.seed = 1000 + int(a.workload[1])
        self.buf = PriorityReplayBuffer(0.6, self.capacity, self.batch, self.shapes,
                                        [getattr(torch, d) for d in self.np_dtypes], seed0=self.seed,
                                        packed_rows=a.packed_rows)
        if a.packed_rows:
            packed = not self.buf.storage()[0].is_contiguous()
            self.desc += " [rows packed in one array]" if packed else " [packed rows asked for, row too wide]"
        self.buf.set_option("row_split", a.row_split)
        self.buf.set_option("sample_path", a.sample_path)
        t0 = time.perf_counter()
        fill_per(self.buf, torch, self.capacity, self.shapes, self.np_dtypes, self.seed, lognormal=not self.loop_step)
        self.fill_s = time.perf_counter() - t0
        self.K, self.W = a.steps, a.warmup
        # draws for the timed steps and, beyond them, for the untimed side figures (which take their own step
        # counts, so that a short timed run does not make them noisy)
        n, batch = max(self.K + self.W, 1200), self.batch
        self.n_draws = n
        self.rng = np.random.default_rng(self.seed + 1)
        self.uniforms = torch.from_numpy(self.rng.random((n, batch)).astype(np.float32)).cuda()
        self.betas = np.resize((np.linspace(0.4, 1.0, self.K + self.W) if a.workload == "c3"
                                else np.full(self.K + self.W, 0.4)).astype(np.float32), n)
        self.idx = torch.empty(batch, dtype=torch.int64, device="cuda")
        self.wts = torch.empty(batch, dtype=torch.float32, device="cuda")
        self.fields = self.buf._layout.empty(batch, self.buf._dev)
        self.fptr = pointers(self.fields)
        self.L = _lib.lib()
        self.stream = torch.cuda.current_stream()
        self.sp = C.c_void_p(self.stream.cuda_stream)
        self.h = self.buf._h
        self.upd = min(self.upd_n, batch)
        self.upr = torch.from_numpy((np.abs(self.rng.normal(size=(64, self.upd_n))) + 1e-6).astype(np.float32)).cuda()
        ins_n = self.ins_n
        self.src = [f[:ins_n].contiguous() if f.shape[0] >= ins_n else
                    f.repeat((ins_n + f.shape[0] - 1) // f.shape[0], *([1] * (f.dim() - 1)))[:ins_n].contiguous()
                    for f in self.fields]
        self.sptr = pointers(self.src)
        # config 4 inserts its rows at actor-side priorities |N(0,1)| + eps; the others at the running max
        self.ins_prio = (torch.randn(ins_n, device="cuda").abs() + 1e-6) if a.workload == "c4" else None
        self.ins_pr = self.ins_prio.data_ptr() if self.ins_prio is not None else None

    def bind_sample_calls(self):
        """The arguments of every step's sample call, converted once: the timed loop then only makes the calls."""
        base, ip, wp = self.uniforms.data_ptr(), self.idx.data_ptr(), self.wts.data_ptr()
        self._sample_fn = self.L.mrb_per_sample
        self._sample_args = [(self.h, self.batch, float(self.betas[i]), base + i * self.batch * 4, ip, wp, self.fptr, self.sp)
                             for i in range(self.n_draws)]
        self._update_fn, self._push_fn = self.L.mrb_per_update, self.L.mrb_per_push
        self._update_args = [(self.h, ip, self.upr[j].data_ptr(), self.upd, self.sp) for j in range(64)]
        self._push_args = (self.h, self.sptr, self.ins_n, self.ins_pr, self.sp)
        self._update_push_fn = self.L.mrb_per_update_push
        self._update_push_args = [(self.h, ip, self.upr[j].data_ptr(), self.upd, self.sptr, self.ins_n, self.ins_pr, self.sp)
                                  for j in range(64)]
        # the whole step as one call: the update at the indices the previous step sampled, the push, the next sample
        self._step_fn = self.L.mrb_per_update_push_sample
        self._step_args = [(self.h, ip, self.upr[i % 64].data_ptr(), self.upd, self.sptr, self.ins_n, self.ins_pr, self.batch,
                            float(self.betas[i]), base + i * self.batch * 4, ip, wp, self.fptr, self.sp)
                           for i in range(self.n_draws)]

    def sample_bound(self, i):
        if self._sample_fn(*self._sample_args[i]):
            self._lib.check(1)

    def loop_bound(self, i):
        """One step of the config's loop on the bench's stream: sample, update_priorities at the sampled indices, push."""
        if (self._sample_fn(*self._sample_args[i]) or self._update_fn(*self._update_args[i % 64])
                or self._push_fn(*self._push_args)):
            self._lib.check(1)

    def loop_fused_bound(self, i):
        """The same step with update_priorities and the push as ONE call (mrb_per_update_push)."""
        if self._sample_fn(*self._sample_args[i]) or self._update_push_fn(*self._update_push_args[i % 64]):
            self._lib.check(1)

    def loop_one_call_bound(self, i):
        """The same step as ONE call (mrb_per_update_push_sample): the update at the rows the step before sampled,
        the push, and the sample the next step learns from."""
        if self._step_fn(*self._step_args[i]):
            self._lib.check(1)

    def sample(self, i, sp=None, out=None):
        ip, wp, fptr = out if out else (self.idx.data_ptr(), self.wts.data_ptr(), self.fptr)
        rc = self.L.mrb_per_sample(self.h, self.batch, float(self.betas[i]), self.uniforms.data_ptr() + i * self.batch * 4,
                                   ip, wp, fptr, sp or self.sp)
        if rc:
            self._lib.check(rc)

    def loop(self, i, sp=None, fused=False):
        if fused == "one call":  # the whole step as one library call (mrb_per_update_push_sample)
            a = self._step_args[i]
            rc = self._step_fn(*(a[:-1] + (sp or self.sp,)))
            if rc:
                self._lib.check(rc)
            return
        self.sample(i, sp)
        if fused:
            rc = self.L.mrb_per_update_push(self.h, self.idx.data_ptr(), self.upr[i % 64].data_ptr(), self.upd, self.sptr,
                                            self.ins_n, self.ins_pr, sp or self.sp)
        else:
            rc = self.L.mrb_per_update(self.h, self.idx.data_ptr(), self.upr[i % 64].data_ptr(), self.upd, sp or self.sp)
            rc = rc or self.L.mrb_per_push(self.h, self.sptr, self.ins_n, self.ins_pr, sp or self.sp)
        if rc:
            self._lib.check(rc)


def bench_per(a):
    """Configs 1, 3, 4, 5 (prioritized buffers)."""
    import torch

    r = PerRun(a, torch)
    K, W, batch = r.K, r.W, r.batch
    defaults = not (a.capacity or a.row_split or a.sample_path or a.graph or a.packed_rows)
    r.bind_sample_calls()
    step = r.loop_bound if r.loop_step else r.sample_bound
    settle_calls = 0
    if a.settle_ms > 0:
        # not part of the W warm-up steps and not timed: the set-up above leaves the GPU idle for a while
        t_end = time.perf_counter() + a.settle_ms * 1e-3
        while time.perf_counter() < t_end:
            for i in range(100):
                step(i % r.n_draws)
            torch.cuda.synchronize()
            settle_calls += 100
    for i in range(W):
        step(i)
    torch.cuda.synchronize()

    ev0, ev1 = events(torch)
    graph = None
    if a.graph:
        if r.loop_step:
            raise SystemExit("bench.py: --graph captures sample() steps; the config-1 loop advances host-side counters")
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            sp_side = C.c_void_p(side.cuda_stream)
            graph.capture_begin()
            for i in range(W, W + K):
                r.sample(i, sp_side)
            graph.capture_end()
        torch.cuda.synchronize()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev0.record(r.stream)
    if graph is not None:
        graph.replay()
    else:
        for i in range(W, W + K):
            step(i)
    ev1.record(r.stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    dev_s = ev0.elapsed_time(ev1) * 1e-3
    flags = r.buf.check()

    row_bytes = sum(r.buf._layout.bytes)
    levels = max(1, (r.capacity - 1).bit_length())
    # the library's own choice (mrb_per_sample): the LDS-top kernel for many narrow rows, else the wide-row kernel
    lds_path = a.sample_path == 2 or (a.sample_path == 0 and batch >= 8192 and max(r.buf._layout.bytes) <= 256)
    # (rows of at most 4 KB in 16-byte fields: the workgroup kernel with two copy waves, or, for launches of at least
    # 2048 rows, the wave-per-row kernel)
    wide_granules = sum(b // 16 for b in r.buf._layout.bytes if b % 16 == 0)
    narrow_bytes = sum(b for b in r.buf._layout.bytes if b % 16)
    if lds_path:
        kernel_name = "k_per_sample_lds"
    elif wide_granules <= 256 and narrow_bytes <= 256 and batch >= 2048 and not a.row_split:
        kernel_name = "k_per_sample_rows"
    elif wide_granules <= 256 and levels != 22 and not a.row_split:
        kernel_name = "k_per_sample_light"
    else:
        kernel_name = "k_per_sample_wide"
    if a.workload == "c3":
        # rows read + rows written + index (8) + weight (4): the gather-bound headline figure
        algo_bytes, formula = batch * (2 * row_bytes + 12), "batch * (2 * row_bytes + 12)"
    else:
        # narrow rows: the descent's own bytes count too (one left-child sum per level and the leaf)
        algo_bytes = batch * (2 * row_bytes + 12 + 4 * levels + 4)
        formula = "batch * (2 * row_bytes + 12 + 4 * levels + 4), levels = %d" % levels
    if r.loop_step:
        metric, value, unit = "config-1 loop steps/sec (sample 64 + update_priorities 64 + insert 1)", K / wall, "steps/s"
    else:
        metric = ("sampled transitions/sec (sample+IS+gather) at cap 1M; HBM GB/s vs peak" if a.workload == "c3" else
                  "sampled transitions/sec (sample+IS+gather), %s" % r.desc.split(":")[0])
        value, unit = K * batch / wall, "transitions/s"
    out = {
        "metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": wall * 1e3 / K, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8", "data": "synthetic",
        "config": {"workload": r.desc, "capacity": r.capacity, "batch": batch, "row_bytes": row_bytes, "alpha": 0.6,
                   "beta": "0.4->1.0" if a.workload == "c3" else "0.4",
                   "launch": "hip graph replay" if a.graph else "eager C-ABI calls, one stream, in order",
                   "prefill_s": round(r.fill_s, 2), "settle_calls_before_warmup": settle_calls, "device_flags": flags},
    }
    if r.loop_step:
        # the sample kernel's share of a loop step is timed on its own; the loop itself is launch-bound
        for i in range(20):
            r.sample(i)
        torch.cuda.synchronize()
        e0, e1 = events(torch)
        e0.record(r.stream)
        for i in range(K):
            r.sample(W + i)
        e1.record(r.stream)
        torch.cuda.synchronize()
        out["roofline"] = roofline(kernel_name, algo_bytes, e0.elapsed_time(e1) * 1e-3 / K, wall / K, a.workload, formula, defaults)
        out["roofline"]["note"] = ("the loop is bound by kernel launches, not by bytes: frac is the sample kernel alone, "
                                   "frac_wall prices the sample's bytes against a whole loop step")
    else:
        out["roofline"] = roofline(kernel_name, algo_bytes, dev_s / K, wall / K, a.workload, formula, defaults)
    if not a.no_extras:
        out["extras"] = per_extras(a, torch, r, algo_bytes)
        if a.workload == "c3":
            out["roofline"]["floor"] = sample_floor(torch, r, algo_bytes)
            # the same kernel with several batches per launch (mrb_per_sample_many): where the 60 % of peak lie
            many = out["extras"].get("sample_many_batches_per_launch", {})
            out["roofline"]["frac_with_batches_per_launch"] = {k: round(v["frac_of_peak"], 4) for k, v in many.items()}
    if a.no_cpu_baseline:
        out["cpu_baseline"] = None
    elif r.loop_step:
        out["cpu_baseline"] = cpu_baseline_loop(a.workload, r.shapes, r.np_dtypes, batch, r.upd_n, r.ins_n, r.seed)
    else:
        out["cpu_baseline"] = cpu_baseline_sample(a.workload, r.shapes, r.np_dtypes, batch, r.seed)
    r.buf.destroy()
    print(json.dumps(out))
    return 0


def sample_floor(torch, r, algo_bytes):
    """What this machine charges for the pieces of a config-3 sample call, each timed by HIP events over
    back-to-back calls on the bench's stream (us per call): a launch of a kernel that does nothing; the runtime's
    own contiguous device-to-device copy (hipMemcpyDtoDAsync) of as many bytes as a call gathers, from another
    place of the ring every call (HBM) and from the same place (caches); the gather alone (mrb_per_gather, no
    tree descent) at given slots that differ from call to call, over the whole ring and confined to its first
    GiB; and the same slots every call (served by the caches). A sample call is the gather plus a descent that
    must end before the first row byte can be requested."""
    L, h, sp, batch = r.L, r.h, r.sp, r.batch
    n = 400

    def timed(fn):
        for i in range(20):
            fn(i)
        torch.cuda.synchronize()
        e0, e1 = events(torch)
        e0.record(r.stream)
        for i in range(n):
            fn(i)
        e1.record(r.stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / n

    out = {"unit": "us per call, HIP events over %d back-to-back calls" % n}
    out["empty_launch"] = timed(lambda i: L.mrb_bench_launch(0, None, None, 0, sp))
    store = r.buf.storage()[0]  # [capacity, 84, 84, 4] u8
    row = r.buf._layout.bytes[0]
    dst = r.fields[0]
    nbytes = batch * row
    places = max(1, (r.capacity // batch) - 1)
    base = store.data_ptr()
    out["d2d_copy_same_bytes_fresh_source"] = timed(
        lambda i: L.mrb_bench_launch(1, dst.data_ptr(), base + ((i * 37) % places) * nbytes, nbytes, sp))
    out["d2d_copy_same_bytes_same_source"] = timed(lambda i: L.mrb_bench_launch(1, dst.data_ptr(), base, nbytes, sp))
    gfields = r.buf._layout.empty(batch, r.buf._dev)
    gptr = r.pointers(gfields)
    rng = np.random.default_rng(r.seed + 3)
    nset = 256
    for key, window in (("gather_fresh_slots_whole_ring", r.capacity),
                        ("gather_fresh_slots_first_GiB", min(r.capacity, (1 << 30) // sum(r.buf._layout.bytes)))):
        idx = torch.from_numpy(rng.integers(0, window, (nset, batch))).cuda()
        out[key] = timed(lambda i: L.mrb_per_gather(h, idx[i % nset].data_ptr(), batch, gptr, sp))
    out["gather_same_slots_every_call"] = timed(lambda i: L.mrb_per_gather(h, idx[0].data_ptr(), batch, gptr, sp))
    out["frac_of_peak_of_d2d_copy_fresh_source"] = (
        algo_bytes / (out["d2d_copy_same_bytes_fresh_source"] * 1e-6) / 1e9 / HBM_PEAK_GBS)
    out["frac_of_peak_of_gather_fresh_slots"] = (
        algo_bytes / (out["gather_fresh_slots_whole_ring"] * 1e-6) / 1e9 / HBM_PEAK_GBS)
    r.buf.check()
    return out


def per_extras(a, torch, r, algo_bytes):
    """Untimed side figures: the other operations of the config's step, the same sample steps replayed from
    a HIP graph, and issued round robin on several streams (independent calls, one output set per stream)."""
    L, h, sp, W, batch = r.L, r.h, r.sp, r.W, r.batch
    K = r.n_draws - W  # the side figures run over all the draws there are, whatever the timed run's step count
    extras = {}
    n_it = 300

    def timed(fn, n=n_it):
        for i in range(10):
            fn(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n):
            fn(i)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n

    uidx = torch.from_numpy(r.rng.integers(0, r.capacity, (64, r.upd_n))).cuda()
    extras["updates_per_s"] = r.upd_n / timed(
        lambda i: L.mrb_per_update(h, uidx[i % 64].data_ptr(), r.upr[i % 64].data_ptr(), r.upd_n, sp))
    extras["inserts_per_s"] = r.ins_n / timed(lambda i: L.mrb_per_push(h, r.sptr, r.ins_n, r.ins_pr, sp))
    extras["loop_steps_per_s"] = 1.0 / timed(lambda i: r.loop_bound(W + i % K))
    # the same step with update_priorities and the insert as one call (mrb_per_update_push: fewer launches)
    extras["update_push_us_per_call"] = timed(lambda i: r._update_push_fn(*r._update_push_args[i % 64])) * 1e6
    extras["loop_update_push_steps_per_s"] = 1.0 / timed(lambda i: r.loop_fused_bound(W + i % K))
    # ... and with the sample in that call too (mrb_per_update_push_sample: one launch on a small buffer)
    extras["loop_one_call_steps_per_s"] = 1.0 / timed(lambda i: r.loop_one_call_bound(W + i % K))
    # the same loop recorded ONCE into a HIP graph (50 steps) with the buffer's counters kept on the device, so
    # that every replay continues where the last one stopped; replayed 10 times
    if r.upd <= 1024:  # device-resident counters take updates of at most 1024 entries
        r.buf.set_option("device_counters", 1)
        n_l = min(K, 50)
        for key, fused in (("loop_graph_replay_steps_per_s", False), ("loop_update_push_graph_replay_steps_per_s", True),
                           ("loop_one_call_graph_replay_steps_per_s", "one call")):
            lgraph = torch.cuda.CUDAGraph()
            lside = torch.cuda.Stream()
            with torch.cuda.stream(lside):
                lsp = C.c_void_p(lside.cuda_stream)
                lgraph.capture_begin()
                for i in range(n_l):
                    r.loop(W + i, lsp, fused)
                lgraph.capture_end()
            torch.cuda.synchronize()
            lgraph.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(10):
                lgraph.replay()
            torch.cuda.synchronize()
            extras[key] = 10 * n_l / (time.perf_counter() - t0)
            del lgraph
        r.buf.set_option("device_counters", 0)
    if not r.loop_step:
        extras["sample_us_per_call"] = timed(lambda i: r.sample(W + i % K)) * 1e6
        # spread over the run: an event after every 10 calls (an event after every call would add its own ~3 us),
        # 40 groups of 10 back-to-back calls
        evs = [torch.cuda.Event(enable_timing=True) for _ in range(41)]
        torch.cuda.synchronize()
        evs[0].record(r.stream)
        for g in range(40):
            for i in range(10):
                r.sample(W + (10 * g + i) % K)
            evs[g + 1].record(r.stream)
        torch.cuda.synchronize()
        per_call = np.sort(np.array([evs[g].elapsed_time(evs[g + 1]) * 100.0 for g in range(40)]))
        extras["sample_us_p10_p50_p90_of_10_call_groups"] = [float(per_call[4]), float(per_call[20]), float(per_call[36])]
        if a.workload == "c3":
            # the frame-shared next observation: rows at the sampled transitions' next_idx, through mrb_per_gather
            # (whole rows, 2 * 28,241 B each: 28.9 MB per call on top of the sample's)
            nxt = r.fields[1].reshape(-1)
            gfields = r.buf._layout.empty(batch, r.buf._dev)
            gptr = r.pointers(gfields)
            r.sample(W)
            extras["next_obs_gather_same_slots_us_per_call"] = timed(
                lambda i: L.mrb_per_gather(h, nxt.data_ptr(), batch, gptr, sp)) * 1e6
            # sample, then gather at the slots that very sample returned: other rows every call
            extras["sample_plus_next_obs_us"] = timed(
                lambda i: (r.sample(W + i % K), L.mrb_per_gather(h, nxt.data_ptr(), batch, gptr, sp))) * 1e6
            # the same in ONE launch: the sample plus the observation at each sampled row's next_idx
            # (mrb_per_sample_next: 2 * 28,224 B more per row, the launch and the descent paid once)
            nobs = torch.empty_like(r.fields[0])
            def fused(i):
                rc = L.mrb_per_sample_next(h, batch, float(r.betas[W + i % K]),
                                           r.uniforms.data_ptr() + (W + i % K) * batch * 4, 1, 0, r.idx.data_ptr(),
                                           r.wts.data_ptr(), r.fptr, nobs.data_ptr(), sp)
                if rc:
                    r._lib.check(rc)
            us = timed(fused) * 1e6
            extras["sample_with_next_obs_one_launch_us"] = us
            extras["sample_with_next_obs_one_launch_frac_of_peak"] = (
                (algo_bytes + batch * 2 * r.buf._layout.bytes[0]) / (us * 1e-6) / 1e9 / HBM_PEAK_GBS)
            del gfields, nobs
        # the same calls replayed from one captured HIP graph (a chain: every call ordered after the one before)
        n_g = min(K, 200)
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            sps = C.c_void_p(side.cuda_stream)
            graph.capture_begin()
            for i in range(n_g):
                r.sample(W + i, sps)
            graph.capture_end()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(5):
            graph.replay()
        torch.cuda.synchronize()
        extras["graph_replay_us_per_call"] = (time.perf_counter() - t0) / (5 * n_g) * 1e6
        del graph
        # independent sample calls issued round robin on several streams, each stream with its own outputs:
        # what a prefetching caller sustains when calls need not wait for one another
        sets = []
        for _ in range(4):
            st = torch.cuda.Stream()
            f = r.buf._layout.empty(batch, r.buf._dev)
            io_, wo_ = torch.empty(batch, dtype=torch.int64, device="cuda"), torch.empty(batch, dtype=torch.float32, device="cuda")
            sets.append((C.c_void_p(st.cuda_stream), (io_.data_ptr(), wo_.data_ptr(), r.pointers(f)), (io_, wo_, f, st)))
        torch.cuda.synchronize()
        pipelined = {}
        for ns in (2, 4):
            def rr(i):
                s_, out_, _ = sets[i % ns]
                r.sample(W + i % K, s_, out_)
            pipelined[str(ns)] = timed(rr, max(n_it, 200)) * 1e6
        extras["streams_round_robin_us_per_call"] = pipelined
        row_bytes = sum(r.buf._layout.bytes)
        extras["streams_round_robin_frac_of_peak"] = algo_bytes / (min(pipelined.values()) * 1e-6) / 1e9 / HBM_PEAK_GBS
        # several batches per launch (mrb_per_sample_many): the launch and the descent are paid once for
        # all of them, which is what a learner that prefetches batches between priority updates can use
        many = {}
        for nb in (4, 16):
            if nb > K + W or nb * batch * row_bytes > (8 << 30):
                continue
            fo = r.buf._layout.empty(nb * batch, r.buf._dev)
            io = torch.empty(nb * batch, dtype=torch.int64, device="cuda")
            wo = torch.empty(nb * batch, dtype=torch.float32, device="cuda")
            fp = r.pointers(fo)
            # every call takes other draws, so no call finds the rows of the one before in the caches
            nset = (K + W) // nb
            call = lambda i: L.mrb_per_sample_many(h, nb, batch, float(r.betas[W]),
                                                   r.uniforms.data_ptr() + (i % nset) * nb * batch * 4,
                                                   io.data_ptr(), wo.data_ptr(), fp, sp)
            for i in range(5):
                call(i)
            torch.cuda.synchronize()
            e0, e1 = events(torch)
            reps = max(10, 200 // nb)
            e0.record(r.stream)
            for i in range(reps):
                call(i)
            e1.record(r.stream)
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / (reps * nb)
            many[str(nb)] = {"us_per_batch": us,
                             "frac_of_peak": algo_bytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS}
            del fo, io, wo
        extras["sample_many_batches_per_launch"] = many
    r.buf.check()
    return extras


def bench_uniform(a):
    """Config 2: SAC MuJoCo-shaped UniformReplayBuffer, capacity 1,000,000, 165 B rows; insert in chunks of
    1000, then sample batch 256 with seeded uniform integer indices drawn on the host."""
    import torch

    from mindrl_amd import _lib
    from mindrl_amd.core import UniformReplayBuffer
    from mindrl_amd.core._rows import pointers

    capacity, batch = (a.capacity or 1_000_000), 256
    shapes, np_dtypes = [(17,), (6,), (1,), (17,), (1,)], ["float32", "float32", "float32", "float32", "bool"]
    buf = UniformReplayBuffer(batch, capacity, shapes, [getattr(torch, d) for d in np_dtypes], seed=1002,
                              packed_rows=a.packed_rows)
    gen = torch.Generator(device="cuda").manual_seed(1002)
    chunk = 1000
    src = [torch.randn((chunk,) + s, device="cuda", generator=gen) if d != "bool"
           else torch.rand((chunk,) + s, device="cuda", generator=gen) < 0.01 for s, d in zip(shapes, np_dtypes)]
    L = _lib.lib()
    sp = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    sptr = pointers(src)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(capacity // chunk):
        _lib.check(L.mrb_urb_append(buf._h, sptr, chunk, sp))
    torch.cuda.synchronize()
    ins_s = time.perf_counter() - t0
    K, W = a.steps, a.warmup
    rng = np.random.default_rng(1002)
    idx = torch.from_numpy(rng.integers(0, capacity, (K + W, batch))).cuda()
    out = buf._layout.empty(batch, buf._dev)
    optr = pointers(out)
    ibase = idx.data_ptr()
    for i in range(W):
        _lib.check(L.mrb_urb_gather(buf._h, ibase + i * batch * 8, batch, optr, sp))
    torch.cuda.synchronize()
    ev0, ev1 = events(torch)
    t0 = time.perf_counter()
    ev0.record()
    for i in range(W, W + K):
        L.mrb_urb_gather(buf._h, ibase + i * batch * 8, batch, optr, sp)
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    buf.check()
    row_bytes = sum(buf._layout.bytes)
    algo = batch * (2 * row_bytes + 8)
    kern_s = ev0.elapsed_time(ev1) * 1e-3 / K
    res = {
        "metric": "sampled transitions/sec (sample+gather), uniform buffer at cap 1M", "value": K * batch / wall,
        "unit": "transitions/s", "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": wall * 1e3 / K,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": "config 2: SAC-shaped UniformReplayBuffer, capacity %d, 165 B rows, batch 256, "
                               "host-drawn indices" % capacity, "row_bytes": row_bytes},
        "roofline": roofline("k_rows_gather", algo, kern_s, wall / K, "c2", "batch * (2 * row_bytes + 8)"),
        "extras": {"inserts_per_s": capacity / ins_s, "insert_chunk": chunk},
        "cpu_baseline": None,
    }
    if not a.no_cpu_baseline:
        from oracle import orc
        cap_c = min(capacity, 1 << 20)
        o = orc.OracleUniform(cap_c, shapes, np_dtypes, seed=1002)
        rows = [np.asarray(t.cpu().numpy()) for t in src]
        for _ in range(cap_c // chunk):
            o.append(rows, chunk)
        Lo = orc.lib()
        dst = o._dst(batch)
        dptr = orc._ptr_array(dst)
        hidx = rng.integers(0, o.count, (256, batch))
        calls, t_end = 0, time.perf_counter() + 5.0
        t0 = time.perf_counter()
        while time.perf_counter() < t_end:
            Lo.orc_urb_gather(o.h, hidx[calls % 256].ctypes.data, batch, dptr)
            calls += 1
        dt = time.perf_counter() - t0
        res["cpu_baseline"] = {"value": calls * batch / dt, "unit": "transitions/s", "cores": 1, "kind": "port",
                               "sample": "%d gather calls of batch %d in %.1f s, capacity %d, 1 thread" % (
                                   calls, batch, dt, cap_c)}
    buf.destroy()
    print(json.dumps(res))
    return 0


def bench_reservoir(a):
    """ReservoirReplayBuffer, capacity 1,000,000, rows f32[17] + i32[6] (92 B): push batches of 4096 well past
    the capacity (so every batch draws replacement slots and elects winners), then sample 256 per call."""
    import torch

    from mindrl_amd import _lib
    from mindrl_amd.core import ReservoirReplayBuffer
    from mindrl_amd.core._rows import pointers

    capacity, batch, chunk = (a.capacity or 1_000_000), 256, 4096
    shapes, np_dtypes = [(17,), (6,)], ["float32", "int32"]
    buf = ReservoirReplayBuffer(capacity, batch, shapes, [torch.float32, torch.int32], seed1=1006)
    src = [torch.randn(chunk, 17, device="cuda"), torch.randint(0, 9, (chunk, 6), dtype=torch.int32, device="cuda")]
    L = _lib.lib()
    sp = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    sptr = pointers(src)
    for _ in range(capacity // chunk + 1):
        _lib.check(L.mrb_res_push(buf._h, sptr, chunk, sp))
    torch.cuda.synchronize()
    n_push = 500
    t0 = time.perf_counter()
    for _ in range(n_push):
        L.mrb_res_push(buf._h, sptr, chunk, sp)
    torch.cuda.synchronize()
    push_s = time.perf_counter() - t0
    K, W = a.steps, a.warmup
    out = buf._layout.empty(batch, buf._dev)
    optr = pointers(out)
    for _ in range(W):
        _lib.check(L.mrb_res_sample(buf._h, batch, None, optr, sp))
    torch.cuda.synchronize()
    ev0, ev1 = events(torch)
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(K):
        L.mrb_res_sample(buf._h, batch, None, optr, sp)
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    row_bytes = sum(buf._layout.bytes)
    algo = batch * 2 * row_bytes
    kern_s = ev0.elapsed_time(ev1) * 1e-3 / K
    res = {
        "metric": "sampled transitions/sec, reservoir buffer at cap 1M", "value": K * batch / wall,
        "unit": "transitions/s", "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": wall * 1e3 / K,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": "ReservoirReplayBuffer, capacity %d, 92 B rows, push 4096 per call past capacity, "
                               "sample 256 per call" % capacity, "row_bytes": row_bytes},
        "roofline": roofline("k_rows_gather", algo, kern_s, wall / K, "res", "batch * 2 * row_bytes"),
        "extras": {"pushes_per_s": n_push * chunk / push_s, "push_chunk": chunk},
        "cpu_baseline": None,
    }
    if not a.no_cpu_baseline:
        from oracle import orc
        o = orc.OracleReservoir(capacity, shapes, np_dtypes, seed=1006)
        rows = [t.cpu().numpy() for t in src]
        for _ in range(capacity // chunk + 1):
            o.push(rows, chunk)
        t0 = time.perf_counter()
        for _ in range(100):
            o.push(rows, chunk)
        cpu_push = 100 * chunk / (time.perf_counter() - t0)
        Lo = orc.lib()
        dst = o._dst(batch)
        dptr = orc._ptr_array(dst)
        calls, t_end = 0, time.perf_counter() + 4.0
        t0 = time.perf_counter()
        while time.perf_counter() < t_end:
            Lo.orc_res_sample(o.h, batch, None, dptr)
            calls += 1
        dt = time.perf_counter() - t0
        res["cpu_baseline"] = {"value": calls * batch / dt, "unit": "transitions/s", "cores": 1, "kind": "port",
                               "sample": "%d sample calls of batch %d in %.1f s (and %.3g pushed rows/s), capacity "
                                         "%d, 1 thread" % (calls, batch, dt, cpu_push, capacity)}
    buf.destroy()
    print(json.dumps(res))
    return 0


def bench_discounted_return(a):
    """DiscountedReturn on [Timestep 1000, Batch 16384] float32 rewards with 1 % episode ends."""
    import torch

    from mindrl_amd import _lib

    t, b, inner, gamma = 1000, (a.capacity or 16384), 1, 0.99
    gen = torch.Generator(device="cuda").manual_seed(7)
    # four sets of inputs and outputs taken in turn (590 MB together): no step finds its input in the 256 MB
    # memory-side cache because the step before read the same tensors
    nsets = 4
    sets = []
    for _ in range(nsets):
        r = torch.randn(t, b, inner, device="cuda", generator=gen)
        d = torch.rand(t, b, device="cuda", generator=gen) < 0.01
        v = torch.randn(b, inner, device="cuda", generator=gen)
        sets.append((r, d, v, torch.empty_like(r)))
    r, d, v, out = sets[0]
    L = _lib.lib()
    sp = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    K, W = min(a.steps, 200), min(a.warmup, 20)

    def step(i):
        ri, di, vi, oi = sets[i % nsets]
        rc = L.mrb_discounted_return(ri.data_ptr(), di.data_ptr(), vi.data_ptr(), oi.data_ptr(), t, b, inner, gamma, sp)
        if rc:
            _lib.check(rc)

    for i in range(W):
        step(i)
    torch.cuda.synchronize()
    ev0, ev1 = events(torch)
    t0 = time.perf_counter()
    ev0.record()
    for i in range(K):
        step(W + i)
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    algo = t * b * inner * 8 + t * b
    kern_s = ev0.elapsed_time(ev1) * 1e-3 / K
    res = {
        "metric": "discounted-return elements/sec", "value": K * t * b * inner / wall, "unit": "elements/s",
        "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": wall * 1e3 / K, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "DiscountedReturn, reward [1000, %d, 1] f32, gamma 0.99, 1 %% dones" % b},
        "roofline": roofline("k_discounted_return_tiled" if b * inner <= 16384 else "k_discounted_return", algo, kern_s,
                             wall / K, "dr", "T * B * (4 read + 4 written) + T * B done flags"),
        "cpu_baseline": None,
    }
    if not a.no_cpu_baseline:
        from oracle import orc
        rn, dn, vn = r.cpu().numpy(), d.cpu().numpy(), v.cpu().numpy()
        calls, t_end = 0, time.perf_counter() + 5.0
        t0 = time.perf_counter()
        while time.perf_counter() < t_end:
            orc.discounted_return(rn, dn, vn, gamma)
            calls += 1
        dt = time.perf_counter() - t0
        res["cpu_baseline"] = {"value": calls * t * b * inner / dt, "unit": "elements/s", "cores": 1, "kind": "port",
                               "sample": "%d calls on the same [1000, %d, 1] input in %.1f s, 1 thread" % (calls, b, dt)}
    print(json.dumps(res))
    return 0


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py: this benchmark measures one GPU; --gpus %d is not supported (every box here has one GPU)"
              % a.gpus, file=sys.stderr)
        return 2
    import torch

    assert torch.cuda.is_available(), "bench.py needs a HIP device"
    torch.cuda.set_device(0)
    if a.workload == "c2":
        return bench_uniform(a)
    if a.workload == "res":
        return bench_reservoir(a)
    if a.workload == "dr":
        return bench_discounted_return(a)
    return bench_per(a)


if __name__ == "__main__":
    sys.exit(main())
