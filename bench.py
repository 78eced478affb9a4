#!/usr/bin/env python3
"""Benchmark of the fused sparse tree attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--extra]

Workload (the configuration the headline metric is quoted on): 256-node
Medusa-style tree, B=1, H=32, D=128, bf16, query block 64, synthetic CPU-seeded
N(0,1) q/k/v, sm_scale = 1/sqrt(D).  A step is one call of the attention entry
point of the C ABI (``fsta_attention_fwd``) with the per-block kernel inputs
already built (they are built once per decoding step and reused by every layer,
which is also how the reference's own benchmark times it).

Timed region: exactly K steps, recorded into one HIP graph so that the host's
launch rate does not hide the kernel, each step on its own q/k/v/o buffer set;
the sets rotate over more memory than the 256 MB Infinity Cache, so K/V rows come
from HBM ("cold").  The same loop over one buffer set ("warm": everything cache
resident) and plain stream launches are reported beside it.

Prints ONE JSON line.  ``value`` = K/V bytes the op loads per step (per head:
2*D*2 bytes for every valid ancestor slot and every valid leaf slot of every
block) divided by the wall time per step.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

REPO = os.path.dirname(os.path.abspath(__file__))
if REPO not in sys.path:
    sys.path.insert(0, REPO)

HBM_PEAK_GBPS = 8000.0       # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0
INFINITY_CACHE_BYTES = 256 << 20

# HBM bytes per launch of the headline kernel come from a tracked rocprofv3 counter summary (two
# --pmc runs, FETCH_SIZE and WRITE_SIZE, scaled by what the counters read for a plain copy); the
# summary names the kernel it was taken from, and the figure is only reported for that kernel.
TRAFFIC_PROFILE = os.path.join(REPO, "profiles", "attn_mfma16_kernel_cfg2_medusa256_hbm_traffic.txt")
HEADLINE_MIN_STEPS = 400     # the headline is also timed over at least this many steps, whatever --steps says


def measured_traffic(kernel_name):
    """HBM bytes per launch from the tracked counter summary, if it was taken from `kernel_name`
    (template arguments included), else None."""
    import re
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return None
    kernel = re.search(r"^kernel:\s*(.+)$", text, re.M)
    traffic = re.search(r"^traffic_bytes_per_launch:\s*(\d+)", text, re.M)
    squeeze = lambda t: t.replace(" ", "")
    if not kernel or not traffic or squeeze(kernel.group(1)) != squeeze(kernel_name.split(">")[0] + ">"):
        return None
    return int(traffic.group(1))


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--config", type=int, default=2, help="benchmark configuration 1..5 (headline: 2)")
    ap.add_argument("--extra", action="store_true",
                    help="also time the depth-first orderings, the front-end kernels, decoding steps and prefixes")
    ap.add_argument("--quick", action="store_true",
                    help="headline only: skip the other configurations and the reference's benchmark shapes")
    ap.add_argument("--regimes", action="store_true",
                    help="also time the warm-cache loop, plain stream launches, the Python entry point "
                         "and the GPU precompute")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MIB",
                    help="instead of the benchmark, run 10 device-to-device copies of MIB MiB "
                         "(reference point for the FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--dtype", choices=["bf16", "f16", "f32"], default=None,
                    help="storage type of q/k/v (default: the configuration's own, bf16 for the headline)")
    ap.add_argument("--prefix", type=int, default=0, metavar="KEYS",
                    help="put a shared dense prefix of KEYS keys in front of the tree (reference "
                         "fstattention.py:113-136); not the headline workload, implies --no-cpu")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-graph", action="store_true", help="time plain stream launches only")
    return ap.parse_args()


class Workload:
    """Device-resident inputs of one configuration, in `sets` rotating copies."""

    def __init__(self, index, sets_bytes, dtype=None, heads=None, batch=None, order=None, prefix=0,
                 key_splits=None, device_rng=False, kv8=False):
        import torch
        from fstattention_amd import _lib, create_fst_attention_kernel_inputs, shift_for_prefix, trees
        from fstattention_amd.attention import _DTYPES, _packed_for

        self.torch = torch
        # `index`: one of the five benchmark configurations, or a TreeConfig of the caller's
        self.cfg = cfg = trees.config(index, dtype) if isinstance(index, int) else index
        self.cfg_index = index if isinstance(index, int) else None
        if order is not None:
            # the same tree with its nodes (tokens) numbered depth-first (reference README.md:19-20)
            import dataclasses
            new_parent, _ = trees.renumber_parents(cfg.parent, trees.dfs_order(cfg.parent, order))
            self.cfg = cfg = dataclasses.replace(cfg, parent=new_parent)
        self.lib = _lib.load()
        self._check = _lib.check
        dev = torch.device("cuda", 0)
        self.z = batch or cfg.batch
        self.h = heads or cfg.heads
        self.n, self.d, self.m = cfg.n_nodes + cfg.pad_rows, cfg.head_dim, cfg.block_m
        self.dtype = cfg.dtype
        self.code = _DTYPES[cfg.dtype]
        self.esz = torch.tensor([], dtype=cfg.dtype).element_size()
        self.scale = 1.0 / math.sqrt(self.d)

        # kernel inputs: GPU precompute from the device-resident lineage
        lineage, level = trees.lineage_from_parents(cfg.parent)
        self.lineage, self.level = lineage.to(dev), level.to(dev)
        self.max_anc = cfg.max_ancestors or trees.required_max_ancestors(cfg.parent, self.m, 16)
        self.a_idx, self.a_mask, self.l_idx = create_fst_attention_kernel_inputs(
            self.lineage, self.level, self.m, self.max_anc, mutate_lineage=False)
        # K/V laid out as [shared prefix | tree] (reference fstattention.py:209-212)
        self.prefix = prefix
        self.nk = self.n + prefix
        if prefix:
            self.a_idx, self.l_idx = shift_for_prefix(self.a_idx, self.l_idx, prefix)
        self.packed = _packed_for(self.a_idx, self.a_mask, self.l_idx, self.nk)
        self.plan_ptr = self.packed.plan.data_ptr() if self.packed.plan is not None else None
        self.nb = self.a_idx.shape[0]
        rows = int((self.a_idx >= 0).sum().item() + (self.l_idx >= 0).sum().item())
        self.kv_rows = rows + self.nb * prefix       # every block walks the whole prefix
        # 8-bit K/V storage: K and V rows are float8_e4m3fn with a scale per (batch, head) slice
        self.kv8 = kv8
        self.kv_esz = 1 if kv8 else self.esz
        self.kv_bytes = self.z * self.h * 2 * self.d * self.kv_esz * self.kv_rows
        depth = trees.levels_from_parents(cfg.parent)
        self.pairs = int(depth.sum() + cfg.n_nodes) + cfg.n_nodes * prefix
        self.flops = 4 * self.d * self.z * self.h * self.pairs

        # HBM bytes a launch has to move at least once when nothing is cached from before:
        # every K and V row, Q, O and the log-sum-exp (rows shared by blocks come from L2)
        self.min_traffic_bytes = self.z * self.h * ((2 * self.n * self.esz + 2 * self.nk * self.kv_esz) * self.d + 4 * self.n)
        per_set = self.z * self.h * (2 * self.n * self.esz + 2 * self.nk * self.kv_esz) * self.d
        self.per_set_bytes = per_set
        # (one set that is larger than twice the Infinity Cache is cold by itself)
        self.n_sets = max(1 if per_set >= 2 * INFINITY_CACHE_BYTES else 2, min(256, -(-sets_bytes // per_set)))
        shape = (self.z, self.h, self.n, self.d)
        kv_shape = (self.z, self.h, self.nk, self.d)
        # workspace for a prefix cut into runs of keys (none wanted: plain entry point)
        self.flags = _lib.flag_key_splits(key_splits) if key_splits else 0
        need = self.lib.fsta_attention_workspace_bytes(self.z, self.h, self.n, self.nk, self.d, self.code, self.m,
                                                       self.max_anc, self.scale, self.flags) if prefix else 0
        self.key_runs = need // (self.z * self.h * self.n * (self.d + 1) * 4) if need else 1
        self.work = torch.empty((need,), dtype=torch.uint8, device=dev) if need else None
        g = torch.Generator().manual_seed(cfg.tensor_seed)
        self.sets = []
        base = None
        for s in range(self.n_sets):
            if device_rng and base is None:
                # N(0,1) drawn on the device (seeded): the large configurations, timing only
                gd = torch.Generator(device=dev).manual_seed(cfg.tensor_seed)
                q, k, v = (torch.randn(sh, generator=gd, dtype=torch.float32, device=dev).to(cfg.dtype)
                           if sh[0] * sh[1] * sh[2] * sh[3] <= 1 << 28 else
                           torch.cat([torch.randn((1,) + sh[1:], generator=gd, dtype=torch.float32, device=dev).to(cfg.dtype)
                                      for _ in range(sh[0])])
                           for sh in (shape, kv_shape, kv_shape))
                base = (q, k, v)
            elif not device_rng and (s < 4 or base is None):
                # CPU-seeded N(0,1), rounded to the storage type, then moved
                q, k, v = (torch.randn(sh, generator=g, dtype=torch.float32).to(cfg.dtype).to(dev)
                           for sh in (shape, kv_shape, kv_shape))
                base = (q, k, v)
            else:
                # further sets: device-side copies rolled along the sequence axis (distinct
                # memory, same distribution) so that building them stays cheap
                q, k, v = (torch.roll(t, shifts=s, dims=2).contiguous() for t in base)
            o = torch.empty(shape, dtype=cfg.dtype, device=dev)
            if kv8:
                from fstattention_amd import quantize_kv_fp8
                k, v, self.k_scale, self.v_scale = quantize_kv_fp8(k, v)     # (every set is a roll of the first: same scales)
            self.sets.append((q, k, v, o))
        self.lse = torch.empty((self.z * self.h, self.n), dtype=torch.float32, device=dev)

    def launch(self, s=0, flags=0):
        """One step: a single call through the C ABI on torch's current stream."""
        torch = self.torch
        q, k, v, o = self.sets[s % self.n_sets]
        if self.kv8:
            self._check(self.lib.fsta_attention_fwd_kv8(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), self.k_scale.data_ptr(), self.v_scale.data_ptr(), o.data_ptr(),
                self.lse.data_ptr(), self.plan_ptr, self.packed.key_shift, self.z, self.h, self.n, self.nk, self.d,
                self.code, self.code, self.m, self.max_anc, self.nb, self.scale, torch.cuda.current_stream().cuda_stream))
            return
        if self.work is not None:
            self._check(self.lib.fsta_attention_fwd_ws(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), self.lse.data_ptr(),
                self.a_idx.data_ptr(), self.packed.mask_bits.data_ptr(), self.packed.anc_count.data_ptr(),
                self.l_idx.data_ptr(), self.plan_ptr, self.packed.key_shift,
                self.z, self.h, self.n, self.nk, self.d, self.code, self.code,
                self.m, self.max_anc, self.nb, self.scale, flags | self.flags, self.work.data_ptr(),
                self.work.numel(), torch.cuda.current_stream().cuda_stream))
            return
        self._check(self.lib.fsta_attention_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), self.lse.data_ptr(),
            self.a_idx.data_ptr(), self.packed.mask_bits.data_ptr(), self.packed.anc_count.data_ptr(),
            self.l_idx.data_ptr(), self.plan_ptr, self.packed.key_shift,
            self.z, self.h, self.n, self.nk, self.d, self.code, self.code,
            self.m, self.max_anc, self.nb, self.scale, flags | self.flags,
            torch.cuda.current_stream().cuda_stream))

    def run_default(self, heads):
        """float32 output of the default kernel on the first `heads` slices of set 0."""
        torch = self.torch
        from fstattention_amd import fst_attention
        q, k, v, _ = self.sets[0]
        hh = min(heads, self.h)
        self._sample = tuple(t[:1, :hh].contiguous() for t in (q, k, v))
        self._sample_scales = {}
        if self.kv8:
            self._sample_scales = {"k_scale": self.k_scale[:hh].contiguous(), "v_scale": self.v_scale[:hh].contiguous()}
        return fst_attention(*self._sample, self.a_idx, self.a_mask, self.l_idx, self.scale,
                             BLOCK_M=self.m, MAX_ANCESTORS=self.max_anc, out_dtype=torch.float32, **self._sample_scales)

    def cross_check(self, heads=2):
        """Default kernel vs the library's scalar kernel (an independent second implementation)
        on a sample: a GPU-only sanity check of every timed configuration.  Parity against the
        CPU oracle is asserted by the test suite and, for the headline workload, by the
        cpu_baseline leg below."""
        torch = self.torch
        from fstattention_amd import fst_attention
        o = self.run_default(heads)
        sample = self._sample
        if self.kv8:      # the scalar kernel in float32 on the widened rows (a 16-bit copy of them would be rounded again)
            qs, k8, v8 = sample
            widen = lambda t, sc: t.float() * sc.view(1, -1, 1, 1)
            sample = (qs.float(), widen(k8, self._sample_scales["k_scale"]), widen(v8, self._sample_scales["v_scale"]))
        ref = fst_attention(*sample, self.a_idx, self.a_mask, self.l_idx, self.scale,
                            BLOCK_M=self.m, MAX_ANCESTORS=self.max_anc, out_dtype=torch.float32, generic=True)
        tol = 1e-5 if self.dtype == torch.float32 else 2e-3
        err = (o.double() - ref.double()).abs()
        ok = bool((err <= tol + tol * ref.double().abs()).all()) and bool(torch.isfinite(o).all())
        return ok, float(err.max()), tol


def time_steps(wl, steps, warmup, rotate, use_graph, flags=0):
    """(wall seconds per step, event seconds per step) over exactly `steps` steps."""
    torch = wl.torch
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for i in range(warmup):
            wl.launch(i if rotate else 0, flags)
        stream.synchronize()
        graph = None
        if use_graph:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                for i in range(steps):
                    wl.launch(i if rotate else 0, flags)
            graph.replay()          # one untimed replay: uploads the graph
            stream.synchronize()
        ev0 = torch.cuda.Event(enable_timing=True)
        ev1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ev0.record(stream)
        if graph is not None:
            graph.replay()
        else:
            for i in range(steps):
                wl.launch(i if rotate else 0, flags)
        ev1.record(stream)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
    return (t1 - t0) / steps, ev0.elapsed_time(ev1) * 1e-3 / steps


def time_python_api(wl, steps, warmup):
    """Seconds per call of the Python entry point (allocates o and lse every call)."""
    torch = wl.torch
    from fstattention_amd import fst_attention
    q, k, v, _ = wl.sets[0]
    call = lambda: fst_attention(q, k, v, wl.a_idx, wl.a_mask, wl.l_idx, wl.scale,
                                 BLOCK_M=wl.m, MAX_ANCESTORS=wl.max_anc)
    for _ in range(warmup):
        call()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        call()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def time_precompute(wl, reps=50):
    """Seconds per GPU rebuild of the kernel inputs (packed mask only, no host sync)."""
    torch = wl.torch
    from fstattention_amd import create_fst_attention_kernel_inputs
    call = lambda: create_fst_attention_kernel_inputs(wl.lineage, wl.level, wl.m, wl.max_anc,
                                                      mutate_lineage=False, check=False,
                                                      want_bool_mask=False)
    for _ in range(5):
        call()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        call()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / reps


def time_front_end(index, reps=20, stages=None):
    """Device microseconds of the per-step tree front-end of configuration `index`, each stage
    recorded `reps` times into a HIP graph (allocations of the Python wrappers included, host time not):
    draft probabilities -> parent array (cfg2's generator only), depth-first order, parent array ->
    lineage, lineage -> kernel inputs."""
    import torch
    from fstattention_amd import (create_fst_attention_kernel_inputs, dfs_order_gpu, kernel_inputs_from_parents_gpu,
                                  lineage_from_parents_gpu, medusa_parents_gpu, trees)
    dev = torch.device("cuda", 0)
    cfg = trees.config(index)
    parent = torch.from_numpy(cfg.parent).to(dev)
    lineage, level = trees.lineage_from_parents(cfg.parent)
    lineage, level = lineage.to(dev), level.to(dev)
    width = lineage.shape[1]
    max_anc = trees.required_max_ancestors(cfg.parent, cfg.block_m, 16)

    def device_us(fn):
        stream = torch.cuda.Stream()
        with torch.cuda.stream(stream):
            for _ in range(3):
                fn()
            stream.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                for _ in range(reps):
                    fn()
            graph.replay()
            stream.synchronize()
            ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            ev0.record(stream)
            graph.replay()
            ev1.record(stream)
            torch.cuda.synchronize()
        return round(ev0.elapsed_time(ev1) * 1e3 / reps, 2)

    # the status word the stages of a step share: zeroed once per step by the caller, not by every stage
    st = torch.zeros((1,), dtype=torch.int32, device=dev)
    calls = {
        "dfs_order_us": lambda: dfs_order_gpu(parent, "light_first", check=False, status=st),
        "lineage_from_parents_us": lambda: lineage_from_parents_gpu(parent, width=width, check=False, status=st),
        "kernel_inputs_us": lambda: create_fst_attention_kernel_inputs(
            lineage, level, cfg.block_m, max_anc, mutate_lineage=False, check=False, want_bool_mask=False, status=st),
        # the two stages above in one launch (lineage rows built in every workgroup's LDS)
        "kernel_inputs_from_parents_us": lambda: kernel_inputs_from_parents_gpu(parent, cfg.block_m, max_anc, width, check=False,
                                                                                status=st),
    }
    if index == 2:
        probs = torch.from_numpy(trees.medusa_probs()).to(dev)
        calls["tree_from_probabilities_us"] = lambda: medusa_parents_gpu(probs, cfg.n_nodes, status=st)
        # five draft depths of 10 ranks: 111110 candidate paths, the multi-launch builder over a workspace
        probs5 = torch.from_numpy(trees.medusa_probs(5, 10)).to(dev)
        calls["tree_from_probabilities_111110_paths_us"] = lambda: medusa_parents_gpu(probs5, 1024, status=st)
    return {name: device_us(fn) for name, fn in calls.items() if stages is None or name in stages}


def time_decoding_step(wl, layers=32, reps=5, depth_first=True, fused=True):
    """One decoding step of the headline workload as one HIP graph: draft probabilities -> tree ->
    (depth-first order ->) kernel inputs (lineage rows built inside that launch; `fused=False`: lineage and kernel inputs as
    two launches) once, then `layers` attention calls on rotating
    q/k/v/o sets that all use those inputs.  Microseconds per step from HIP events."""
    import torch
    from fstattention_amd import (create_fst_attention_kernel_inputs, dfs_order_gpu, fst_attention, kernel_inputs_from_parents_gpu,
                                  lineage_from_parents_gpu, medusa_parents_gpu, renumber_parents_gpu, trees)
    dev = torch.device("cuda", 0)
    probs = torch.from_numpy(trees.medusa_probs()).to(dev)
    depths = probs.shape[0]

    def step():
        status = torch.zeros((1,), dtype=torch.int32, device=dev)
        parent = medusa_parents_gpu(probs, wl.n, status=status)
        if depth_first:
            perm, rank = dfs_order_gpu(parent, "light_first", check=False, status=status)
            parent = renumber_parents_gpu(parent, perm, rank)
        if fused:
            a_idx, packed, l_idx, _ = kernel_inputs_from_parents_gpu(parent, wl.m, wl.max_anc, depths + 1, check=False, status=status)
        else:
            lineage, level = lineage_from_parents_gpu(parent, width=depths + 1, check=False, status=status)
            a_idx, packed, l_idx, _ = create_fst_attention_kernel_inputs(
                lineage, level, wl.m, wl.max_anc, check=False, want_bool_mask=False, status=status)
        for layer in range(layers):
            q, k, v, _ = wl.sets[layer % wl.n_sets]
            fst_attention(q, k, v, a_idx, packed, l_idx, wl.scale, BLOCK_M=wl.m, MAX_ANCESTORS=wl.max_anc)

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        step()
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            step()
        graph.replay()
        stream.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record(stream)
        for _ in range(reps):
            graph.replay()
        ev1.record(stream)
        torch.cuda.synchronize()
    return ev0.elapsed_time(ev1) * 1e3 / reps


def cpu_baseline(wl, budget_s=10.0):
    """The oracle's dense-masked attention (reference fstattention.py:214-219 restated for
    the CPU, float32 arithmetic on the bf16-rounded inputs) on the host cores."""
    import torch
    from oracle import dense_attention, tree_precompute
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))   # the share of the host this job owns
    torch.set_num_threads(cores)
    q, k, v, _ = wl.sets[0]
    heads = min(wl.h, 32)
    qs, ks, vs = (t[:1, :heads].cpu() for t in (q, k, v))
    mask = tree_precompute.dense_tree_mask(wl.cfg.parent)
    run = lambda: dense_attention.dense_tree_attention(qs, ks, vs, mask, wl.scale, dtype=torch.float32)
    ref, _ = run()
    # the same run is the checker of the GPU result (2e-3 for 16-bit inputs, 1e-5 for float32)
    got = wl.run_default(heads).cpu().double()
    tol = 1e-5 if wl.dtype == torch.float32 else 2e-3
    err = (got - ref.double()).abs()
    parity = {"max_abs_err_vs_oracle": float(err.max()), "tol": tol, "slices_checked": heads,
              "ok": bool((err <= tol + tol * ref.double().abs()).all())}
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < 200):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    scale_up = (wl.z * wl.h) / heads      # slices not run: time extrapolated linearly
    per_call = med * scale_up
    # the same routine in the storage type's own arithmetic (what the reference's oracle does on its
    # fp16 tensors, fstattention.py:214-219): reported beside the float32 run, not used as the checker
    narrow_us = None
    if wl.dtype != torch.float32:
        narrow = []
        while len(narrow) < 3 or (sum(narrow) < 2.0 and len(narrow) < 50):
            t0 = time.perf_counter()
            dense_attention.dense_tree_attention(qs, ks, vs, mask, wl.scale, dtype=wl.dtype)
            narrow.append(time.perf_counter() - t0)
        narrow.sort()
        narrow_us = round(narrow[len(narrow) // 2] * scale_up * 1e6, 1)
    # the per-tree precompute (reference utils.py:104-129) restated in numpy, beside the HIP kernel
    lin, lvl = wl.lineage.cpu().numpy(), wl.level.cpu().numpy()
    pre = []
    for _ in range(5):
        t0 = time.perf_counter()
        tree_precompute.block_inputs(lin.copy(), lvl, wl.m, wl.max_anc)
        pre.append(time.perf_counter() - t0)
    pre.sort()
    return {
        "value": round(wl.kv_bytes / per_call / 1e9, 4),
        "unit": "GB/s",
        "cores": cores,
        "kind": "port",
        "us_per_call": round(per_call * 1e6, 1),
        "us_per_call_in_storage_type_arithmetic": narrow_us,
        "sample": (f"dense-masked attention oracle, float32 on {wl.dtype}-rounded inputs, "
                   f"{heads} of {wl.z * wl.h} (batch, head) slices of the same workload, "
                   f"median of {len(times)} runs" + (", scaled linearly to all slices" if scale_up != 1 else "")),
        "precompute_us_per_tree": {"cpu_numpy_port": round(pre[len(pre) // 2] * 1e6, 1),
                                   "gpu_device": time_front_end(wl.cfg_index, stages=("kernel_inputs_us",))["kernel_inputs_us"]},
    }, parity


def graph_us_per_node(call, nodes, reps=3):
    """Microseconds per node of a HIP graph of `nodes` calls of `call` (HIP events on the launch stream,
    best of `reps` replays after one untimed replay)."""
    import torch
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        call()
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for _ in range(nodes):
                call()
        graph.replay()
        stream.synchronize()
        best = None
        for _ in range(reps):
            ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            ev0.record(stream)
            graph.replay()
            ev1.record(stream)
            torch.cuda.synchronize()
            us = ev0.elapsed_time(ev1) * 1e3 / nodes
            best = us if best is None else min(best, us)
    return best


def measured_ceilings(wl, nodes=HEADLINE_MIN_STEPS):
    """This GPU's own ceilings, measured in this run: what a graph node of the headline launch's shape
    costs when the kernel does nothing (`launch_floor_us`), and what a kernel that only reads gets out
    of HBM (`hbm_read_probe_gbps`: 1 GiB, 16 bytes per lane, eight non-temporal loads per lane in flight, 4096
    workgroups that each walk a contiguous piece -- the best of the eight variants of the probe on this GPU: striding
    over the buffer with the whole grid, as a naive copy does, reads 5.1-5.7 TB/s, contiguous pieces with non-temporal
    loads 7.0; the buffer is four times the Infinity Cache, so every pass comes from HBM), beside torch's plain copy."""
    import torch
    lib, check = wl.lib, wl._check
    cur = lambda: torch.cuda.current_stream().cuda_stream
    # the headline launch: 256 workgroups (half-blocks) of 256 threads
    floor_us = graph_us_per_node(lambda: check(lib.fsta_probe_empty_launch(256, 256, cur())), nodes)
    one_wave_us = graph_us_per_node(lambda: check(lib.fsta_probe_empty_launch(1, 64, cur())), nodes)
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device="cuda").fill_(3)
    sink = torch.zeros((1,), dtype=torch.int32, device="cuda")
    read_us = graph_us_per_node(lambda: check(lib.fsta_probe_hbm_read(src.data_ptr(), n, 4096, 6, sink.data_ptr(), cur())), 4, reps=3)
    strided_us = graph_us_per_node(lambda: check(lib.fsta_probe_hbm_read(src.data_ptr(), n, 2048, 0, sink.data_ptr(), cur())), 4, reps=3)
    dst = torch.empty(n // 4, dtype=torch.uint8, device="cuda")
    copy_us = graph_us_per_node(lambda: dst.copy_(src[: n // 4]), 4, reps=3)
    del src, dst
    torch.cuda.empty_cache()
    return {
        "launch_floor_us": round(floor_us, 3),
        "launch_floor_note": f"per node of a HIP graph of {nodes} launches of an empty kernel, 256 workgroups x 256 threads "
                             "(the headline launch's shape)",
        "one_wave_graph_node_us": round(one_wave_us, 3),
        "hbm_read_probe_gbps": round(n / read_us / 1e3, 1),
        "hbm_read_probe_note": "read-only kernel over 1 GiB, 16 B per lane, 8 non-temporal loads in flight per lane, 4096 "
                               "workgroups, a contiguous piece each",
        "hbm_read_probe_grid_strided_gbps": round(n / strided_us / 1e3, 1),
        "torch_copy_read_plus_write_gbps": round(2 * (n // 4) / copy_us / 1e3, 1),
    }


def summarize(wl, steps, warmup, use_graph, regimes):
    cold_wall, cold_ev = time_steps(wl, steps, warmup, rotate=True, use_graph=use_graph)
    out = {"cold_us": cold_wall * 1e6, "cold_event_us": cold_ev * 1e6}
    if regimes:
        warm_wall, warm_ev = time_steps(wl, steps, warmup, rotate=False, use_graph=use_graph)
        stream_wall, _ = time_steps(wl, steps, warmup, rotate=True, use_graph=False)
        out.update({"warm_us": warm_wall * 1e6, "warm_event_us": warm_ev * 1e6,
                    "stream_launch_us": stream_wall * 1e6})
    return out


def brief(w, steps, warmup, use_graph):
    """Cold timing of one workload with the figures every configuration is reported with."""
    ok, err, _ = w.cross_check()
    wall, ev = time_steps(w, steps, warmup, rotate=True, use_graph=use_graph)
    return {
        "us_per_call_cold": round(wall * 1e6, 2), "kernel": w.lib.fsta_last_attention_kernel().decode(),
        "kv_bytes_per_call": w.kv_bytes, "kv_gbps_cold": round(w.kv_bytes / ev / 1e9, 1),
        "hbm_frac": round(w.kv_bytes / ev / 1e9 / HBM_PEAK_GBPS, 4),
        "q_k_v_o_once_gbps": round(w.min_traffic_bytes / ev / 1e9, 1),
        "effective_tflops": round(w.flops / ev / 1e12, 3),
        "batch": w.z, "heads": w.h, "nodes": w.cfg.n_nodes, "block_m": w.m, "max_ancestors": w.max_anc,
        "dtype": str(w.dtype).replace("torch.", ""), "buffer_sets": w.n_sets, "steps": steps,
        "cross_check_ok": ok, "max_abs_diff_vs_scalar_kernel": err,
    }


def time_layer_loop_with_precompute(w, layers, reps=3):
    """Configuration 5 as written: ONE HIP graph holding the rebuild of the kernel inputs on the GPU from the
    device-resident lineage (reference utils.py:104-129, one launch) followed by `layers` attention calls that
    all read those inputs, each layer on its own q/k/v/o.  Returns (total us per step, us of the rebuild alone)."""
    import torch
    from fstattention_amd import create_fst_attention_kernel_inputs
    lib, check = w.lib, w._check

    def rebuild():
        return create_fst_attention_kernel_inputs(w.lineage, w.level, w.m, w.max_anc, mutate_lineage=False,
                                                  check=False, want_bool_mask=False)

    def step():
        a_idx, packed, l_idx, _ = rebuild()
        stream = torch.cuda.current_stream().cuda_stream
        for layer in range(layers):
            q, k, v, o = w.sets[layer % w.n_sets]
            check(lib.fsta_attention_fwd(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), w.lse.data_ptr(),
                a_idx.data_ptr(), packed.mask_bits.data_ptr(), packed.anc_count.data_ptr(), l_idx.data_ptr(),
                packed.plan.data_ptr(), packed.key_shift, w.z, w.h, w.n, w.nk, w.d, w.code, w.code,
                w.m, w.max_anc, w.nb, w.scale, 0, stream))

    def timed(fn):
        stream = torch.cuda.Stream()
        with torch.cuda.stream(stream):
            fn()
            stream.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                fn()
            graph.replay()
            stream.synchronize()
            ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            ev0.record(stream)
            for _ in range(reps):
                graph.replay()
            ev1.record(stream)
            torch.cuda.synchronize()
        return ev0.elapsed_time(ev1) * 1e3 / reps

    return timed(step), timed(rebuild)


def other_configurations(use_graph, wl2):
    """The benchmark configurations beside the headline: 1 (float32, vector-ALU kernel), 3, 4 and 5, and the
    headline tree in float16 (the type BASELINE's configuration 2 states; the metric is quoted on bfloat16).
    Configuration 5 is run the way it is written: 32 layers, each on its own q/k/v/o (32 GiB resident), the
    kernel inputs rebuilt on the GPU once per step inside the same graph."""
    import torch
    out = {}
    for idx in (1, 3, 4):
        w = Workload(idx, sets_bytes=2 * INFINITY_CACHE_BYTES, device_rng=idx != 1)
        out[w.cfg.name] = brief(w, 100, 5, use_graph)
        del w
        torch.cuda.empty_cache()
    w = Workload(2, sets_bytes=2 * INFINITY_CACHE_BYTES, dtype=torch.float16)
    out[w.cfg.name + "_fp16"] = brief(w, HEADLINE_MIN_STEPS, 20, use_graph)
    del w
    torch.cuda.empty_cache()
    free_bytes = torch.cuda.mem_get_info()[0]
    layers = 32
    w = Workload(5, sets_bytes=min(32 << 30, int(free_bytes * 0.8)), device_rng=True)
    layers = min(layers, w.n_sets)
    entry = brief(w, layers, layers, use_graph)       # one call per layer, every layer on its own buffers
    total_us, rebuild_us = time_layer_loop_with_precompute(w, layers)
    entry["decoding_step"] = {
        "layers": layers, "total_us": round(total_us, 1), "kernel_inputs_rebuild_us": round(rebuild_us, 2),
        "per_layer_us": round((total_us - rebuild_us) / layers, 2),
        "hbm_frac_over_the_step": round(w.kv_bytes * layers / (total_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
        "resident_gib": round(w.n_sets * w.per_set_bytes / 2 ** 30, 1),
        "note": "one HIP graph: kernel inputs rebuilt on the GPU from the device-resident lineage, then one attention "
                "call per layer, each layer on its own seeded q/k/v/o, all layers sharing those inputs",
    }
    out[w.cfg.name] = entry
    del w
    torch.cuda.empty_cache()
    return out


def reference_benchmark(use_graph):
    """The workload the reference's own benchmark is quoted on (fstattention.py:240-296): batch 4, 48 heads,
    head dim 64, float16, create_tree(DEPTH_MAPPING[N]) for N = 2^10 .. 2^16, blocks of 128 rows, 64
    ancestor slots; the reference reports milliseconds per call of the attention operator."""
    import torch
    from fstattention_amd import trees
    out = {}
    for k in range(10, 17):
        w = Workload(trees.reference_benchmark_config(2 ** k), sets_bytes=2 * INFINITY_CACHE_BYTES, device_rng=True)
        b = brief(w, 20 if k >= 15 else 50, 3, use_graph)
        out[f"n_ctx_{2 ** k}"] = {key: b[key] for key in ("us_per_call_cold", "kv_bytes_per_call", "kv_gbps_cold", "hbm_frac",
                                                         "q_k_v_o_once_gbps", "buffer_sets", "cross_check_ok", "kernel")}
        out[f"n_ctx_{2 ** k}"]["ms_per_call"] = round(b["us_per_call_cold"] / 1e3, 4)
        del w
        torch.cuda.empty_cache()
    return out


def fp8_kv_storage(use_graph):
    """16-bit against 8-bit K/V storage where the 16-bit kernel already runs near the rate of a plain copy:
    configuration 4, configuration 5 with its tokens in depth-first order, one of the reference's benchmark shapes."""
    import torch
    from fstattention_amd import trees
    cases = (("cfg4_wide4096", lambda kv8: Workload(4, 2 * INFINITY_CACHE_BYTES, device_rng=True, kv8=kv8), 100),
             ("cfg5_batched2048_depth_first", lambda kv8: Workload(5, 2 * INFINITY_CACHE_BYTES, device_rng=True,
                                                                   order="light_first", kv8=kv8), 30),
             ("reference_benchmark_n16384", lambda kv8: Workload(trees.reference_benchmark_config(16384),
                                                                 2 * INFINITY_CACHE_BYTES, device_rng=True, kv8=kv8), 30))
    out = {}
    for name, make, steps in cases:
        entry = {}
        for label, kv8 in (("k_v_16bit", False), ("k_v_fp8_e4m3", True)):
            w = make(kv8)
            b = brief(w, steps, 3, use_graph)
            entry[label] = {key: b[key] for key in ("us_per_call_cold", "kv_bytes_per_call", "kv_gbps_cold", "hbm_frac",
                                                    "q_k_v_o_once_gbps", "cross_check_ok", "kernel")}
            entry[label]["q_k_v_o_once_bytes"] = w.min_traffic_bytes
            del w
            torch.cuda.empty_cache()
        out[name] = entry
    return out


def copy_calibration(mib):
    """10 plain device copies of `mib` MiB: what FETCH_SIZE / WRITE_SIZE read for known traffic."""
    import torch
    n = mib << 20
    src = torch.empty(n, dtype=torch.uint8, device="cuda").fill_(1)
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    for _ in range(10):
        dst.copy_(src)
    ev1.record()
    torch.cuda.synchronize()
    seconds = ev0.elapsed_time(ev1) * 1e-3 / 10
    # read + write traffic of a plain copy: what this box's HBM delivers to a streaming kernel
    print(json.dumps({"copy_bytes": n, "copies": 10, "us_per_copy": round(seconds * 1e6, 1),
                      "read_plus_write_gbps": round(2 * n / seconds / 1e9, 1)}))


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU (got --gpus {args.gpus}); the op shards over "
              "batch*heads without communication (every GPU would run this same launch on its share of "
              "the heads)", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the hot path has no CPU fallback", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    if args.copy_calibration:
        copy_calibration(args.copy_calibration)
        return
    use_graph = not args.no_graph

    dtype = {None: None, "bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[args.dtype]
    wl = Workload(args.config, sets_bytes=2 * INFINITY_CACHE_BYTES, dtype=dtype, prefix=args.prefix)
    ok, max_err, tol = wl.cross_check()
    if not ok:
        print(f"bench.py: the two kernels disagree (max difference {max_err:.3e} > {tol})", file=sys.stderr)
        sys.exit(1)

    t = summarize(wl, args.steps, args.warmup, use_graph, args.regimes)
    kernel_name = wl.lib.fsta_last_attention_kernel().decode()
    step_s = t["cold_us"] * 1e-6
    # the dominant kernel's average launch duration: HIP events on the launch stream around a graph of
    # at least HEADLINE_MIN_STEPS launches (a 20-step region is 0.1 ms, too short to trust on its own)
    long_steps = max(args.steps, HEADLINE_MIN_STEPS)
    long_wall, long_ev = (t["cold_us"] * 1e-6, t["cold_event_us"] * 1e-6) if long_steps == args.steps else \
        time_steps(wl, long_steps, args.warmup, rotate=True, use_graph=use_graph)
    kernel_s = long_ev
    # Behind a shared prefix the step is two launches (dense prefix kernel, then the tree part which joins) and the dense
    # kernel reads a prefix row once per 128 query rows, not once per block: the per-block byte count of the reference
    # formulation no longer describes what moves, so the roofline figure is taken on q, k, v, o once.
    roofline_bytes = wl.min_traffic_bytes if args.prefix else wl.kv_bytes
    achieved = roofline_bytes / kernel_s / 1e9
    headline = args.config == 2 and not args.prefix
    result = {
        "metric": "K/V GB/s loaded (us/call in us_per_call), 256-node Medusa tree H32 D128 bf16"
                  if headline else
                  f"K/V GB/s loaded, {wl.cfg.name}" + (f" behind {args.prefix} prefix keys" if args.prefix else ""),
        "value": round(wl.kv_bytes / step_s / 1e9, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 6),
        "us_per_call": round(step_s * 1e6, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}[wl.dtype],
        "data": "synthetic",
        "config": {
            "workload": wl.cfg.name + (f"_prefix{args.prefix}" if args.prefix else ""), "nodes": wl.n, "batch": wl.z, "heads": wl.h, "head_dim": wl.d,
            "block_m": wl.m, "max_ancestors": wl.max_anc, "kv_rows_per_head": wl.kv_rows,
            "kv_bytes_per_call": wl.kv_bytes, "attended_pairs": wl.pairs, "flops_per_call": wl.flops,
            "timed_region": ("hip graph of K steps" if use_graph else "K stream launches") +
                            f", {wl.n_sets} rotating q/k/v/o sets ({wl.n_sets * wl.per_set_bytes >> 20} MiB)",
        },
        "effective_tflops": round(wl.flops / step_s / 1e12, 4),
        "same_loop_over_more_steps": {"steps": long_steps, "us_per_call": round(long_wall * 1e6, 3),
                                      "value": round(wl.kv_bytes / long_wall / 1e9, 2)},
        "cross_check": {"max_abs_diff_vs_scalar_kernel": max_err, "tol": tol, "ok": ok},
        "roofline": {
            "bound": "hbm",
            "kernel": kernel_name + (" behind prefix_attn_kernel (whole step: both launches)" if args.prefix and wl.key_runs > 1
                                     else ""),
            "achieved": round(achieved, 2),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 5),
            "traffic": measured_traffic(kernel_name) if headline and wl.dtype == torch.bfloat16 else None,
            "algorithmic_bytes_per_launch": roofline_bytes,
            "avg_launch_us": round(kernel_s * 1e6, 3),
            "launches_timed": long_steps,
            "mfma_frac_of_bf16_peak": round(wl.flops / kernel_s / 1e12 / MFMA_BF16_PEAK_TFLOPS, 6),
        },
    }
    if headline:
        ceil = measured_ceilings(wl)
        roof = result["roofline"]
        roof.update(ceil)
        # the time of a launch that did nothing but start and stream this launch's bytes at the probe's rate
        moved = roof["traffic"] or wl.min_traffic_bytes
        floor_us = ceil["launch_floor_us"] + moved / (ceil["hbm_read_probe_gbps"] * 1e3)
        roof["floor_us"] = round(floor_us, 3)
        roof["frac_of_floor"] = round(floor_us / (kernel_s * 1e6), 4)
        roof["floor_note"] = ("floor_us = launch_floor_us + HBM bytes of the launch (traffic, else q+k+v+o once) / "
                              "hbm_read_probe_gbps; frac_of_floor = floor_us / avg_launch_us")
    if args.regimes:
        result["regimes_us_per_call"] = {
            "cold_graph": round(t["cold_us"], 3), "warm_graph": round(t["warm_us"], 3),
            "cold_stream_launches": round(t["stream_launch_us"], 3),
            "python_api_warm": round(time_python_api(wl, args.steps, args.warmup) * 1e6, 3),
            "gpu_precompute": round(time_precompute(wl) * 1e6, 3),
        }
    if args.prefix:
        result["config"]["prefix_keys"] = args.prefix
        result["config"]["key_runs"] = int(wl.key_runs)
    if not args.no_cpu and not args.prefix:
        result["cpu_baseline"], result["parity"] = cpu_baseline(wl)
        if not result["parity"]["ok"]:
            print(f"bench.py: parity against the CPU oracle failed: {result['parity']}", file=sys.stderr)
            sys.exit(1)
    if not args.quick and not args.prefix:
        result["configs"] = other_configurations(use_graph, wl)
        result["reference_benchmark"] = reference_benchmark(use_graph)
        result["fp8_kv_storage"] = fp8_kv_storage(use_graph)
        if headline:
            # the integer kernels that turn a new tree into kernel inputs once per decoding step, and the whole step
            result["front_end_device_us"] = {"cfg2_medusa256": time_front_end(2)}
            result["cfg2_decoding_step"] = {
                "layers": 32,
                "total_us": round(time_decoding_step(wl, depth_first=False), 1),
                "total_us_lineage_and_kernel_inputs_as_two_launches": round(time_decoding_step(wl, depth_first=False, fused=False), 1),
                "total_us_depth_first_order": round(time_decoding_step(wl), 1),
                "note": "one graph: probabilities -> tree (-> depth-first order) -> lineage -> kernel inputs, then 32 "
                        "attention calls (Python wrapper, output allocated per call) on rotating q/k/v sets; a tree "
                        "this small gains nothing from the depth-first order, the large ones do",
            }
    if args.extra:
        extra = {}
        for idx in (3, 4, 5):
            # configuration 5 is a 32-layer decoding step: one tree, 32 layers with their own q/k/v/o
            # (34 GB resident), so its buffer rotation is the layer loop itself
            w = Workload(idx, sets_bytes=(32 << 30) if idx == 5 else 2 * INFINITY_CACHE_BYTES, device_rng=True)
            ok_i, err_i, _ = w.cross_check()
            steps = max(20, min(args.steps, 100 if idx == 5 else args.steps))
            ti = summarize(w, steps, min(args.warmup, 10), use_graph, True)
            ks = ti["cold_event_us"] * 1e-6
            extra[w.cfg.name] = {
                "us_per_call_cold": round(ti["cold_us"], 2), "us_per_call_warm": round(ti["warm_us"], 2),
                "kv_bytes_per_call": w.kv_bytes, "kv_gbps_cold": round(w.kv_bytes / ks / 1e9, 1),
                "hbm_frac": round(w.kv_bytes / ks / 1e9 / HBM_PEAK_GBPS, 4),
                "effective_tflops": round(w.flops / ks / 1e12, 3),
                "q_k_v_o_bytes_once": w.min_traffic_bytes,
                "q_k_v_o_gbps_cold": round(w.min_traffic_bytes / ks / 1e9, 1),
                "gpu_precompute_us": round(time_precompute(w) * 1e6, 2),
                "cross_check_ok": ok_i, "max_abs_diff_vs_scalar_kernel": err_i,
                "batch": w.z, "heads": w.h, "max_ancestors": w.max_anc,
            }
            if idx == 5:
                layers = min(w.cfg.layers, w.n_sets)
                wall, _ = time_steps(w, layers, layers, rotate=True, use_graph=use_graph)
                pre_us = extra[w.cfg.name]["gpu_precompute_us"]
                extra[w.cfg.name]["decoding_step"] = {
                    "layers": layers, "per_layer_us": round(wall * 1e6, 2),
                    "all_layers_us": round(wall * layers * 1e6, 1), "gpu_precompute_us": pre_us,
                    "total_us": round(wall * layers * 1e6 + pre_us, 1),
                    "resident_gib": round(w.n_sets * w.per_set_bytes / 2 ** 30, 1),
                    "note": "one graph of one attention call per layer, each layer on its own q/k/v/o; "
                            "kernel inputs built once on the GPU and shared by all layers",
                }
            del w
            torch.cuda.empty_cache()
        # the same four trees with tokens laid out depth-first: fewer K/V rows per block, so the
        # byte count changes with the time; both are reported
        for idx in (2, 3, 4, 5):
            w = Workload(idx, sets_bytes=2 * INFINITY_CACHE_BYTES, order="light_first")
            ok_i, err_i, _ = w.cross_check()
            steps = max(20, min(args.steps, 100 if idx == 5 else args.steps))
            ti = summarize(w, steps, min(args.warmup, 10), use_graph, False)
            ks = ti["cold_event_us"] * 1e-6
            extra[w.cfg.name + "_depth_first"] = {
                "us_per_call_cold": round(ti["cold_us"], 2), "kv_rows_per_head": w.kv_rows,
                "kv_bytes_per_call": w.kv_bytes, "kv_gbps_cold": round(w.kv_bytes / ks / 1e9, 1),
                "hbm_frac": round(w.kv_bytes / ks / 1e9 / HBM_PEAK_GBPS, 4),
                "q_k_v_o_bytes_once": w.min_traffic_bytes,
                "q_k_v_o_gbps_cold": round(w.min_traffic_bytes / ks / 1e9, 1),
                "cross_check_ok": ok_i, "max_abs_diff_vs_scalar_kernel": err_i, "max_ancestors": w.max_anc,
            }
            del w
            torch.cuda.empty_cache()
        # the integer kernels that turn a new tree into kernel inputs once per decoding step
        extra["front_end_device_us"] = {trees_name: time_front_end(idx) for idx, trees_name in
                                        ((3, "cfg3_deep1024"), (4, "cfg4_wide4096"), (5, "cfg5_batched2048"))}
        # the headline tree behind a shared prefix (the KV cache of a decoding step, reference
        # fstattention.py:113-136): the prefix as each block's own loop, and cut into runs of keys
        for prefix in (4096, 16384):
            entry = {}
            for label, forced in (("one_launch", 1), ("key_runs", None)):
                w = Workload(2, sets_bytes=2 * INFINITY_CACHE_BYTES, prefix=prefix, key_splits=forced)
                ok_i, err_i, _ = w.cross_check()
                ti = summarize(w, max(20, min(args.steps, 100)), min(args.warmup, 10), use_graph, False)
                ks = ti["cold_event_us"] * 1e-6
                entry[label] = {
                    "us_per_call_cold": round(ti["cold_us"], 2), "key_runs": int(w.key_runs),
                    "kv_bytes_per_call": w.kv_bytes, "kv_gbps_cold": round(w.kv_bytes / ks / 1e9, 1),
                    "q_k_v_o_bytes_once": w.min_traffic_bytes,
                    "q_k_v_o_gbps_cold": round(w.min_traffic_bytes / ks / 1e9, 1),
                    "effective_tflops": round(w.flops / ks / 1e12, 1),
                    "cross_check_ok": ok_i, "max_abs_diff_vs_scalar_kernel": err_i,
                }
                del w
                torch.cuda.empty_cache()
            extra[f"medusa256_behind_prefix_{prefix}"] = entry
        result["extra"] = extra
    print(json.dumps(result))


if __name__ == "__main__":
    main()
