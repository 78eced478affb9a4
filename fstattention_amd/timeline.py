"""Where a workgroup of the matrix-core attention kernel spends its time.

    python -m fstattention_amd.build --timeline        # builds libfsta_timeline.so (-DFSTA_TIMELINE)
    python -m fstattention_amd.timeline [--config 2] [--warm] [--stream]

Runs one launch of a benchmark configuration through the instrumented library: every wave notes the
100 MHz clock at fixed points of the kernel (``FSTA_STAMP`` in ``csrc/fsta_attention_mfma16.hip``)
(the constant 100 MHz clock, 10 ns per tick).  Printed: the mean time between consecutive points over all
waves, a wave's lifetime and the spread of the waves' start times.  Every stamp is a scalar memory
instruction the wave waits for: the shares matter, not the total.  ``--stream`` runs the streaming kernel (``csrc/fsta_attention_stream.hip``, workgroups that walk a list of blocks)
instead and prints where its waves' shader-clock cycles go, by kind of segment.
Measuring tool; the regular library has no such code.
"""
from __future__ import annotations

import argparse
import ctypes
import math
import os

import numpy as np
import torch

from . import _lib, create_fst_attention_kernel_inputs, trees
from .build import TIMELINE_LIB_PATH

POINTS = ["entry", "start-up requests issued (plan, Q rows, early leaf tiles)", "plan arrived", "ancestor tiles requested",
          "Q fragments read", "leaf tile landed (barrier)", "leaf step done", "ancestor step 0 begins", "ancestor step 1 begins",
          "ancestor step 2 begins", "ancestor step 3 begins", "ancestor step 4 begins", "all tiles done",
          "normalised, O rows turned around, stores issued", "stores retired",
          "barrier in front of the epilogue passed (wave pairs by head-dim halves only; reached between 12 and 13)"]
STAMPS = 16


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", type=int, default=2)
    ap.add_argument("--warm", action="store_true", help="run the launch twice on the same buffers and time the second")
    ap.add_argument("--stream", action="store_true", help="the streaming kernel's cycle shares instead")
    ap.add_argument("--slowest", type=int, default=0, help="also print the points of the N waves that end last")
    args = ap.parse_args()
    if not os.path.exists(TIMELINE_LIB_PATH):
        raise SystemExit(f"{TIMELINE_LIB_PATH} is missing: python -m fstattention_amd.build --timeline")
    lib = ctypes.CDLL(TIMELINE_LIB_PATH)
    fwd = lib.fsta_attention_fwd
    fwd.restype, fwd.argtypes = _lib.SIGNATURES["fsta_attention_fwd"]
    lib.fsta_timeline_buffer.restype, lib.fsta_timeline_buffer.argtypes = ctypes.c_int, [ctypes.c_void_p]
    lib.fsta_last_attention_kernel.restype = ctypes.c_char_p

    cfg = trees.config(args.config)
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    lineage, level = trees.lineage_from_parents(cfg.parent)
    max_anc = trees.required_max_ancestors(cfg.parent, cfg.block_m, 16)
    a_idx, packed, l_idx = create_fst_attention_kernel_inputs(lineage.to(dev), level.to(dev), cfg.block_m, max_anc,
                                                              want_bool_mask=False)
    q, k, v = trees.make_qkv(cfg, device=dev) if cfg.batch * cfg.heads <= 64 else (
        torch.randn((cfg.batch, cfg.heads, cfg.n_nodes, cfg.head_dim), device=dev).to(cfg.dtype) for _ in range(3))
    o = torch.empty_like(q)
    code = {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16, torch.float32: _lib.F32}[cfg.dtype]
    max_wgs = 8 * -(-cfg.batch * cfg.heads // 8) * a_idx.shape[0] * 2          # (half-block launches double the grid)
    buf = torch.zeros((max_wgs * 16 * (STAMPS + 2),), dtype=torch.int64, device=dev)
    # flush the caches with a large fill so that q/k/v come from HBM, unless a warm run is wanted
    flush = torch.empty((1 << 30,), dtype=torch.uint8, device=dev)

    def launch(flags=0):
        rc = fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), None, a_idx.data_ptr(), packed.mask_bits.data_ptr(),
                 packed.anc_count.data_ptr(), l_idx.data_ptr(), packed.plan.data_ptr(), 0, cfg.batch, cfg.heads, cfg.n_nodes,
                 cfg.n_nodes, cfg.head_dim, code, code, cfg.block_m, max_anc, a_idx.shape[0], 1.0 / math.sqrt(cfg.head_dim),
                 flags, torch.cuda.current_stream().cuda_stream)
        assert rc == 0, lib.fsta_last_error()

    if args.stream:
        stream_shares(lib, launch, flush, cfg)
        return

    assert lib.fsta_timeline_buffer(None) == 0
    launch()                                   # first launch: code upload, LDS limits
    if not args.warm:
        flush.fill_(1)
    torch.cuda.synchronize()
    assert lib.fsta_timeline_buffer(buf.data_ptr()) == 0
    launch()
    torch.cuda.synchronize()
    kernel = lib.fsta_last_attention_kernel().decode()
    data = buf.cpu().numpy().reshape(-1, STAMPS + 2)
    data = data[data[:, STAMPS] != 0]          # waves that ran
    ticks = data[:, :STAMPS].astype(np.int64)  # low 32 bits of the 100 MHz clock at every point (0 = not reached)
    real = data[:, STAMPS:].astype(np.int64)   # the full clock at entry and exit
    rel = (ticks - ticks[:, :1]) % (1 << 32)
    life_us = (real[:, 1] - real[:, 0]) / 100.0
    print(f"kernel: {kernel}")
    print(f"workload: {cfg.name}, {'cache-resident' if args.warm else 'cold'} buffers; {data.shape[0]} waves; "
          f"100 MHz clock (10 ns per tick)")
    print(f"{'point':<62}{'mean us since the point before':>32}{'mean us since entry':>22}")
    last = np.zeros(rel.shape[0], dtype=np.int64)
    for i in (1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 15, 13, 14):
        reached = ticks[:, i] != 0
        if not reached.any():
            continue
        delta = np.where(reached, rel[:, i] - last, 0)
        print(f"{i:>2} {POINTS[i]:<59}{delta[reached].mean() / 100.0:>32.2f}{rel[reached, i].mean() / 100.0:>22.2f}"
              f"   ({int(reached.sum())} waves)")
        last = np.where(reached, rel[:, i], last)
    print(f"lifetime of a wave: mean {life_us.mean():.2f} us, longest {life_us.max():.2f} us")
    start = (real[:, 0] - real[:, 0].min()) / 100.0
    end = (real[:, 1] - real[:, 0].min()) / 100.0
    print(f"waves start over {start.max():.2f} us (mean {start.mean():.2f}); the last one ends {end.max():.2f} us after the first started")
    if args.slowest:
        # the waves that end last set the launch's time: their own points, in us since their entry
        print(f"the {args.slowest} waves that end last (entry in us after the first wave's, then us since entry at every point reached):")
        for w in np.argsort(end)[::-1][:args.slowest]:
            pts = " ".join(f"{i}:{rel[w, i] / 100.0:.2f}" for i in (1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 15, 13, 14) if ticks[w, i] != 0)
            print(f"  entry {start[w]:.2f}  {pts}  exit {life_us[w]:.2f}")


SEGMENTS = ["wait for the step's tile (vmcnt)", "workgroup barrier", "plan published, next tile requested (scalar bookkeeping)",
            "Q fragments read", "leaf tile, own rows", "leaf tile, other waves' rows", "ancestor tile computed",
            "ancestor tile skipped (no query of the wave attends)", "normalise, store, next pair"]


def stream_shares(lib, launch, flush, cfg):
    """One launch of the streaming kernel: cycles per kind of segment, summed per wave by the kernel itself."""
    lib.fsta_stream_profile_buffer.restype, lib.fsta_stream_profile_buffer.argtypes = ctypes.c_int, [ctypes.c_void_p]
    waves = cfg.block_m // 16
    buf = torch.zeros((512 * waves * 20,), dtype=torch.int64, device=flush.device)
    assert lib.fsta_stream_profile_buffer(None) == 0
    launch(_lib.FLAG_STREAM)
    flush.fill_(1)
    torch.cuda.synchronize()
    assert lib.fsta_stream_profile_buffer(buf.data_ptr()) == 0
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    launch(_lib.FLAG_STREAM)
    ev1.record()
    torch.cuda.synchronize()
    print(f"kernel: {lib.fsta_last_attention_kernel().decode()} (instrumented), {ev0.elapsed_time(ev1) * 1e3:.1f} us")
    data = buf.cpu().numpy().reshape(-1, 20)
    data = data[data[:, 10:].sum(1) != 0]
    cyc, cnt = data[:, :10].sum(0), data[:, 10:].sum(0)
    n = data.shape[0]
    print(f"workload: {cfg.name}; {n} waves; shader-clock cycles per wave: {cyc.sum() / n:.0f}")
    print(f"{'segment':<60}{'share':>8}{'times per wave':>16}{'cycles each':>14}")
    for i, name in enumerate(SEGMENTS):
        print(f"{name:<60}{100.0 * cyc[i] / cyc.sum():>7.1f}%{cnt[i] / n:>16.1f}{cyc[i] / max(cnt[i], 1):>14.0f}")


if __name__ == "__main__":
    main()
