"""Issue rate of the bf16 matrix instructions on one SIMD, alone and with vector-ALU work between them.

    python -m fstattention_amd.build --timeline        # builds libfsta_timeline.so (holds the probe kernels)
    python -m fstattention_amd.mfma_rate

Every wave runs rounds of 8 matrix instructions into 1..8 accumulators in turn, each followed by 0..8
independent multiply-adds; one or two waves per SIMD on every SIMD of the GPU.  Each case is timed twice:
one launch on an idle GPU (about 0.2 ms) and the last of 60 launches back to back (about 10 ms of the same
load before it), because the clock the GPU holds under a load depends on how long the load lasts.  Printed:
nanoseconds per matrix instruction and SIMD, the chip-wide TFLOP/s that rate amounts to, and the shader clock
the first wave saw (its cycle counter against the constant 100 MHz clock).  Measuring tool; the regular library
has no such code.
"""
from __future__ import annotations

import ctypes
import os
import time

import torch

from .build import TIMELINE_LIB_PATH

CASES = [  # (shape, accumulators, multiply-adds per matrix instruction)
    (16, 1, 0), (16, 2, 0), (16, 4, 0), (16, 8, 0), (32, 1, 0), (32, 4, 0),
    (0, 0, 2), (0, 0, 4), (0, 0, 8),
    (16, 1, 4), (16, 8, 2), (16, 8, 4), (16, 8, 8), (32, 4, 4), (32, 4, 8),
]
ITERS = 2000
SUSTAINED_LAUNCHES = 60
SIMDS = 1024


def main():
    if not os.path.exists(TIMELINE_LIB_PATH):
        raise SystemExit(f"{TIMELINE_LIB_PATH} is missing: python -m fstattention_amd.build --timeline")
    lib = ctypes.CDLL(TIMELINE_LIB_PATH)
    probe = lib.fsta_probe_mfma_rate
    probe.restype = ctypes.c_int
    probe.argtypes = [ctypes.c_int32] * 5 + [ctypes.c_void_p] * 3
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    g = torch.Generator().manual_seed(5)
    # bf16 pairs with random mantissas around +-1 (switching activity of real data, no infinities)
    words = torch.randint(0, 256, (2048, 2), generator=g, dtype=torch.int64)
    data = ((0x3F00 | words[:, 0]) | ((0xBF00 | words[:, 1]) << 16)).to(torch.int32).to(dev)
    out = torch.empty((2 * 256 * 256 + 2,), dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    print(f"{'case':58s} {'waves/SIMD':>10s} | {'one launch: ns':>14s} {'TFLOP/s':>8s} {'GHz':>5s} | {'sustained: ns':>13s} {'TFLOP/s':>8s} {'GHz':>5s}")
    for shape, accs, valu in CASES:
        for waves in (1, 2):
            def launch(iters):
                rc = probe(shape, accs, valu, waves, iters, data.data_ptr(), out.data_ptr(), stream)
                assert rc == 0, lib.fsta_last_error()

            def timed(before):
                for _ in range(before):
                    launch(ITERS)
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                launch(ITERS)
                e1.record()
                torch.cuda.synchronize()
                steps = ITERS * 8 * waves               # matrix instructions (or groups of multiply-adds) per SIMD
                cycles, ticks = out[256 * 256 * waves:256 * 256 * waves + 2].tolist()
                return e0.elapsed_time(e1) * 1e6 / steps, cycles / (ticks * 10.0) if ticks else 0.0

            launch(10)
            torch.cuda.synchronize()
            time.sleep(0.05)
            ns1, ghz1 = timed(0)
            ns2, ghz2 = timed(SUSTAINED_LAUNCHES - 1)
            flop = {16: 16384, 32: 32768, 0: 0}[shape]
            name = (f"{'16x16x32' if shape == 16 else '32x32x16'} bf16, {accs} accumulator{'s' if accs > 1 else ''} in turn"
                    if shape else "vector ALU alone:")
            name += f", {valu} multiply-adds each" if valu and shape else (f" {valu} multiply-adds" if valu else "")
            tf = lambda ns: SIMDS * flop / ns / 1e3 if flop else 0
            print(f"{name:58s} {waves:10d} | {ns1:14.2f} {tf(ns1):8.0f} {ghz1:5.2f} | {ns2:13.2f} {tf(ns2):8.0f} {ghz2:5.2f}")


if __name__ == "__main__":
    main()
