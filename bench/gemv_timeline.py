#!/usr/bin/env python3
"""Where the time goes inside the decode GEMV (w4_gemv_dot8_kernel): wall-clock stamps of every wave.

    make -C bench librumus_timers.so && python bench/gemv_timeline.py [k] [n]

Runs the one-row INT4 matmul of the headline benchmark (group 128, decode layout, 64 weight sets in
rotation so that every launch reads its weights from HBM) on the instrumented build of the library and
prints, per stamp, the spread over all waves of the last launch in microseconds since its first wave
started: start, planes (the activations of the wave's chunk are nibble planes in registers), dots (every
weight word has arrived and is multiplied), reduced (wave sum in LDS), barrier (passed), stored.  The
launch-to-launch time of the same loop on the product build is what bench.py reports; an empty launch
and a launch that only reads the same bytes are measured by bench/probe_stream.
"""
import ctypes
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import numpy as np
import torch

from rumus_amd import _lib

_lib.LIB_PATH = os.path.join(ROOT, "bench", "librumus_timers.so")
from rumus_amd import ops  # noqa: E402  (binds to the instrumented library)

k = int(sys.argv[1]) if len(sys.argv) > 1 else 4096
n = int(sys.argv[2]) if len(sys.argv) > 2 else 4096
G = 128
_lib.call("rumus_hip_init", 0)
dev = torch.device("cuda:0")
gen = torch.Generator(device=dev).manual_seed(0)
sets = []
for _ in range(64):
    w = torch.randn((k, n), generator=gen, device=dev) * 0.02
    sets.append(ops.w4_decode_layout(*ops.w4_quantize_pack(w, G), G))
    del w
x = torch.randn((1, k), generator=gen, device=dev)
y = torch.empty((1, n), dtype=torch.float32, device=dev)
for _ in range(3):
    for p, s, z in sets:
        ops.qmatmul_int4_decode(x, p, s, z, k, G, out=y)
torch.cuda.synchronize()
buf = np.zeros(256 * 8 * 8, dtype=np.uint64)        # the first 256 workgroups of the last launch
assert _lib.lib().rumus_dbg_d8_stamps(buf.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(buf.size)) == 0
st = buf.reshape(-1, 8, 8).astype(np.int64)[:, :, :6]
st = st[st[:, 0, 0] > 0]                       # workgroups that ran
t0 = st[:, :, 0].min()
rel = (st - t0) * 0.01                         # 100 MHz ticks -> us
print(f"1 x {k} x {n}: {st.shape[0]} workgroups of 8 waves recorded")
for i, name in enumerate(["start", "planes", "dots", "reduced", "barrier", "stored"]):
    v = rel[:, :, i]
    v = v[st[:, :, i] > 0]
    print(f"{name:9s} min {v.min():6.2f}  median {np.median(v):6.2f}  p90 {np.percentile(v, 90):6.2f}  max {v.max():6.2f}")
d = rel[:, :, 2].max(axis=1) - rel[:, :, 2].min(axis=1)
print(f"dots, last wave of a workgroup behind its first: median {np.median(d):.2f}  max {d.max():.2f}")
tail = rel[:, :, 5].max(axis=1) - rel[:, :, 2].max(axis=1)
print(f"stored behind the workgroup's last dots: median {np.median(tail):.2f}  max {tail.max():.2f}")
print("by wave of the workgroup (median over workgroups): start, planes, dots, since the workgroup's first wave started")
wg0 = st[:, :, 0].min(axis=1, keepdims=True)
for w in range(8):
    print(f"  wave {w}: " + "  ".join(f"{np.median((st[:, w, i] - wg0[:, 0]) * 0.01):5.2f}" for i in (0, 1, 2)))
