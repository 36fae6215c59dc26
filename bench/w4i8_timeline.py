#!/usr/bin/env python3
"""Where the time goes inside w4_gemm_i8_kernel: wall-clock stamps of every wave at fixed points.

    make -C bench librumus_timers.so && python bench/w4i8_timeline.py [m] [k] [n] [perm]

Runs the INT4 matmul (group 128, symmetric, weights rotating over copies so that they come from HBM)
on the instrumented build of the library and prints, per stamp, the spread over all waves of the last
launch in microseconds since the first wave started: start, issued (all of the wave's first loads are
queued), chunk0 (first chunk multiplied and folded), loop_end, reduced (partial tiles in LDS, barrier passed).
Then the same for w4_i8_prepare_kernel, which turns the activations into digit planes before it: start,
staged (with `perm`, act-order: the row is in LDS), maxed (largest magnitude of the share known), end.
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

use_perm = "perm" in sys.argv
argv = [a for a in sys.argv if a != "perm"]
m = int(argv[1]) if len(argv) > 1 else 16
k = int(argv[2]) if len(argv) > 2 else 4096
n = int(argv[3]) if len(argv) > 3 else 11008
G = 128
_lib.call("rumus_hip_init", 0)
dev = torch.device("cuda:0")
gen = torch.Generator(device=dev).manual_seed(2)
w = torch.randn((k, n), generator=gen, device=dev) * 0.02
packed, scales, zp = ops.w4_quantize_pack(w, G, symmetric=True)
perm = None
if use_perm:
    g_idx = (torch.randperm(k, generator=gen, device=dev) // G).to(torch.int32)
    packed, perm = ops.w4_actorder_prepare(packed, g_idx, G)
copies = [(packed.clone(), scales.clone(), zp.clone()) for _ in range(max(2, 600_000_000 // (k * n // 2)))]
x = torch.randn((m, k), generator=gen, device=dev)
y = torch.empty((m, n), dtype=torch.float32, device=dev)
for _ in range(3):
    for p, s, z in copies:
        ops.qmatmul_int4_perm(x, p, s, z, k, G, perm=perm, out=y)
torch.cuda.synchronize()
buf = np.zeros(512 * 8 * 8, dtype=np.uint64)        # the first 512 workgroups of the last launch
assert _lib.lib().rumus_dbg_w4i8_stamps(buf.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(buf.size)) == 0
st = buf.reshape(-1, 8, 8).astype(np.int64)
st = st[st[:, 0, 0] > 0]                       # workgroups that ran
rel = (st - st[:, :, 0].min()) * 0.01          # 100 MHz ticks -> us
print(f"{m} x {k} x {n}: {st.shape[0]} workgroups of 8 waves recorded")
for i, name in enumerate(["start", "issued", "chunk0", "loop_end", "reduced"]):
    v = rel[:, :, i]
    print(f"{name:9s} min {v.min():6.2f}  median {np.median(v):6.2f}  p90 {np.percentile(v, 90):6.2f}  max {v.max():6.2f}")

buf = np.zeros(256 * 8 * 8, dtype=np.uint64)        # the first 256 workgroups of the last prepare launch
assert _lib.lib().rumus_dbg_w4i8_prep_stamps(buf.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(buf.size)) == 0
st = buf.reshape(-1, 8, 8).astype(np.int64)[:, :, :4]
st = st[(st[:, :, 0] > 0)]                     # waves that ran (one wave per workgroup without perm)
rel = (st - st[:, 0].min()) * 0.01
print(f"w4_i8_prepare_kernel{' (act-order)' if use_perm else ''}: {st.shape[0]} waves recorded")
for i, name in enumerate(["start", "staged", "maxed", "end"]):
    v = rel[:, i]
    print(f"{name:9s} min {v.min():6.2f}  median {np.median(v):6.2f}  p90 {np.percentile(v, 90):6.2f}  max {v.max():6.2f}")
