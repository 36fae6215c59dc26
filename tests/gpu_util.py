"""Helpers shared by the GPU parity tests."""
import sys

import numpy as np
import torch

RTOL, ATOL = 1e-3, 1e-4   # f32 outputs: rel 1e-3, abs 1e-4 (the reduction order differs from the sequential restatement)


def say(msg: str) -> None:
    """Name the case before the GPU step runs, so a crash names its culprit."""
    print(f"[gpu-case] {msg}", flush=True)
    sys.stdout.flush()


def dev(a: np.ndarray) -> torch.Tensor:
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    return torch.from_numpy(a).cuda()


def host(t: torch.Tensor) -> np.ndarray:
    torch.cuda.synchronize()
    return t.cpu().numpy()


def host_u32(t: torch.Tensor) -> np.ndarray:
    return host(t).view(np.uint32)


def assert_close(got, want, what=""):
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL, err_msg=what)
