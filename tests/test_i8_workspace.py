"""The INT8 GEMM's workspace arithmetic, replayed on the host (no GPU): what the dispatch asks for never
exceeds the documented bound, and the Q8 matmul that nests an INT8 GEMM reserves room for it."""
import itertools

import pytest

from rumus_amd import _lib

MIB = 1 << 20


@pytest.fixture(scope="module")
def library():
    return _lib.lib()


def test_workspace_size_never_exceeds_the_documented_bound(library):
    # include/rumus_hip.h: at most min(32 * m * n, 16 MiB)
    rows = sorted(set(list(range(1, 70)) + [96, 127, 128, 129, 200, 255, 256, 257, 383, 384, 392, 500, 517, 520, 1023,
                                            1024, 1500, 2047, 2048, 2068, 2080, 2081, 3000, 4096, 6144, 8204, 8192 * 4,
                                            32832]))
    worst = 0
    for m, k, n in itertools.product(rows, (64, 256, 1024, 4096, 11008, 16384), (16, 64, 352, 4096, 11008, 14336, 22016)):
        need = library.rumus_hip_i8_gemm_workspace_size(m, k, n)
        assert need <= min(32 * m * n, 16 * MIB), (m, k, n, need)
        worst = max(worst, need)
    assert worst == 16 * MIB                       # the bound is reached (256 x 11008 x 4096: 8 shares of 128 x 128 tiles)


def test_row_split_remainders_are_counted(library):
    # 2080 rows x 11008 columns, K = 11008: 2048 rows of wide blocks (no workspace) + 32 rows that share K over
    # workgroups; the size of the whole is the size of the remainder, not 0
    assert library.rumus_hip_i8_gemm_workspace_size(2048, 11008, 11008) == 0
    rest = library.rumus_hip_i8_gemm_workspace_size(32, 11008, 11008)
    assert rest > 0
    assert library.rumus_hip_i8_gemm_workspace_size(2080, 11008, 11008) == rest
    for m in (2068, 2072, 2076, 2080):
        assert library.rumus_hip_i8_gemm_workspace_size(m, 11008, 11008) > 0


def test_resident_activation_kernel_needs_nothing(library):
    # 5 to 64 rows with K of 3072 to 4096 (to 8192 up to 32 rows, to 12288 up to 16): one launch, no partial sums in memory
    for m, k in ((5, 4096), (32, 4096), (64, 3072), (64, 4096), (32, 8192), (16, 11008), (16, 12288)):
        assert library.rumus_hip_i8_gemm_workspace_size(m, k, 11008) == 0, (m, k)
    assert library.rumus_hip_i8_gemm_workspace_size(2080, 4096, 11008) == 0   # 2048 rows of wide blocks + 32 resident


def test_degenerate_shapes_need_nothing(library):
    assert library.rumus_hip_i8_gemm_workspace_size(0, 4096, 4096) == 0
    assert library.rumus_hip_i8_gemm_workspace_size(64, 4096, 0) == 0
    assert library.rumus_hip_i8_gemm_workspace_size(64, 24, 64) == 0      # k % 16 != 0 is refused by the call itself
    assert library.rumus_hip_i8_gemm_workspace_size(1, 4096, 11008) == 0  # decode kernels take no workspace
