"""Host-only checks of the workspace sizing of the many-row products: whatever kernel variant and number of
contraction splits the launch plan picks, the integer totals it writes (one slice per split and product) fit
the buffer the sizing functions reserve.  Nothing is launched; no GPU needed."""
import ctypes as C
import os

import pytest


@pytest.fixture(scope="module")
def lib():
    import shutil
    from rwkvstic_amd import _native
    if not os.path.exists(_native.LIB_PATH):
        if not (shutil.which("hipcc") or os.path.exists("/opt/rocm/bin/hipcc")):
            pytest.skip("librwkv_hip.so is not built and there is no hipcc to build it with")
        from rwkvstic_amd import build
        build.build(verbose=False)
    return _native.lib()


def _plan(lib, T, K, N, n):
    plan = (C.c_int * 4)()
    tot = C.c_size_t()
    assert lib.rwkv_gemm8_plan(T, K, N, n, C.byref(plan), C.byref(tot)) == 0, lib.rwkv_last_error()
    return tuple(plan), tot.value


ROWS = list(range(1, 40)) + [47, 48, 63, 64, 65, 100, 127, 128, 129, 255, 256, 257, 300, 400, 511, 512, 513, 640,
                             700, 768, 769, 800, 832, 896, 960, 961, 1000, 1023, 1024]
WIDTHS = [16, 64, 72, 256, 512, 768, 1024, 2048, 2560, 3072, 4096, 5120, 10240, 20480, 50277]
DEPTHS = [64, 512, 1024, 2560, 5120, 10240, 20480]


def test_totals_buffer_holds_every_slice(lib):
    worst = 0
    for T in ROWS:
        for N in WIDTHS:
            slice_bytes = -(-T // 4) * 4 * (-(-N // 16) * 16) * 8
            for K in DEPTHS:
                for n in (1, 2, 3):
                    (kind, gx, gy, split), tot = _plan(lib, T, K, N, n)
                    assert 1 <= split <= 8 and kind in (0, 1, 2, 3)
                    assert split * slice_bytes <= tot, (T, K, N, n, kind, split, tot)
                    worst = max(worst, split)
    assert worst > 1          # the sweep does reach split contractions


def test_split_contractions_are_where_the_grid_is_small(lib):
    """A split contraction costs a second launch, so only grids far below the device split: [800 x 2560] x
    [2560 x 2560] takes the 64 x 160 variant (208 workgroups) unsplit with the tail in its epilogue, the same
    product for 250 rows (80 workgroups of 64 x 128) splits in two, for 60 rows (20 workgroups) in four (parts of
    at least 8 contraction blocks)."""
    (kind, gx, gy, split), tot = _plan(lib, 800, 2560, 2560, 1)
    assert kind == 3 and split == 1 and gx * gy == 208
    (kind, gx, gy, split), tot = _plan(lib, 250, 2560, 2560, 1)
    assert kind == 2 and split == 2 and gx * gy == 80
    assert split * 252 * 2560 * 8 <= tot
    (kind, gx, gy, split), tot = _plan(lib, 60, 2560, 2560, 1)
    assert kind == 2 and split == 4 and split * 60 * 2560 * 8 <= tot
    # a contraction of 200 blocks and more splits once while the grid is below the device: the ffn value product of
    # the 14B shape on a 256-token chunk (160 workgroups), not the same width's [5120 x 5120] products
    (kind, gx, gy, split), tot = _plan(lib, 256, 20480, 5120, 1)
    assert kind == 2 and gx * gy == 160 and split == 2 and split * 256 * 5120 * 8 <= tot
    assert _plan(lib, 256, 5120, 5120, 1)[0][3] == 1


def test_gemm8_workspace_covers_quantiser_scratch(lib):
    """A few rows of a long contraction are quantised in parts whose records sit in the totals area."""
    for T in (1, 4, 8):
        for K in (8192, 20480, 131072, 1 << 20):
            need = T * -(-K // (4 * 256 * 3)) * 16
            fixed = 3 * (-(-T * 8 // 256) * 256) + (-(-(-(-T // 4) * (K // 64) * 1024) // 256) * 256)
            assert lib.rwkv_gemm8_workspace_bytes(T, K, 16) - fixed >= need, (T, K)
