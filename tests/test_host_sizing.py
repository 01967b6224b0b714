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


def test_wide_variant_with_split_contraction_is_covered(lib):
    """The 64 x 160 variant has fewer workgroups than the 64 x 128 one for the same product, so it can split the
    contraction where the other would not: [800 x 2560] x [2560 x 2560] is such a case."""
    (kind, gx, gy, split), tot = _plan(lib, 800, 2560, 2560, 1)
    assert kind == 3 and split == 2
    assert split * 800 * 2560 * 8 <= tot


def test_gemm8_workspace_covers_quantiser_scratch(lib):
    """A few rows of a long contraction are quantised in parts whose records sit in the totals area."""
    for T in (1, 4, 8):
        for K in (8192, 20480, 131072, 1 << 20):
            need = T * -(-K // (4 * 256 * 3)) * 16
            fixed = 3 * (-(-T * 8 // 256) * 256) + (-(-(-(-T // 4) * (K // 64) * 1024) // 256) * 256)
            assert lib.rwkv_gemm8_workspace_bytes(T, K, 16) - fixed >= need, (T, K)
