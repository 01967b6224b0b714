"""CPU checks of the C-ABI library: it loads, exports every symbol include/rwkv_hip.h declares,
and validates arguments on the host without touching a GPU."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "rwkv_hip.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b(rwkv_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


@pytest.fixture(scope="module")
def lib():
    from rwkvstic_amd import _native
    if not os.path.exists(_native.LIB_PATH):
        from rwkvstic_amd import build
        build.build(verbose=False)
    return _native.lib()


def test_header_and_binding_agree(lib):
    from rwkvstic_amd import _native
    assert _declared() == sorted(_native.EXPORTS)


def test_every_declared_symbol_is_exported(lib):
    for name in _declared():
        assert hasattr(lib, name), name
    assert lib.rwkv_version() >= 100


def test_host_side_validation_without_gpu(lib):
    # pure host functions
    assert lib.rwkv_packed_bytes(2560, 2560) == 2560 * 2560
    assert lib.rwkv_packed_bytes(130, 77) == 10 * 2 * 1024
    assert lib.rwkv_packed_bytes(0, 5) == 0
    assert lib.rwkv_mm8_workspace_bytes(2560, 2560, 3) == 20 * 3 * 2560 * 4
    # argument errors are reported before anything is launched
    assert lib.rwkv_quantize_u8(None, None, 4, 4, None, None, None) == -1
    assert b"null" in lib.rwkv_last_error()
    assert lib.rwkv_mm8_packed(None, 3, 128, 8, 16, 16, 16, 16, None, None, 16) == -3
    assert lib.rwkv_mm8_packed(None, 1, 128, 8, 16, 8, 16, 16, None, None, 16) == -2     # packed misaligned
    assert lib.rwkv_mm8_one(None, 128, 8, 16, 16, 4, 16, 16, None, 0) == -1               # stride < n_out
    assert lib.rwkv_mm8_one(None, 128, 8, 16, 16, 8, 16, 16, None, 0) == -4               # no workspace
    assert lib.rwkv_model_create(None, None) == -1
    assert lib.rwkv_model_workspace_bytes(None, 1) == 0


def test_generated_back_wave_program_is_current():
    """csrc/rwkv_decode_back.inc is generated; the committed file must be what the generator writes."""
    import subprocess
    import sys
    csrc = os.path.join(ROOT, "rwkvstic_amd", "csrc")
    env = {k: v for k, v in os.environ.items() if k != "RWKV_BACK_WINDOW"}
    out = subprocess.run([sys.executable, os.path.join(csrc, "gen_decode_back.py")], capture_output=True, text=True,
                         check=True, env=env).stdout
    assert out == open(os.path.join(csrc, "rwkv_decode_back.inc")).read()


def test_single_token_kernels_do_not_spill_ring_registers():
    """The back-wave program reloads fixed registers in place behind the compiler's back; that is only sound while
    the compiler neither spills nor copies them, i.e. while the asm statement owns them outright.  The check here
    is on the source: every register of the ring is on the statement's clobber list."""
    inc = open(os.path.join(ROOT, "rwkvstic_amd", "csrc", "rwkv_decode_back.inc")).read()
    for block in inc.split("template <> struct BackCfg<")[1:]:
        regs = set(int(x) for x in re.findall(r"global_load_dwordx4 v\[(\d+):", block))
        regs |= set(r + i for r in list(regs) for i in range(4))
        clob = set(int(x) for x in re.findall(r'"v(\d+)"', block))
        assert regs and regs <= clob
