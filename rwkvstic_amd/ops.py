"""Operator-level host interface: torch tensors in, HIP kernels underneath.

``mm8_one`` / ``mm8_three`` / ``wkv_forward`` mirror the reference's native
operators ``torch.ops.rwkv.*`` (reference
src/rwkvstic/agnostic/backends/cuda/wrapper.cpp:45-127): same names, argument
order and in-place semantics.  ``register_torch_ops()`` publishes them under
the same ``rwkv::`` namespace so reference-style modules resolve them.

Every function requires CUDA (ROCm) tensors and raises on anything else;
nothing here falls back to torch arithmetic.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _native as N

_scratch: dict = {}


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _req(t: torch.Tensor, dtype, name: str) -> None:
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise ValueError(f"{name} must be a CUDA tensor")
    if t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")


def _contig(t: torch.Tensor, name: str) -> None:
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


def _workspace(nbytes: int, device) -> torch.Tensor:
    """Grow-only per-device scratch for the reference-layout operators."""
    key = (device.index if device.index is not None else torch.cuda.current_device())
    buf = _scratch.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _scratch[key] = buf
    return buf


# ---------------------------------------------------------------- reference operators
def _mm8_dtype(x: torch.Tensor, others, what: str) -> torch.dtype:
    """float32 or float64, shared by x, y and r (the dispatch of wrapper.cpp:58-60)."""
    if x.dtype not in (torch.float32, torch.float64):
        raise TypeError(f"{what}: x, y, r must be float32 or float64, got {x.dtype}")
    for t in others:
        _req(t, x.dtype, "x/y/r")
    return x.dtype


def mm8_one(N_in: int, M_out: int, x: torch.Tensor, w: torch.Tensor, y: torch.Tensor, r: torch.Tensor) -> None:
    """``y[k] += sum_j x[j]*(w[j,k]*r[j])``; argument meaning of wrapper.cpp:52-54 (N=in, M=out); x, y, r all
    float32 or all float64 (wrapper.cpp:60-77)."""
    dt = _mm8_dtype(x, (x, y, r), "mm8_one"); _req(w, torch.uint8, "w")
    if x.dim() != 1 or x.stride(0) != 1 or y.stride(0) != 1 or w.dim() != 2 or w.stride(1) != 1:
        raise ValueError("mm8_one: x, y need unit stride and w.stride(1) == 1 (wrapper.cpp:55-57)")
    if x.numel() < N_in or r.numel() < N_in or y.numel() < M_out or w.shape[0] < N_in or w.shape[1] < M_out:
        raise ValueError("mm8_one: tensor smaller than (N, M)")
    L = N.lib()
    f64 = dt == torch.float64
    ws = _workspace((L.rwkv_mm8_f64_workspace_bytes if f64 else L.rwkv_mm8_workspace_bytes)(N_in, M_out, 1), x.device)
    N.check((L.rwkv_mm8_one_f64 if f64 else L.rwkv_mm8_one)(_stream(), N_in, M_out, x.data_ptr(), w.data_ptr(), w.stride(0),
                                                            y.data_ptr(), r.data_ptr(), ws.data_ptr(), ws.numel()))


def mm8_three(N_in: int, M_out: int, x0, x1, x2, w0, w1, w2, y0, y1, y2, r0, r1, r2) -> None:
    """Three ``mm8_one`` problems in one call (wrapper.cpp:82-86); float32 or float64 like ``mm8_one``."""
    dt = _mm8_dtype(x0, (x0, x1, x2, y0, y1, y2, r0, r1, r2), "mm8_three")
    for t in (x0, x1, x2, y0, y1, y2, r0, r1, r2):
        if t.stride(0) != 1:
            raise ValueError("mm8_three: x, y, r need unit stride")
    for t in (w0, w1, w2):
        _req(t, torch.uint8, "w")
        if t.dim() != 2 or t.stride(1) != 1 or t.shape[0] < N_in or t.shape[1] < M_out:
            raise ValueError("mm8_three: w must be [>=N, >=M] with unit inner stride")
    L = N.lib()
    f64 = dt == torch.float64
    ws = _workspace((L.rwkv_mm8_f64_workspace_bytes if f64 else L.rwkv_mm8_workspace_bytes)(N_in, M_out, 3), x0.device)
    N.check((L.rwkv_mm8_three_f64 if f64 else L.rwkv_mm8_three)(
        _stream(), N_in, M_out, x0.data_ptr(), x1.data_ptr(), x2.data_ptr(),
        w0.data_ptr(), w0.stride(0), w1.data_ptr(), w1.stride(0), w2.data_ptr(), w2.stride(0),
        y0.data_ptr(), y1.data_ptr(), y2.data_ptr(),
        r0.data_ptr(), r1.data_ptr(), r2.data_ptr(), ws.data_ptr(), ws.numel()))


def wkv_forward(B: int, T: int, C: int, w, u, k, v, y, aa, bb, pp) -> None:
    """float64 WKV with the reference's state convention (wrapper.cpp:45-50)."""
    for name, t in (("w", w), ("u", u), ("k", k), ("v", v), ("y", y), ("aa", aa), ("bb", bb), ("pp", pp)):
        _req(t, torch.float64, name); _contig(t, name)
    if k.numel() < B * T * C or v.numel() < B * T * C or y.numel() < B * T * C:
        raise ValueError("wkv_forward: k/v/y smaller than B*T*C")
    if min(aa.numel(), bb.numel(), pp.numel()) < B * C or min(w.numel(), u.numel()) < C:
        raise ValueError("wkv_forward: state or w/u too small")
    N.check(N.lib().rwkv_wkv_forward_f64(_stream(), B, T, C, w.data_ptr(), u.data_ptr(), k.data_ptr(),
                                         v.data_ptr(), y.data_ptr(), aa.data_ptr(), bb.data_ptr(), pp.data_ptr()))


_registered = False


def register_torch_ops() -> None:
    """Publish ``torch.ops.rwkv.{wkv_forward,mm8_one,mm8_three}`` with the
    reference's schemas (wrapper.cpp:131-141: TORCH_LIBRARY(rwkv, m))."""
    global _registered
    if _registered:
        return
    lib = torch.library.Library("rwkv", "DEF")
    lib.define("wkv_forward(int B, int T, int C, Tensor(a!) w, Tensor(b!) u, Tensor(c!) k, Tensor(d!) v, "
               "Tensor(e!) y, Tensor(f!) aa, Tensor(g!) bb, Tensor(h!) pp) -> ()")
    lib.define("mm8_one(int N, int M, Tensor(a!) x, Tensor(b!) w, Tensor(c!) y, Tensor(d!) r) -> ()")
    lib.define("mm8_three(int N, int M, Tensor(a!) x, Tensor(b!) x1, Tensor(c!) x2, Tensor(d!) w, Tensor(e!) w1, "
               "Tensor(f!) w2, Tensor(g!) y, Tensor(h!) y1, Tensor(i!) y2, Tensor(j!) r, Tensor(k!) r1, "
               "Tensor(l!) r2) -> ()")
    lib.impl("wkv_forward", wkv_forward, "CUDA")
    lib.impl("mm8_one", mm8_one, "CUDA")
    lib.impl("mm8_three", mm8_three, "CUDA")
    register_torch_ops._lib = lib     # keep alive
    _registered = True


# ---------------------------------------------------------------- quantiser / layouts
def quantize(weight: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``weight[out, in]`` float32 -> ``(codes[in, out] uint8, range[in] float32, offset[in] float64)``
    (MM8.QuantizeMatrix, matmul.py:24-40)."""
    _req(weight, torch.float32, "weight"); _contig(weight, "weight")
    n_out, n_in = weight.shape
    codes = torch.empty((n_in, n_out), dtype=torch.uint8, device=weight.device)
    rng = torch.empty(n_in, dtype=torch.float32, device=weight.device)
    off = torch.empty(n_in, dtype=torch.float64, device=weight.device)
    N.check(N.lib().rwkv_quantize_u8(_stream(), weight.data_ptr(), n_out, n_in,
                                     codes.data_ptr(), rng.data_ptr(), off.data_ptr()))
    return codes, rng, off


def pack(codes: torch.Tensor) -> torch.Tensor:
    """Reference layout ``codes[in, out]`` -> streaming block layout (1-D uint8)."""
    _req(codes, torch.uint8, "codes")
    if codes.dim() != 2 or codes.stride(1) != 1:
        raise ValueError("codes must be 2-D with unit inner stride")
    n_in, n_out = codes.shape
    L = N.lib()
    packed = torch.empty(L.rwkv_packed_bytes(n_in, n_out), dtype=torch.uint8, device=codes.device)
    N.check(L.rwkv_pack_u8(_stream(), codes.data_ptr(), codes.stride(0), n_in, n_out, packed.data_ptr()))
    return packed


def unpack(packed: torch.Tensor, n_in: int, n_out: int) -> torch.Tensor:
    _req(packed, torch.uint8, "packed"); _contig(packed, "packed")
    L = N.lib()
    if packed.numel() < L.rwkv_packed_bytes(n_in, n_out):
        raise ValueError("packed buffer too small")
    codes = torch.empty((n_in, n_out), dtype=torch.uint8, device=packed.device)
    N.check(L.rwkv_unpack_u8(_stream(), packed.data_ptr(), n_in, n_out, codes.data_ptr(), n_out))
    return codes


def pack_m16(codes: torch.Tensor) -> torch.Tensor:
    """Reference layout ``codes[in, out]`` -> 16x64 signed blocks for the matrix-core decode kernel."""
    _req(codes, torch.uint8, "codes")
    if codes.dim() != 2 or codes.stride(1) != 1:
        raise ValueError("codes must be 2-D with unit inner stride")
    n_in, n_out = codes.shape
    L = N.lib()
    packed = torch.empty(L.rwkv_packed_m16_bytes(n_in, n_out), dtype=torch.uint8, device=codes.device)
    N.check(L.rwkv_pack_m16(_stream(), codes.data_ptr(), codes.stride(0), n_in, n_out, packed.data_ptr()))
    return packed


def unpack_m16(packed: torch.Tensor, n_in: int, n_out: int) -> torch.Tensor:
    _req(packed, torch.uint8, "packed"); _contig(packed, "packed")
    L = N.lib()
    if packed.numel() < L.rwkv_packed_m16_bytes(n_in, n_out):
        raise ValueError("packed buffer too small")
    codes = torch.empty((n_in, n_out), dtype=torch.uint8, device=packed.device)
    N.check(L.rwkv_unpack_m16(_stream(), packed.data_ptr(), n_in, n_out, codes.data_ptr(), n_out))
    return codes


def dequant_packed(packed, rng, off, n_in: int, n_out: int) -> torch.Tensor:
    _req(packed, torch.uint8, "packed"); _req(rng, torch.float32, "range"); _req(off, torch.float64, "offset")
    L = N.lib()
    if packed.numel() < L.rwkv_packed_bytes(n_in, n_out) or rng.numel() < n_in or off.numel() < n_in:
        raise ValueError("buffer too small")
    dq = torch.empty((n_in, n_out), dtype=torch.float32, device=packed.device)
    N.check(L.rwkv_dequant_packed(_stream(), packed.data_ptr(), rng.data_ptr(), off.data_ptr(), n_in, n_out,
                                  dq.data_ptr()))
    return dq


# ---------------------------------------------------------------- stand-alone kernels
def mm8_packed(x: torch.Tensor, packed: torch.Tensor, n_in: int, n_out: int,
               r_row: torch.Tensor, m_row: torch.Tensor,
               r_col: Optional[torch.Tensor] = None, m_col: Optional[torch.Tensor] = None,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``y[B, out]`` float64 for ``x[B, in]`` float32, B in {1, 2, 4, 8}."""
    _req(x, torch.float32, "x"); _contig(x, "x")
    _req(packed, torch.uint8, "packed"); _req(r_row, torch.float32, "r_row"); _req(m_row, torch.float64, "m_row")
    if x.dim() != 2 or x.shape[1] != n_in:
        raise ValueError("x must be [B, n_in]")
    L = N.lib()
    if packed.numel() < L.rwkv_packed_bytes(n_in, n_out) or r_row.numel() < n_in or m_row.numel() < n_in:
        raise ValueError("buffer too small")
    for t, nm in ((r_col, "r_col"), (m_col, "m_col")):
        if t is not None:
            _req(t, torch.float32, nm)
            if t.numel() < n_out:
                raise ValueError(f"{nm} too small")
    B = x.shape[0]
    y = out if out is not None else torch.empty((B, n_out), dtype=torch.float64, device=x.device)
    _req(y, torch.float64, "out"); _contig(y, "out")
    N.check(L.rwkv_mm8_packed(_stream(), B, n_in, n_out, x.data_ptr(), packed.data_ptr(), r_row.data_ptr(),
                              m_row.data_ptr(), r_col.data_ptr() if r_col is not None else None,
                              m_col.data_ptr() if m_col is not None else None, y.data_ptr()))
    return y


def mm8_m16(x: torch.Tensor, packed16: torch.Tensor, n_in: int, n_out: int,
            r_row: torch.Tensor, m_row: torch.Tensor,
            r_col: Optional[torch.Tensor] = None, m_col: Optional[torch.Tensor] = None,
            out: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``mm8_packed`` on the matrix cores: ``y[B, out]`` float64 for ``x[B, in]`` float32, any B in 1..8, weights in
    the M16 layout (``pack_m16``); exact integer sums instead of float32 accumulation."""
    _req(x, torch.float32, "x"); _contig(x, "x")
    _req(packed16, torch.uint8, "packed16"); _req(r_row, torch.float32, "r_row"); _req(m_row, torch.float64, "m_row")
    if x.dim() != 2 or x.shape[1] != n_in:
        raise ValueError("x must be [B, n_in]")
    L = N.lib()
    if packed16.numel() < L.rwkv_packed_m16_bytes(n_in, n_out) or r_row.numel() < n_in or m_row.numel() < n_in:
        raise ValueError("buffer too small")
    for t, nm in ((r_col, "r_col"), (m_col, "m_col")):
        if t is not None:
            _req(t, torch.float32, nm)
            if t.numel() < n_out:
                raise ValueError(f"{nm} too small")
    B = x.shape[0]
    y = out if out is not None else torch.empty((B, n_out), dtype=torch.float64, device=x.device)
    _req(y, torch.float64, "out"); _contig(y, "out")
    need = L.rwkv_mm8_m16_workspace_bytes(B, n_in)
    ws = workspace if workspace is not None else torch.empty(max(need, 1), dtype=torch.uint8, device=x.device)
    N.check(L.rwkv_mm8_m16(_stream(), B, n_in, n_out, x.data_ptr(), packed16.data_ptr(), r_row.data_ptr(),
                           m_row.data_ptr(), r_col.data_ptr() if r_col is not None else None,
                           m_col.data_ptr() if m_col is not None else None, y.data_ptr(), ws.data_ptr(), ws.numel()))
    return y


def gemm8(x: torch.Tensor, packed16: torch.Tensor, rng: torch.Tensor, off: torch.Tensor,
          n_in: int, n_out: int) -> torch.Tensor:
    """``y[T, n_out] = x[T, n_in] @ dequantised matrix`` with the single-token arithmetic
    (fp32(x*range) as exact fixed point, integer dot products, float64 zero-point term);
    the T > 1 branch of MM8.forward (matmul.py:56-57) without its bfloat16 rounding."""
    _req(x, torch.float64, "x"); _contig(x, "x")
    _req(packed16, torch.uint8, "packed16"); _req(rng, torch.float32, "range"); _req(off, torch.float64, "offset")
    if x.dim() != 2 or x.shape[1] != n_in:
        raise ValueError("gemm8: x must be [T, n_in]")
    T = x.shape[0]
    L = N.lib()
    if packed16.numel() < L.rwkv_packed_m16_bytes(n_in, n_out) or rng.numel() < n_in or off.numel() < n_in:
        raise ValueError("gemm8: matrix buffers smaller than (n_in, n_out)")
    y = torch.empty((T, n_out), dtype=torch.float64, device=x.device)
    ws = _workspace(L.rwkv_gemm8_workspace_bytes(T, n_in, n_out), x.device)
    N.check(L.rwkv_gemm8(_stream(), T, n_in, n_out, x.data_ptr(), packed16.data_ptr(), rng.data_ptr(),
                         off.data_ptr(), y.data_ptr(), ws.data_ptr(), ws.numel()))
    return y


def wkv_f32(w, u, k, v, aa, bb, pp) -> torch.Tensor:
    """Max-shifted float32 WKV; ``k, v`` are ``[B, T, C]``; state ``[B, C]`` updated in place."""
    for name, t in (("w", w), ("u", u), ("k", k), ("v", v), ("aa", aa), ("bb", bb), ("pp", pp)):
        _req(t, torch.float32, name); _contig(t, name)
    if k.dim() != 3 or v.shape != k.shape:
        raise ValueError("k, v must be [B, T, C]")
    B, T, Cn = k.shape
    if min(aa.numel(), bb.numel(), pp.numel()) < B * Cn or min(w.numel(), u.numel()) < Cn:
        raise ValueError("state or w/u too small")
    y = torch.empty_like(k)
    N.check(N.lib().rwkv_wkv_f32(_stream(), B, T, Cn, w.data_ptr(), u.data_ptr(), k.data_ptr(), v.data_ptr(),
                                 y.data_ptr(), aa.data_ptr(), bb.data_ptr(), pp.data_ptr()))
    return y


def sample_token(logits: torch.Tensor, *, greedy: bool = False, temp: float = 1.0, tau: float = 0.8, end_adj: float = 0.0,
                 seed: int = 0, counter: int = 0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One choice of the device-side sampler (typical.py:1-17; ``logits[0] += end_adj`` in place first,
    rwkvMaster.py:37); the uniform number is a hash of ``(seed, counter)``."""
    _req(logits, torch.float64, "logits"); _contig(logits, "logits")
    out = out if out is not None else torch.empty(1, dtype=torch.int64, device=logits.device)
    N.check(N.lib().rwkv_sample_token(_stream(), logits.data_ptr(), logits.numel(), 1 if greedy else 0, float(temp),
                                      float(tau), float(end_adj), int(seed) & (2 ** 64 - 1), int(counter), out.data_ptr()))
    return out


def argmax(logits: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _req(logits, torch.float64, "logits"); _contig(logits, "logits")
    out = out if out is not None else torch.empty(1, dtype=torch.int64, device=logits.device)
    N.check(N.lib().rwkv_argmax_f64(_stream(), logits.data_ptr(), logits.numel(), out.data_ptr()))
    return out
