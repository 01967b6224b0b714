"""CPU oracle for the FASTQUANT (fp32i8) RWKV-4 forward path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``rwkvstic_amd/`` may import this
module: it is the checker that the HIP path is compared against (``tests/``,
``__graft_entry__.smoke`` and the ``cpu_baseline`` leg of ``bench.py``), never
the thing measured or shipped.

It restates, in plain torch-on-CPU arithmetic, what the reference's CPU
configuration computes (``config={"devices":[{"device":"cpu","dtype":uint8}],
"custom":False}``): float32 ``@`` on a per-call uint8->float32 cast, float64
elementwise work and state, a Python-loop WKV.  Every function cites the
reference lines it follows (paths relative to ``src/rwkvstic/``).

Pinning status (what, besides a re-reading of the formula, fixes each function;
the checks live in ``tests/test_oracle_*.py``):

* ``quantize_matrix``  – closed-form invariants (code range, per-channel min
  code 0 / max code >= 254, zero mean error per input channel, |err| < range,
  ``range == fp32((max-min)/255)``) and a pure-Python brute force on tiny
  matrices.  The reference holds no golden vectors for it.
* ``mm8_naive``        – equals a float64 dense product on the canonically
  dequantised matrix to float32 accumulation error.
* ``mm8_general_f64``  – the four-vector form (row and column ranges and
  offsets) equals three nested scalar loops on a 3 x 4 matrix, with each of the
  per-column vectors present or absent.
* ``layernorm``        – equals ``torch.nn.functional.layer_norm`` in float64.
* ``wkv_naive``        – equals the O(T^2) direct sum of textbook RWKV-4, the
  max-shifted recurrence ``wkv_stable``, the geometric-series closed form for
  constant input, and is split-invariant in T.
* ``typical_distribution`` – hand-worked kept sets and probabilities for the
  distribution (1/2, 1/4, 1/8, 1/8) at four values of tau and with a
  temperature; uniform logits keep every token.
* ``block_forward`` / ``forward`` – with ``matmul_dtype=float64`` the model equals,
  to 1e-12 (logits and every carried state row, prompt fed in two calls), a
  textbook RWKV-4 written with ``nn.functional`` ops and the direct-sum WKV on
  the canonically dequantised matrices; the same check is shown to fail (by
  >= 1e-3) for swapped mix rows, reversed mix direction, a dropped bonus, a
  changed decay, swapped key/receptance matrices, swapped LayerNorms and
  swapped state rows.  The float32 default differs from that only by the
  accumulation type of the products.  Also: chunk-size invariance and
  ``state[0]/state[1]`` equalling the last LayerNorm outputs.
* No reference-generated vectors exist (the reference has no tests and was not
  imported), so what stays "parity unpinned" is what only its own run could
  show: bit-exact ``(code, range, offset)`` triples from its torch build and
  the attribute tree of its ``.rwkv`` export.
"""
from __future__ import annotations

import math
from typing import Dict, List, Tuple

import torch

Tensor = torch.Tensor


# --------------------------------------------------------------------------
# a8  quantiser  (agnostic/backends/modules/matmul.py:18-40)
# --------------------------------------------------------------------------
def quantize_matrix(weight: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
    """Quantise ``weight[out, in]`` to uint8 with one scale/min per INPUT channel.

    Follows ``MM8.chunkQuantizeMatrix``/``QuantizeMatrix`` (matmul.py:18-40):
    the reduction runs over the output dimension, all arithmetic is float64,
    the code is the truncated quotient, and the mean truncated fraction is
    folded back into the offset.  Returns ``(codes[in,out] uint8 contiguous,
    range[in] float32, offset[in] float64)``.
    """
    x = weight                                # [out, in]
    mini = x.min(0)[0].double()               # [in]      matmul.py:31
    out = x - mini                            # float64   matmul.py:32
    ran = out.max(0)[0].double() / 255        # matmul.py:33
    out = out / ran                           # matmul.py:34
    fract = out.frac().double().mean(0)       # matmul.py:35-36
    offset = mini + fract * ran               # matmul.py:37
    codes = out.t().to(torch.uint8).contiguous()   # trunc toward zero, matmul.py:21
    return codes, ran.to(torch.float32), offset.to(torch.float64)


def dequant_canonical(codes: Tensor, rng: Tensor, offset: Tensor) -> Tensor:
    """``fp32(fp64(code) * fp64(range) + offset)`` laid out ``[in, out]``."""
    return (codes.double() * rng.double()[:, None] + offset[:, None]).to(torch.float32)


# --------------------------------------------------------------------------
# a12  mm8Naive / mm8_3Naive  (matmul.py:124-142)
# --------------------------------------------------------------------------
def mm8_naive(x: Tensor, codes: Tensor, rng: Tensor, offset: Tensor,
              dtype: torch.dtype = torch.float32) -> Tensor:
    """``fp32(x*range) @ fp32(codes) + (x @ offset)[:, None]`` for ``x[T,in]`` float64.

    matmul.py:131: the product ``x*range`` is formed in float64 (float64 times
    float32 promotes), rounded to ``dtype``, multiplied by the ``dtype`` cast of
    the codes with ``dtype`` accumulation, and the float64 zero-point term is
    added last (float32 + float64 -> float64).  ``dtype`` is the reference's
    ``naivedtype`` (matmul.py:183: float32 on the CPU by default; float64 is
    the same network evaluated without accumulation error and is what the
    float32 path is noisy around: for F = 10240 the float32 sum of the
    all-positive relu^2 terms cancels against the zero-point term and loses
    about 1e-4 absolute, by an amount that changes with the BLAS thread count).
    """
    main = (x * rng).to(dtype) @ codes.to(dtype)
    return main + x.mv(offset).reshape(-1, 1)


def mm8_general_f64(x: Tensor, codes: Tensor, r_row: Tensor, m_row: Tensor,
                    r_col: Tensor | None, m_col: Tensor | None) -> Tensor:
    """Float64 dense product on the four-vector dequantisation
    ``dq[j,k] = codes[j,k]*r_row[j]*r_col[k] + m_row[j] + m_col[k]``.

    The reference layout is the special case ``r_col=1, m_col=0``
    (matmul.py:18-40); the general form is the isolated-matvec workload.
    """
    dq = codes.double() * r_row.double()[:, None]
    if r_col is not None:
        dq = dq * r_col.double()[None, :]
    dq = dq + m_row.double()[:, None]
    if m_col is not None:
        dq = dq + m_col.double()[None, :]
    return x.double() @ dq


# --------------------------------------------------------------------------
# a5  LayerNorm  (agnostic/backends/modules/layernorm.py:11-20)
# --------------------------------------------------------------------------
def layernorm(x: Tensor, w: Tensor, b: Tensor) -> Tensor:
    """Biased variance, eps inside the sqrt, float64 (layernorm.py:15-20)."""
    x = x.to(torch.float64)
    d = x - torch.mean(x, dim=1, keepdim=True)
    s = torch.sqrt(torch.mean(d * d, dim=1, keepdim=True) + 1e-5)
    return w * (d / s) + b


# --------------------------------------------------------------------------
# a14/a15  WKV  (modules/wkv.py:23-39, cuda/operators.cu:6-37)
# --------------------------------------------------------------------------
def wkv_naive(w: Tensor, u: Tensor, k: Tensor, v: Tensor,
              aa: Tensor, bb: Tensor, pp: Tensor):
    """Naive (not max-shifted) float64 recurrence; ``w = -exp(time_decay) < 0``.

    wkv.py:31-39: ``y = (aa + e^{u+w+k} v)/(bb + e^{u+w+k})``; the stored state
    is pre-multiplied by ``e^w`` (``aa <- (aa + e^k v) e^w``); ``pp`` is passed
    through untouched.  ``k, v`` are ``[T, C]``.
    """
    T = k.shape[0]
    y = torch.empty_like(k, dtype=torch.float64)
    aa = aa.clone().double()
    bb = bb.clone().double()
    for i in range(T):
        kk = torch.exp(k[i])
        e = torch.exp(u + w + k[i])
        y[i] = (aa + e * v[i]) / (bb + e)
        aa = (aa + kk * v[i]) * torch.exp(w)
        bb = (bb + kk) * torch.exp(w)
    return y, aa, bb, pp


def wkv_stable(w: Tensor, u: Tensor, k: Tensor, v: Tensor,
               aa: Tensor, bb: Tensor, pp: Tensor):
    """Max-shifted recurrence on the reference's pre-multiplied state.

    Same outputs as ``wkv_naive`` in real arithmetic; the carried triple
    ``(aa', bb', pp')`` satisfies ``aa_naive = aa' e^{pp'}``, ``bb_naive =
    bb' e^{pp'}``.  This is the closed form of agnostic/agnosticRwkv.py:68-103
    with the ``e^w`` factor of operators.cu:27-32 folded into the exponents
    (``q = u+w+k`` for the output, ``s = pp'+w``, ``r = k+w`` for the update).
    """
    T = k.shape[0]
    y = torch.empty_like(k, dtype=torch.float64)
    aa = aa.clone().double(); bb = bb.clone().double(); pp = pp.clone().double()
    for i in range(T):
        q = u + w + k[i]
        p = torch.maximum(pp, q)
        e1 = torch.exp(pp - p); e2 = torch.exp(q - p)
        y[i] = (e1 * aa + e2 * v[i]) / (e1 * bb + e2)
        s = pp + w
        r = k[i] + w
        p2 = torch.maximum(s, r)
        e1 = torch.exp(s - p2); e2 = torch.exp(r - p2)
        aa = e1 * aa + e2 * v[i]
        bb = e1 * bb + e2
        pp = p2
    return y, aa, bb, pp


# --------------------------------------------------------------------------
# model container
# --------------------------------------------------------------------------
class QMat:
    """One quantised matrix in the reference layout (matmul.py:12-16)."""

    def __init__(self, weight: Tensor, dtype: torch.dtype = torch.float32):
        self.codes, self.range, self.offset = quantize_matrix(weight.float())
        self.n_in, self.n_out = self.codes.shape
        self.dtype = dtype

    def __call__(self, x: Tensor) -> Tensor:
        return mm8_naive(x, self.codes, self.range, self.offset, self.dtype)

    @classmethod
    def synthetic(cls, n_in: int, n_out: int, gen: torch.Generator, dtype: torch.dtype = torch.float32) -> "QMat":
        """A matrix given directly by random codes, ranges and offsets (what quantising an ~N(0, 0.02) matrix
        yields in size and spread), for timing the arithmetic at sizes where running the quantiser over a whole
        model would dominate the run; the cost of ``__call__`` does not depend on the values."""
        self = cls.__new__(cls)
        seed = int(torch.randint(1, 2 ** 31 - 1, (1,), generator=gen))
        # bytes of a multiplicative hash of the index: filled at memory speed (the random generators take
        # minutes for the 3 GB of a whole model), and as good as random for what the timing needs
        n8 = (n_in * n_out + 7) // 8
        h = (torch.arange(n8, dtype=torch.int64) + seed) * -7046029254386353131
        h ^= h >> 29
        self.codes = h.view(torch.uint8)[:n_in * n_out].reshape(n_in, n_out)
        self.range = torch.rand(n_in, generator=gen, dtype=torch.float32) * 2e-4 + 5e-4
        self.offset = (torch.rand(n_in, generator=gen, dtype=torch.float64) - 0.5) * 0.02 - 0.08
        self.n_in, self.n_out, self.dtype = n_in, n_out, dtype
        return self


class OracleModel:
    """CPU restatement of ``myRWKV`` (agnostic/backends/opt.py:27-84)."""

    def __init__(self, w: Dict[str, Tensor], matmul_dtype: torch.dtype = torch.float32):
        self.matmul_dtype = matmul_dtype
        QMat = lambda t: globals()["QMat"](t, matmul_dtype)   # noqa: E731  (naivedtype, matmul.py:183)
        self.dims = len(w["blocks.0.att.key.weight"])                 # opt.py:96
        self.layers = len([k for k in w if "blocks" in k and "ln1.bias" in k])  # opt.py:97-98
        f64 = torch.float64
        self.emb = w["emb.weight"].clone()                            # emb.py:7
        self.ln_in = (w["blocks.0.ln0.weight"].to(f64), w["blocks.0.ln0.bias"].to(f64))
        self.ln_out = (w["ln_out.weight"].to(f64), w["ln_out.bias"].to(f64))
        self.head = QMat(w["head.weight"])
        self.blocks: List[dict] = []
        for i in range(self.layers):
            p = f"blocks.{i}."
            blk = dict(
                ln1=(w[p + "ln1.weight"].to(f64), w[p + "ln1.bias"].to(f64)),
                ln2=(w[p + "ln2.weight"].to(f64), w[p + "ln2.bias"].to(f64)),
                att_k=QMat(w[p + "att.key.weight"]),
                att_v=QMat(w[p + "att.value.weight"]),
                att_r=QMat(w[p + "att.receptance.weight"]),
                att_o=QMat(w[p + "att.output.weight"]),
                ffn_k=QMat(w[p + "ffn.key.weight"]),
                ffn_r=QMat(w[p + "ffn.receptance.weight"]),
                ffn_v=QMat(w[p + "ffn.value.weight"]),
                # block.py:35-47
                attmix=torch.stack((w[p + "att.time_mix_k"].squeeze(),
                                    w[p + "att.time_mix_v"].squeeze(),
                                    w[p + "att.time_mix_r"].squeeze())).unsqueeze(1).to(f64),
                ffnmix=torch.stack((w[p + "ffn.time_mix_k"].squeeze(),
                                    w[p + "ffn.time_mix_r"].squeeze())).unsqueeze(1).to(f64),
                time_first=w[p + "att.time_first"].squeeze().to(f64),
                time_decay=w[p + "att.time_decay"].squeeze().double().exp().neg(),
            )
            self.blocks.append(blk)
        # opt.py:31-32, 80
        self.emptyState = torch.tensor(
            self.layers * [[[0.0] * self.dims] * 4 + [[-1e30] * self.dims]], dtype=f64)

    @classmethod
    def synthetic(cls, layers: int, C: int, F: int, V: int, seed: int = 0) -> "OracleModel":
        """The network at full depth with every matrix drawn as codes (``QMat.synthetic``) and unit LayerNorms:
        the same arithmetic, op for op, as a quantised checkpoint, built in seconds.  For timing only."""
        g = torch.Generator().manual_seed(seed)
        f64 = torch.float64
        self = cls.__new__(cls)
        self.matmul_dtype = torch.float32
        self.dims, self.layers = C, layers
        self.emb = torch.randn(V, C, generator=g, dtype=torch.float32) * 0.02
        ones, zeros = torch.ones(C, dtype=f64), torch.zeros(C, dtype=f64)
        self.ln_in, self.ln_out = (ones, zeros), (ones, zeros)
        self.head = QMat.synthetic(C, V, g)
        self.blocks = []
        for _ in range(layers):
            self.blocks.append(dict(
                ln1=(ones, zeros), ln2=(ones, zeros),
                att_k=QMat.synthetic(C, C, g), att_v=QMat.synthetic(C, C, g), att_r=QMat.synthetic(C, C, g),
                att_o=QMat.synthetic(C, C, g), ffn_k=QMat.synthetic(C, F, g), ffn_r=QMat.synthetic(C, C, g),
                ffn_v=QMat.synthetic(F, C, g),
                attmix=torch.rand(3, 1, C, generator=g, dtype=f64), ffnmix=torch.rand(2, 1, C, generator=g, dtype=f64),
                time_first=torch.rand(C, generator=g, dtype=f64) * 2 - 1,
                time_decay=(torch.rand(C, generator=g, dtype=f64) * 6 - 5).exp().neg()))
        self.emptyState = torch.tensor(layers * [[[0.0] * C] * 4 + [[-1e30] * C]], dtype=f64)
        return self

    # block.py:56-102
    def block_forward(self, blk: dict, x: Tensor, state: Tensor) -> Tensor:
        T = x.shape[0]
        xy = layernorm(x, *blk["ln1"])
        tc = xy[torch.arange(T) - 1]              # roll by one, block.py:61
        last = tc[0].clone()
        tc[0] = state[0]
        state[0] = last
        mix = xy.unsqueeze(0) * blk["attmix"] + tc.unsqueeze(0) * (1 - blk["attmix"])
        k = blk["att_k"](mix[0]); v = blk["att_v"](mix[1]); r = blk["att_r"](mix[2])
        r = r.sigmoid()
        wkv, aa, bb, pp = wkv_naive(blk["time_decay"], blk["time_first"], k, v,
                                    state[2], state[3], state[4])
        state[2] = aa; state[3] = bb; state[4] = pp
        rz = x + blk["att_o"](wkv * r)
        ddd = layernorm(rz, *blk["ln2"])
        rc = ddd[torch.arange(T) - 1]
        last = rc[0].clone()
        rc[0] = state[1]
        state[1] = last
        fmix = ddd * blk["ffnmix"] + rc * (1 - blk["ffnmix"])
        rf = blk["ffn_r"](fmix[1]).sigmoid()
        kf = blk["ffn_k"](fmix[0]).relu()
        rvm = blk["ffn_v"](torch.square(kf))
        return rvm * rf + rz

    # opt.py:61-76
    def forward(self, tokens, state: Tensor):
        tokens = torch.as_tensor(tokens, dtype=torch.long).reshape(-1)
        x = self.emb[tokens].to(torch.float64)
        x = layernorm(x, *self.ln_in)
        for i, blk in enumerate(self.blocks):
            x = self.block_forward(blk, x, state[i])
        x = layernorm(x, *self.ln_out)
        logits = self.head(x[-1:]).squeeze()
        return logits, state

    def greedy(self, prompt, n_new: int, chunk: int | None = None):
        """Prefill ``prompt`` (optionally in chunks), then greedy-decode ``n_new`` tokens.

        Returns ``(tokens[n_new], logits[n_new+? , V] as list, state)``; the
        first logits entry is the one produced by the last prompt token.
        """
        state = self.emptyState.clone()
        prompt = list(int(t) for t in prompt)
        chunk = chunk or len(prompt)
        logits = None
        for s in range(0, len(prompt), chunk):
            logits, state = self.forward(prompt[s:s + chunk], state)
        toks, all_logits = [], []
        for _ in range(n_new):
            all_logits.append(logits.clone())
            t = int(torch.argmax(logits))
            toks.append(t)
            logits, state = self.forward([t], state)
        all_logits.append(logits.clone())
        return toks, all_logits, state


def typical_distribution(logits: Tensor, temp: float = 1.0, tau: float = 0.95) -> Tensor:
    """The probability vector the reference's ``typical`` sampler hands to ``torch.multinomial``
    (agnostic/samplers/typical.py:5-16; everything but the draw itself), normalised."""
    probs = torch.nn.functional.softmax(logits.float(), dim=-1)          # typical.py:5
    surprise = -torch.log(probs)                                         # :6
    ent = torch.nansum(surprise * probs, dim=-1, keepdim=True)           # :7
    shifted = torch.abs(surprise - ent)                                  # :8
    sorted_ids = torch.argsort(shifted)                                  # :9
    sorted_shifted = shifted[sorted_ids]                                 # :10
    cumulative = torch.cumsum(probs[sorted_ids], dim=-1)                 # :11-12
    cutoff = int((cumulative < tau).sum())                               # :13
    cutoff = min(cutoff, probs.numel() - 1)
    probs = probs.clone()
    probs[shifted > sorted_shifted[cutoff]] = 0                          # :14
    if temp != 1.0:
        probs = probs ** (1.0 / temp)                                    # :15-16
    return (probs / probs.sum()).double()


def state_naive_from_stable(aa: Tensor, bb: Tensor, pp: Tensor):
    """Map a max-shifted triple to the reference's naive pair (float64)."""
    e = torch.exp(pp.double())
    return aa.double() * e, bb.double() * e


def wkv_direct_sum(w: Tensor, u: Tensor, k: Tensor, v: Tensor) -> Tensor:
    """Textbook RWKV-4 WKV from an empty state as an O(T^2) float64 sum:
    ``y_t = (sum_{i<t} e^{(t-1-i)w + k_i} v_i + e^{u+k_t} v_t) /
            (sum_{i<t} e^{(t-1-i)w + k_i} + e^{u+k_t})``.
    Independent of any recurrence; used only to pin ``wkv_naive``.
    """
    T, C = k.shape
    y = torch.empty(T, C, dtype=torch.float64)
    for t in range(T):
        num = torch.exp(u + k[t]) * v[t]
        den = torch.exp(u + k[t])
        for i in range(t):
            e = torch.exp((t - 1 - i) * w + k[i])
            num = num + e * v[i]
            den = den + e
        y[t] = num / den
    return y
