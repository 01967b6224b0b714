"""Pins for the CPU oracle: each check is something the mathematics fixes
independently of the oracle's own formula (closed forms, invariants, library
routines, brute force on tiny inputs)."""
import math

import pytest
import torch

from oracle import rwkv_oracle as O
from rwkvstic_amd import synth

torch.manual_seed(0)


# ---------------------------------------------------------------- quantiser
def _brute_quant(W):
    """Pure-Python loops, float64, no torch arithmetic (W[out][in] lists)."""
    n_out, n_in = len(W), len(W[0])
    codes = [[0] * n_out for _ in range(n_in)]
    rng, off = [0.0] * n_in, [0.0] * n_in
    for j in range(n_in):
        col = [float(W[k][j]) for k in range(n_out)]
        lo, hi = min(col), max(col)
        ran = (hi - lo) / 255
        fr = 0.0
        for k in range(n_out):
            q = (col[k] - lo) / ran
            codes[j][k] = int(q)
            fr += q - int(q)
        rng[j] = ran
        off[j] = lo + (fr / n_out) * ran
    return codes, rng, off


def test_quantiser_brute_force_tiny():
    W = torch.randn(5, 3) * 0.02
    c, r, o = O.quantize_matrix(W)
    bc, br, bo = _brute_quant(W.tolist())
    assert c.tolist() == bc
    assert torch.equal(r, torch.tensor(br, dtype=torch.float64).float())
    assert torch.allclose(o, torch.tensor(bo, dtype=torch.float64), rtol=1e-14, atol=0)


@pytest.mark.parametrize("shape", [(64, 48), (257, 96), (3072, 768)])
def test_quantiser_invariants(shape):
    W = torch.randn(*shape) * 0.02          # [out, in]
    c, r, o = O.quantize_matrix(W)
    assert c.dtype == torch.uint8 and c.shape == (shape[1], shape[0]) and c.is_contiguous()
    assert r.dtype == torch.float32 and o.dtype == torch.float64
    # every input channel uses the whole code range
    assert int(c.min(1)[0].max()) == 0
    assert int(c.max(1)[0].min()) >= 254
    # range is the float32 rounding of (max-min)/255 formed in float64
    ran = (W.max(0)[0].double() - W.min(0)[0].double()) / 255
    assert torch.equal(r, ran.float())
    # dequantisation error: zero mean per input channel, bounded by one step
    dq = c.double() * ran[:, None] + o[:, None]
    err = W.t().double() - dq
    assert err.mean(1).abs().max() < 1e-12
    assert (err.abs() < ran[:, None] * (1 + 1e-9)).all()


def test_quantiser_idempotent_on_grid():
    """A matrix that already lies on a 256-level grid is reproduced exactly."""
    n_in, n_out = 16, 300
    codes = torch.randint(1, 255, (n_in, n_out))
    codes[:, 0] = 0
    codes[:, 1] = 255
    lo = torch.randn(n_in).double()
    step = torch.rand(n_in).double() + 0.5
    # place values half a step above the grid point so truncation is unambiguous
    W = (lo[:, None] + (codes.double() + 0.0) * step[:, None]).t().float().double()
    c, r, o = O.quantize_matrix(W)
    # float32 rounding of W perturbs the quotient by ~1e-7; allow off-by-one only at .0 boundaries
    assert (c.long() - codes).abs().max() <= 1
    dq = O.dequant_canonical(c, r, o).double()
    assert (dq - W.t()).abs().max() < step.max() * 1.01


# ---------------------------------------------------------------- matvec
@pytest.mark.parametrize("T", [1, 5])
def test_mm8_naive_vs_fp64_dense(T):
    W = torch.randn(200, 96) * 0.02
    c, r, o = O.quantize_matrix(W)
    x = torch.randn(T, 96, dtype=torch.float64)
    got = O.mm8_naive(x, c, r, o)
    want = O.mm8_general_f64(x, c, r, o, None, None)
    assert got.dtype == torch.float64 and got.shape == (T, 200)
    # float32 accumulation bound: n * 2^-23 * sum |terms|
    bound = 96 * 2.0 ** -23 * ((x.abs() * r.double()) @ c.double()).max()
    assert (got - want).abs().max() <= bound
    # and it approximates the unquantised product to about one quantisation step
    assert (got - x @ W.t().double()).abs().max() < 0.05


def test_mm8_general_form_against_scalar_loops():
    """The four-vector dequantisation dq[j,k] = code[j,k] r_row[j] r_col[k] + m_row[j] + m_col[k] written out
    element by element on a 3 x 4 matrix, with and without the per-column vectors: pins the r_col / m_col branch
    of the float64 dense product the GPU kernel of the isolated-matvec workload is checked against."""
    g = torch.Generator().manual_seed(5)
    n_in, n_out, B = 3, 4, 2
    codes = torch.randint(0, 256, (n_in, n_out), generator=g, dtype=torch.uint8)
    r_row = torch.rand(n_in, generator=g) * 1e-3 + 1e-4
    m_row = (torch.randn(n_in, generator=g) * 0.01).double()
    r_col = torch.rand(n_out, generator=g) * 1e-3 + 1e-4
    m_col = torch.randn(n_out, generator=g) * 0.01
    x = torch.randn(B, n_in, generator=g, dtype=torch.float64)
    for rc, mc in ((r_col, m_col), (None, None), (r_col, None), (None, m_col)):
        want = torch.zeros(B, n_out, dtype=torch.float64)
        for b in range(B):
            for k in range(n_out):
                acc = 0.0
                for j in range(n_in):
                    dq = float(codes[j, k]) * float(r_row[j]) * (float(rc[k]) if rc is not None else 1.0) \
                        + float(m_row[j]) + (float(mc[k]) if mc is not None else 0.0)
                    acc += float(x[b, j]) * dq
                want[b, k] = acc
        got = O.mm8_general_f64(x, codes, r_row, m_row, rc, mc)
        assert torch.allclose(got, want, rtol=1e-13, atol=1e-15)
    # a transposed or swapped operand must not pass: the column vectors really act on columns
    bad = O.mm8_general_f64(x, codes, r_row, m_row, r_col.flip(0), m_col)
    assert not torch.allclose(bad, O.mm8_general_f64(x, codes, r_row, m_row, r_col, m_col), rtol=1e-6)


# ---------------------------------------------------------------- layernorm
def test_layernorm_matches_torch():
    x = torch.randn(7, 96, dtype=torch.float64) * 3 + 1
    w = torch.randn(96, dtype=torch.float64); b = torch.randn(96, dtype=torch.float64)
    want = torch.nn.functional.layer_norm(x, (96,), w, b, eps=1e-5)
    assert torch.allclose(O.layernorm(x, w, b), want, rtol=1e-12, atol=1e-12)


# ---------------------------------------------------------------- WKV
def _wkv_inputs(T, C, seed=0):
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(T, C, generator=g, dtype=torch.float64)
    v = torch.randn(T, C, generator=g, dtype=torch.float64)
    w = -torch.exp(torch.rand(C, generator=g, dtype=torch.float64) * 9 - 8)
    u = torch.rand(C, generator=g, dtype=torch.float64) * 2 - 1
    z = torch.zeros(C, dtype=torch.float64)
    return w, u, k, v, z.clone(), z.clone(), torch.full((C,), -1e38, dtype=torch.float64)


def test_wkv_naive_vs_direct_sum():
    w, u, k, v, aa, bb, pp = _wkv_inputs(24, 16)
    y, *_ = O.wkv_naive(w, u, k, v, aa, bb, pp)
    assert torch.allclose(y, O.wkv_direct_sum(w, u, k, v), rtol=1e-11, atol=1e-12)


def test_wkv_naive_vs_stable_and_state_relation():
    w, u, k, v, aa, bb, pp = _wkv_inputs(64, 32, seed=1)
    y1, a1, b1, p1 = O.wkv_naive(w, u, k, v, aa, bb, pp)
    y2, a2, b2, p2 = O.wkv_stable(w, u, k, v, aa, bb, pp)
    assert torch.allclose(y1, y2, rtol=1e-11, atol=1e-12)
    an, bn = O.state_naive_from_stable(a2, b2, p2)
    assert torch.allclose(a1, an, rtol=1e-10, atol=1e-300)
    assert torch.allclose(b1, bn, rtol=1e-10, atol=1e-300)
    assert torch.equal(p1, pp)          # naive form passes pp through untouched


def test_wkv_constant_input_closed_form():
    """k_t = k0, v_t = v0: y_t = v0 for all t; bb_T = e^{k0} e^w (1-e^{wT})/(1-e^w)."""
    C, T = 8, 40
    w = -torch.exp(torch.linspace(-3, 0.5, C, dtype=torch.float64))
    u = torch.linspace(-1, 1, C, dtype=torch.float64)
    k0, v0 = 0.3, -1.7
    k = torch.full((T, C), k0, dtype=torch.float64)
    v = torch.full((T, C), v0, dtype=torch.float64)
    z = torch.zeros(C, dtype=torch.float64)
    y, aa, bb, _ = O.wkv_naive(w, u, k, v, z, z.clone(), z.clone())
    assert torch.allclose(y, torch.full_like(y, v0), rtol=1e-12)
    ew = torch.exp(w)
    bb_closed = math.exp(k0) * ew * (1 - ew ** T) / (1 - ew)
    assert torch.allclose(bb, bb_closed, rtol=1e-11)
    assert torch.allclose(aa, v0 * bb_closed, rtol=1e-11)


def test_wkv_split_invariance():
    w, u, k, v, aa, bb, pp = _wkv_inputs(50, 16, seed=2)
    y, a, b, _ = O.wkv_naive(w, u, k, v, aa, bb, pp)
    y1, a1, b1, p1 = O.wkv_naive(w, u, k[:17], v[:17], aa, bb, pp)
    y2, a2, b2, _ = O.wkv_naive(w, u, k[17:], v[17:], a1, b1, p1)
    assert torch.allclose(torch.cat([y1, y2]), y, rtol=1e-12)
    assert torch.allclose(a2, a, rtol=1e-12) and torch.allclose(b2, b, rtol=1e-12)


def test_wkv_first_step_from_empty_state_is_v():
    w, u, k, v, aa, bb, pp = _wkv_inputs(1, 8, seed=3)
    y, *_ = O.wkv_naive(w, u, k, v, aa, bb, pp)
    assert torch.allclose(y[0], v[0], rtol=1e-14)


# ---------------------------------------------------------------- model
@pytest.fixture(scope="module")
def tiny():
    sd = synth.make_state_dict(layers=3, C=64, V=512, seed=5, ln="random")
    return sd, O.OracleModel(sd)


def test_model_shapes_and_empty_state(tiny):
    sd, m = tiny
    assert m.layers == 3 and m.dims == 64
    assert m.emptyState.shape == (3, 5, 64) and m.emptyState.dtype == torch.float64
    assert (m.emptyState[:, :4] == 0).all() and (m.emptyState[:, 4] == -1e30).all()
    logits, st = m.forward([3, 4, 5], m.emptyState.clone())
    assert logits.shape == (512,) and logits.dtype == torch.float64


def test_model_chunk_invariance(tiny):
    """T tokens at once == T single-token calls (pins token shift, state rows, WKV carry)."""
    sd, m = tiny
    toks = synth.random_tokens(9, V=512, seed=1).tolist()
    la, sa = m.forward(toks, m.emptyState.clone())
    sb = m.emptyState.clone()
    for t in toks:
        lb, sb = m.forward([t], sb)
    assert torch.allclose(la, lb, rtol=0, atol=2e-5)
    assert torch.allclose(sa, sb, rtol=1e-5, atol=1e-6)
    lc, sc = m.forward(toks[:4], m.emptyState.clone())
    lc, sc = m.forward(toks[4:], sc)
    assert torch.allclose(la, lc, rtol=0, atol=2e-5)


def test_model_state_rows_are_last_layernorm_outputs(tiny):
    sd, m = tiny
    toks = [7, 8]
    st = m.emptyState.clone()
    x = O.layernorm(m.emb[torch.tensor(toks)].double(), *m.ln_in)
    xy = O.layernorm(x, *m.blocks[0]["ln1"])
    _, st = m.forward(toks, st)
    assert torch.allclose(st[0, 0], xy[-1], rtol=1e-12)
    assert (st[:, 4] == -1e30).all()        # naive WKV never touches pp


def test_model_matches_unquantised_float64_network(tiny):
    """The quantised oracle tracks an independent plain-float64 RWKV-4 written
    with nn.functional ops and the direct-sum WKV (no shared code)."""
    sd, m = tiny
    toks = synth.random_tokens(6, V=512, seed=2)
    d = {k: v.double() for k, v in sd.items()}
    F = torch.nn.functional
    x = F.layer_norm(d["emb.weight"][toks], (64,), d["blocks.0.ln0.weight"], d["blocks.0.ln0.bias"])
    for i in range(3):
        p = f"blocks.{i}."
        xx = F.layer_norm(x, (64,), d[p + "ln1.weight"], d[p + "ln1.bias"])
        sx = torch.cat([torch.zeros(1, 64, dtype=torch.float64), xx[:-1]])
        mk, mv, mr = (d[p + f"att.time_mix_{c}"].reshape(-1) for c in "kvr")
        k = torch.lerp(sx, xx, mk) @ d[p + "att.key.weight"].t()
        v = torch.lerp(sx, xx, mv) @ d[p + "att.value.weight"].t()
        r = torch.sigmoid(torch.lerp(sx, xx, mr) @ d[p + "att.receptance.weight"].t())
        wkv = O.wkv_direct_sum(-torch.exp(d[p + "att.time_decay"]), d[p + "att.time_first"], k, v)
        x = x + (r * wkv) @ d[p + "att.output.weight"].t()
        xx = F.layer_norm(x, (64,), d[p + "ln2.weight"], d[p + "ln2.bias"])
        sx = torch.cat([torch.zeros(1, 64, dtype=torch.float64), xx[:-1]])
        fk, fr = (d[p + f"ffn.time_mix_{c}"].reshape(-1) for c in "kr")
        kk = torch.relu(torch.lerp(sx, xx, fk) @ d[p + "ffn.key.weight"].t()) ** 2
        x = x + torch.sigmoid(torch.lerp(sx, xx, fr) @ d[p + "ffn.receptance.weight"].t()) * (
            kk @ d[p + "ffn.value.weight"].t())
    x = F.layer_norm(x, (64,), d["ln_out.weight"], d["ln_out.bias"])
    want = x[-1] @ d["head.weight"].t()
    got, _ = m.forward(toks, m.emptyState.clone())
    # 8-bit weights: agreement to quantisation noise, far below the logit scale (~0.16)
    assert (got - want).abs().max() < 0.02
    assert torch.corrcoef(torch.stack([got, want]))[0, 1] > 0.995


# ------------------------------------------------ composition: exact, on the dequantised weights
MATRIX_KEYS = ("att.key", "att.value", "att.receptance", "att.output", "ffn.key", "ffn.receptance", "ffn.value")


def _dequantised_checkpoint(sd):
    """The checkpoint whose matrices are what the quantised layout represents: W'[out,in] = (code * range + offset)^T
    in float64 (quantiser pinned above).  Everything else is taken over in float64."""
    d = {k: v.double() for k, v in sd.items()}
    for key in [k for k in sd if k.endswith(".weight") and (k == "head.weight" or any(m in k for m in MATRIX_KEYS))]:
        c, r, o = O.quantize_matrix(sd[key].float())
        d[key] = (c.double() * r.double()[:, None] + o[:, None]).t().contiguous()
    return d


def _independent_network(d, toks, layers, C):
    """Textbook RWKV-4 (BlinkDL's formulation: lerp token shift, sigmoid receptance, relu^2 channel mix, WKV as a
    direct O(T^2) sum over the history) in float64 with nn.functional ops on the weights ``d``; shares no code with
    the oracle's block/model composition.  Returns logits of the last token and the state the reference keeps:
    per layer (last ln1 output, last ln2 output, aa, bb) with aa, bb the e^w-premultiplied history sums."""
    F = torch.nn.functional
    T = len(toks)
    x = F.layer_norm(d["emb.weight"][toks], (C,), d["blocks.0.ln0.weight"], d["blocks.0.ln0.bias"])
    rows = []
    for i in range(layers):
        p = f"blocks.{i}."
        xx = F.layer_norm(x, (C,), d[p + "ln1.weight"], d[p + "ln1.bias"])
        sx = torch.cat([torch.zeros(1, C, dtype=torch.float64), xx[:-1]])
        mk, mv, mr = (d[p + f"att.time_mix_{c}"].reshape(-1) for c in "kvr")
        k = torch.lerp(sx, xx, mk) @ d[p + "att.key.weight"].t()
        v = torch.lerp(sx, xx, mv) @ d[p + "att.value.weight"].t()
        r = torch.sigmoid(torch.lerp(sx, xx, mr) @ d[p + "att.receptance.weight"].t())
        w = -torch.exp(d[p + "att.time_decay"])
        wkv = O.wkv_direct_sum(w, d[p + "att.time_first"], k, v)
        age = torch.arange(T, 0, -1, dtype=torch.float64)[:, None]          # token i has been decayed T - i times
        e = torch.exp(age * w[None, :] + k)
        aa, bb = (e * v).sum(0), e.sum(0)
        x = x + (r * wkv) @ d[p + "att.output.weight"].t()
        x2 = F.layer_norm(x, (C,), d[p + "ln2.weight"], d[p + "ln2.bias"])
        sx2 = torch.cat([torch.zeros(1, C, dtype=torch.float64), x2[:-1]])
        fk, fr = (d[p + f"ffn.time_mix_{c}"].reshape(-1) for c in "kr")
        kk = torch.relu(torch.lerp(sx2, x2, fk) @ d[p + "ffn.key.weight"].t()) ** 2
        x = x + torch.sigmoid(torch.lerp(sx2, x2, fr) @ d[p + "ffn.receptance.weight"].t()) * (
            kk @ d[p + "ffn.value.weight"].t())
        rows.append((xx[-1], x2[-1], aa, bb))
    x = F.layer_norm(x, (C,), d["ln_out.weight"], d["ln_out.bias"])
    return x[-1] @ d["head.weight"].t(), rows


def _composition_error(m, d, toks, split):
    """Largest deviation (logits absolute, state relative to the row's scale) of the oracle ``m``, fed ``toks`` in
    two calls split at ``split`` so that every state row is carried across a call, from the independent network."""
    want, rows = _independent_network(d, toks, m.layers, m.dims)
    st = m.emptyState.clone()
    _, st = m.forward(toks[:split].tolist(), st)
    got, st = m.forward(toks[split:].tolist(), st)
    err = float((got - want).abs().max())
    for i, (x1, x2, aa, bb) in enumerate(rows):
        for row, ref in ((0, x1), (1, x2), (2, aa), (3, bb)):
            err = max(err, float(((st[i, row] - ref).abs() / (ref.abs().max() + 1e-300)).max()))
    return err


class _RowsSwapped(O.OracleModel):
    """The oracle with the att-shift and ffn-shift state rows exchanged (a wrong state row map)."""

    def block_forward(self, blk, x, state):
        perm = torch.tensor([1, 0, 2, 3, 4])
        s = state[perm].clone()
        out = super().block_forward(blk, x, s)
        state.copy_(s[perm])
        return out


def _mutants():
    def kv_mix(m):
        for b in m.blocks:
            b["attmix"] = b["attmix"][[1, 0, 2]]

    def ffn_mix(m):
        for b in m.blocks:
            b["ffnmix"] = b["ffnmix"][[1, 0]]

    def no_bonus(m):
        for b in m.blocks:
            b["time_first"] = torch.zeros_like(b["time_first"])

    def mix_reversed(m):
        for b in m.blocks:
            b["attmix"] = 1 - b["attmix"]
            b["ffnmix"] = 1 - b["ffnmix"]

    def decay_sign(m):
        for b in m.blocks:
            b["time_decay"] = b["time_decay"] * 0.5

    def kr_matrices(m):
        for b in m.blocks:
            b["att_k"], b["att_r"] = b["att_r"], b["att_k"]

    def ln_swapped(m):
        for b in m.blocks:
            b["ln1"], b["ln2"] = b["ln2"], b["ln1"]

    return dict(kv_mix_rows_swapped=kv_mix, ffn_mix_rows_swapped=ffn_mix, time_first_zero=no_bonus,
                mix_direction_reversed=mix_reversed, decay_halved=decay_sign, key_receptance_swapped=kr_matrices,
                ln1_ln2_swapped=ln_swapped)


COMPOSITION_TOL = 1e-12


def test_model_composition_is_exact_on_dequantised_weights(tiny):
    """With float64 products the oracle is the textbook network on the dequantised matrices, to rounding: logits and
    every carried state row (shift rows, aa, bb) agree to 1e-12 with a network that shares no composition code.
    Pins block_forward / forward: mix row order and direction, bonus, decay, which matrix gets which mix, the
    state row map, the head on the last token (agnostic/backends/modules/block.py:56-102, opt.py:61-76)."""
    sd, _ = tiny
    m = O.OracleModel(sd, matmul_dtype=torch.float64)
    toks = synth.random_tokens(7, V=512, seed=2)
    err = _composition_error(m, _dequantised_checkpoint(sd), toks, split=3)
    assert err < COMPOSITION_TOL, err


@pytest.mark.parametrize("name", sorted(_mutants()) + ["state_rows_0_1_swapped"])
def test_model_composition_pin_rejects_plausible_mistakes(tiny, name):
    """Each one-line mistake in the composition moves the result by nine orders of magnitude more than the pin
    allows, so the pin above cannot pass on a wrong oracle."""
    sd, _ = tiny
    if name == "state_rows_0_1_swapped":
        m = _RowsSwapped(sd, matmul_dtype=torch.float64)
    else:
        m = O.OracleModel(sd, matmul_dtype=torch.float64)
        _mutants()[name](m)
    toks = synth.random_tokens(7, V=512, seed=2)
    err = _composition_error(m, _dequantised_checkpoint(sd), toks, split=3)
    assert err > 1e-4, (name, err)


def test_float32_oracle_is_the_float64_oracle_up_to_accumulation_noise(tiny):
    """matmul_dtype only changes the accumulation type of the products (matmul.py:124-142 naivedtype): the default
    float32 oracle stays within float32 summation noise of the pinned float64 one."""
    sd, m32 = tiny
    m64 = O.OracleModel(sd, matmul_dtype=torch.float64)
    toks = synth.random_tokens(7, V=512, seed=2).tolist()
    l32, s32 = m32.forward(toks, m32.emptyState.clone())
    l64, s64 = m64.forward(toks, m64.emptyState.clone())
    assert (l32 - l64).abs().max() < 2e-5
    assert torch.allclose(s32, s64, rtol=1e-4, atol=1e-5)


# ---------------------------------------------------------------- sampler
def test_typical_distribution_hand_worked_cases():
    """Probabilities (1/2, 1/4, 1/8, 1/8): surprises (1, 2, 3, 3) ln 2, entropy 1.75 ln 2, distances to the entropy
    (0.75, 0.25, 1.25, 1.25) ln 2.  In order of distance the tokens are 1, 0, then 2 and 3 tied, with cumulative mass
    0.25, 0.75, 0.875, 1.  The kept set is everything not farther than the token at position #(cumulative < tau):
    worked by hand for four values of tau, and with a temperature (kept probabilities to the power 1 / temp)."""
    logits = torch.log(torch.tensor([0.5, 0.25, 0.125, 0.125])) + 3.0       # softmax is shift invariant
    cases = {
        0.2: [0.0, 1.0, 0.0, 0.0],                 # only the token closest to the entropy - not the most probable one
        0.5: [2 / 3, 1 / 3, 0.0, 0.0],
        0.8: [0.5, 0.25, 0.125, 0.125],            # position 2 is one of the tied pair: both stay
        0.99: [0.5, 0.25, 0.125, 0.125],
    }
    for tau, want in cases.items():
        got = O.typical_distribution(logits, temp=1.0, tau=tau)
        assert torch.allclose(got, torch.tensor(want, dtype=torch.float64), atol=1e-6), (tau, got)
    got = O.typical_distribution(logits, temp=2.0, tau=0.5)
    a, b = math.sqrt(0.5), math.sqrt(0.25)
    assert torch.allclose(got, torch.tensor([a / (a + b), b / (a + b), 0.0, 0.0], dtype=torch.float64), atol=1e-6)


def test_typical_distribution_uniform_logits_keep_everything():
    """All surprises equal the entropy: every distance is zero, nothing can be cut, whatever tau."""
    for tau in (0.01, 0.5, 0.95):
        got = O.typical_distribution(torch.full((37,), -1.25), temp=0.7, tau=tau)
        assert torch.allclose(got, torch.full((37,), 1 / 37, dtype=torch.float64), atol=1e-7)
