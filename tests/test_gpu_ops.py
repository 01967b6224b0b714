"""GPU parity of the stand-alone operators against the CPU oracle.
Every case goes through the C ABI (rwkvstic_amd.ops -> ctypes -> librwkv_hip.so)."""
import pytest
import torch

from oracle import rwkv_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from rwkvstic_amd import ops as _ops
    return _ops


def _say(msg):
    print(msg, flush=True)


# ------------------------------------------------------------------ quantiser + layouts
@pytest.mark.parametrize("shape", [(8, 8), (5, 3), (300, 130), (3072, 768), (2560, 2560), (1000, 257)])
def test_quantiser_bit_exact_codes_and_1ulp_dequant(ops, shape):
    _say(f"quantise {shape}")
    g = torch.Generator().manual_seed(shape[0] * 7 + shape[1])
    W = torch.randn(*shape, generator=g) * 0.02
    c_ref, r_ref, o_ref = O.quantize_matrix(W)
    codes, rng, off = ops.quantize(W.cuda())
    torch.cuda.synchronize()
    assert torch.equal(codes.cpu(), c_ref), "codes differ"
    assert torch.equal(rng.cpu(), r_ref), "range differs"
    # offset differs only by the summation order of the mean fraction
    assert torch.allclose(off.cpu(), o_ref, rtol=1e-13, atol=1e-300)
    packed = ops.pack(codes)
    assert torch.equal(ops.unpack(packed, *codes.shape).cpu(), c_ref), "pack/unpack round trip"
    dq = ops.dequant_packed(packed, rng, off, *codes.shape).cpu()
    want = O.dequant_canonical(c_ref, r_ref, o_ref)
    ulp = torch.abs(torch.nextafter(want, torch.full_like(want, float("inf"))) - want)
    assert ((dq - want).abs() <= ulp).all(), "dequantised weights differ by more than 1 ulp"


def test_quantiser_constant_channel(ops):
    W = torch.randn(40, 16) * 0.02
    W[:, 3] = 0.125
    codes, rng, off = ops.quantize(W.cuda())
    assert int(codes[3].max()) == 0 and float(rng[3]) == 0.0 and float(off[3]) == 0.125


def test_pack_strided_and_ragged(ops):
    big = torch.randint(0, 256, (200, 400), dtype=torch.uint8, device="cuda")
    view = big[:130, :77]                      # stride 400, ragged in both dims
    packed = ops.pack(view)
    assert torch.equal(ops.unpack(packed, 130, 77), view)


# ------------------------------------------------------------------ packed matvec (isolated workload)
SHAPES = [(2560, 2560), (2560, 10240), (10240, 2560)]


PACKED_CASES = [(n_in, n_out, B) for (n_in, n_out) in SHAPES + [(96, 40), (130, 77), (768, 50277)] for B in (1, 8)]
PACKED_CASES += [(256, 8200, 4), (256, 8200, 2)]     # 1025 column tiles: four per workgroup at B = 4 (ragged last group), one at B = 2


@pytest.mark.parametrize("n_in,n_out,B", PACKED_CASES)
def test_mm8_packed_general_form(ops, n_in, n_out, B):
    _say(f"mm8_packed in={n_in} out={n_out} B={B}")
    g = torch.Generator().manual_seed(n_in + 3 * n_out + B)
    codes = torch.randint(0, 256, (n_in, n_out), generator=g, dtype=torch.uint8)
    m_row = torch.randn(n_in, generator=g) * 0.01
    m_col = torch.randn(n_out, generator=g) * 0.01
    r_row = torch.rand(n_in, generator=g) * 9e-4 + 1e-4
    r_col = torch.rand(n_out, generator=g) * 9e-4 + 1e-4
    x = torch.randn(B, n_in, generator=g)
    want = O.mm8_general_f64(x, codes, r_row, m_row, r_col, m_col)
    packed = ops.pack(codes.cuda())
    got = ops.mm8_packed(x.cuda(), packed, n_in, n_out, r_row.cuda(), m_row.double().cuda(),
                         r_col.cuda(), m_col.cuda()).cpu()
    # float32 accumulation of n_in terms: bound n * 2^-23 * max |partial sum scale|
    scale = (x.abs().double() * r_row.double()) @ codes.double() * r_col.double()
    tol = 2.0 ** -23 * 8 * scale.max()
    err = (got - want).abs().max()
    _say(f"  max err {err:.3e} tol {tol:.3e} |y| {want.abs().max():.3e}")
    assert err <= tol


M16_CASES = [(n_in, n_out, B) for (n_in, n_out) in SHAPES for B in (1, 8)]
M16_CASES += [(96, 40, 3), (130, 77, 5), (768, 50277, 2), (4160, 48, 7), (20480, 32, 8), (64, 16, 1)]


@pytest.mark.parametrize("n_in,n_out,B", M16_CASES)
def test_mm8_m16_general_form(ops, n_in, n_out, B):
    """The matrix-core route of the same product (any B in 1..8, M16 layout): exact integer sums over fp32(x * r_row),
    so it is held to a bound 64 times tighter than the float32-accumulating kernel - what is left is the float32
    rounding of x * r_row itself."""
    _say(f"mm8_m16 in={n_in} out={n_out} B={B}")
    g = torch.Generator().manual_seed(n_in + 3 * n_out + B)
    codes = torch.randint(0, 256, (n_in, n_out), generator=g, dtype=torch.uint8)
    m_row = torch.randn(n_in, generator=g) * 0.01
    m_col = torch.randn(n_out, generator=g) * 0.01
    r_row = torch.rand(n_in, generator=g) * 9e-4 + 1e-4
    r_col = torch.rand(n_out, generator=g) * 9e-4 + 1e-4
    x = torch.randn(B, n_in, generator=g)
    x[0, : n_in // 3] *= 300.0                      # chunks of very different magnitude inside one vector
    want = O.mm8_general_f64(x, codes, r_row, m_row, r_col, m_col)
    p16 = ops.pack_m16(codes.cuda())
    got = ops.mm8_m16(x.cuda(), p16, n_in, n_out, r_row.cuda(), m_row.double().cuda(), r_col.cuda(), m_col.cuda()).cpu()
    scale = (x.abs().double() * r_row.double()) @ codes.double() * r_col.double()
    tol = 2.0 ** -23 * scale.max(dim=1, keepdim=True).values / 8
    err = ((got - want).abs() / tol).max()
    _say(f"  max err / tol {err:.3e}")
    assert err <= 1.0
    # the reference layout (no per-column vectors) against the oracle's mm8_naive with exact accumulation
    got = ops.mm8_m16(x.cuda(), p16, n_in, n_out, r_row.cuda(), m_row.double().cuda()).cpu()
    want = O.mm8_naive(x.double(), codes, r_row, m_row.double(), dtype=torch.float64)
    scale = (x.abs().double() * r_row.double()) @ codes.double()
    assert ((got - want).abs() <= 2.0 ** -23 * scale.max(dim=1, keepdim=True).values / 8).all()


def test_mm8_m16_agrees_with_mm8_packed_and_rejects_bad_arguments(ops):
    from rwkvstic_amd._native import RwkvHipError
    g = torch.Generator().manual_seed(77)
    n_in, n_out = 2560, 2560
    codes = torch.randint(0, 256, (n_in, n_out), generator=g, dtype=torch.uint8).cuda()
    r = (torch.rand(n_in, generator=g) * 9e-4 + 1e-4).cuda()
    m = (torch.randn(n_in, generator=g) * 0.01).double().cuda()
    x = torch.randn(8, n_in, generator=g).cuda()
    a = ops.mm8_packed(x, ops.pack(codes), n_in, n_out, r, m)
    b = ops.mm8_m16(x, ops.pack_m16(codes), n_in, n_out, r, m)
    assert (a - b).abs().max() < 2e-4 * float(b.abs().max())
    # one vector of the eight on its own: the same bits (a vector's digits do not depend on its neighbours)
    b3 = ops.mm8_m16(x[3:4].contiguous(), ops.pack_m16(codes), n_in, n_out, r, m)
    assert torch.equal(b3[0], b[3])
    with pytest.raises(RwkvHipError):
        ops.mm8_m16(torch.zeros(9, n_in, device="cuda"), ops.pack_m16(codes), n_in, n_out, r, m)      # B > 8
    with pytest.raises(RwkvHipError):
        ops.mm8_m16(x, ops.pack_m16(codes), n_in, n_out, r, m, workspace=torch.empty(1024, dtype=torch.uint8, device="cuda"))
    with pytest.raises(ValueError):
        ops.mm8_m16(x, ops.pack_m16(codes)[:1000], n_in, n_out, r, m)


@pytest.mark.parametrize("B", [1, 2, 4])
def test_mm8_packed_reference_form_matches_cpu_path(ops, B):
    """r_col = m_col = None is MM8.forward; compare with the oracle's mm8_naive."""
    W = torch.randn(1000, 384) * 0.02
    c, r, o = O.quantize_matrix(W)
    x = torch.randn(B, 384)
    want = O.mm8_naive(x.double(), c, r, o)
    got = ops.mm8_packed(x.cuda(), ops.pack(c.cuda()), 384, 1000, r.cuda(), o.cuda()).cpu()
    assert (got - want).abs().max() < 2e-5


def test_mm8_packed_rejects_bad_arguments(ops):
    from rwkvstic_amd._native import RwkvHipError
    c = torch.zeros((128, 8), dtype=torch.uint8, device="cuda")
    p = ops.pack(c)
    x = torch.zeros((3, 128), device="cuda")
    r = torch.ones(128, device="cuda"); m = torch.zeros(128, dtype=torch.float64, device="cuda")
    with pytest.raises(RwkvHipError):
        ops.mm8_packed(x, p, 128, 8, r, m)          # B = 3 unsupported
    with pytest.raises(ValueError):
        ops.mm8_packed(x[:1], p[:512], 128, 8, r, m)  # packed too small
    with pytest.raises(TypeError):
        ops.mm8_packed(x[:1].double(), p, 128, 8, r, m)


# ------------------------------------------------------------------ reference-layout operators
@pytest.mark.parametrize("n_in,n_out", [(768, 768), (2560, 2560), (96, 50277), (130, 77)])
def test_mm8_one_reference_semantics(ops, n_in, n_out):
    _say(f"mm8_one in={n_in} out={n_out}")
    g = torch.Generator().manual_seed(n_in * 5 + n_out)
    w = torch.randint(0, 256, (n_in, n_out), generator=g, dtype=torch.uint8)
    r = torch.rand(n_in, generator=g) * 1e-3
    x = torch.randn(n_in, generator=g)
    y0 = torch.randn(n_out, generator=g)
    want = y0.double() + (x.double() * r.double()) @ w.double()
    y = y0.clone().cuda()
    ops.mm8_one(n_in, n_out, x.cuda(), w.cuda(), y, r.cuda())      # accumulates into y
    scale = ((x.abs().double() * r.double()) @ w.double()).max()
    assert (y.cpu().double() - want).abs().max() <= 2.0 ** -23 * 8 * scale + 1e-6 * y0.abs().max()


def test_mm8_three_matches_three_mm8_one(ops):
    n_in, n_out = 512, 520
    g = torch.Generator().manual_seed(11)
    ws = [torch.randint(0, 256, (n_in, n_out), generator=g, dtype=torch.uint8).cuda() for _ in range(3)]
    rs = [(torch.rand(n_in, generator=g) * 1e-3).cuda() for _ in range(3)]
    xs = [torch.randn(n_in, generator=g).cuda() for _ in range(3)]
    y3 = [torch.zeros(n_out, device="cuda") for _ in range(3)]
    y1 = [torch.zeros(n_out, device="cuda") for _ in range(3)]
    ops.mm8_three(n_in, n_out, *xs, *ws, *y3, *rs)
    for i in range(3):
        ops.mm8_one(n_in, n_out, xs[i], ws[i], y1[i], rs[i])
        assert torch.equal(y3[i], y1[i])       # same kernel arithmetic, deterministic


@pytest.mark.parametrize("n_in,n_out", [(768, 768), (130, 77), (2560, 2560), (1000, 50277)])
def test_mm8_one_and_three_float64_instances(ops, n_in, n_out):
    """The `double` branch of the reference's operators (wrapper.cpp:60-77, operators.cu:58-118): x, r, y and the sums
    float64.  Against the float64 dense product at float64 rounding, accumulating into y; three problems in one call
    equal three single calls bit for bit; the float32 instance is left as it was (dtype picks the instance)."""
    _say(f"mm8_one/three f64 in={n_in} out={n_out}")
    g = torch.Generator().manual_seed(n_in * 7 + n_out)
    ws = [torch.randint(0, 256, (n_in, n_out), generator=g, dtype=torch.uint8) for _ in range(3)]
    rs = [torch.rand(n_in, generator=g, dtype=torch.float64) * 1e-3 for _ in range(3)]
    xs = [torch.randn(n_in, generator=g, dtype=torch.float64) for _ in range(3)]
    y0 = [torch.randn(n_out, generator=g, dtype=torch.float64) for _ in range(3)]
    y1 = [t.clone().cuda() for t in y0]
    y3 = [t.clone().cuda() for t in y0]
    dws = [w.cuda() for w in ws]
    for i in range(3):
        ops.mm8_one(n_in, n_out, xs[i].cuda(), dws[i], y1[i], rs[i].cuda())
        want = y0[i] + (xs[i] * rs[i]) @ ws[i].double()
        scale = ((xs[i].abs() * rs[i]) @ ws[i].double()).max()
        assert (y1[i].cpu() - want).abs().max() <= 2.0 ** -52 * 64 * scale + 1e-15 * y0[i].abs().max()
    ops.mm8_three(n_in, n_out, *[x.cuda() for x in xs], *dws, *y3, *[r.cuda() for r in rs])
    for i in range(3):
        assert torch.equal(y3[i], y1[i])
    with pytest.raises(TypeError):
        ops.mm8_one(n_in, n_out, xs[0].cuda(), dws[0], y1[0].float(), rs[0].cuda())      # mixed types, as wrapper.cpp:58 asserts
    # through the registered operator, as scripted reference code reaches it
    ops.register_torch_ops()
    y = torch.zeros(n_out, dtype=torch.float64, device="cuda")
    torch.ops.rwkv.mm8_one(n_in, n_out, xs[0].cuda(), dws[0], y, rs[0].cuda())
    want = (xs[0] * rs[0]) @ ws[0].double()
    assert (y.cpu() - want).abs().max() <= 2.0 ** -52 * 64 * ((xs[0].abs() * rs[0]) @ ws[0].double()).max()


def test_mm8_one_strided_rows(ops):
    big = torch.randint(0, 256, (64, 1003), dtype=torch.uint8, device="cuda")   # odd stride: byte path
    w = big[:, :1000]
    x = torch.randn(64, device="cuda"); r = torch.rand(64, device="cuda")
    y = torch.zeros(1000, device="cuda")
    ops.mm8_one(64, 1000, x, w, y, r)
    want = (x.double() * r.double()) @ w.double()
    assert (y.double() - want).abs().max() < 1e-2 * 1e-3 * want.abs().max() + 1e-3


def test_torch_ops_registered_with_reference_schema(ops):
    ops.register_torch_ops()
    n_in, n_out = 128, 64
    w = torch.randint(0, 256, (n_in, n_out), dtype=torch.uint8, device="cuda")
    x = torch.randn(n_in, device="cuda"); r = torch.rand(n_in, device="cuda")
    y = torch.zeros(n_out, device="cuda")
    torch.ops.rwkv.mm8_one(n_in, n_out, x, w, y, r)
    assert (y.double() - (x.double() * r.double()) @ w.double()).abs().max() < 1e-2


# ------------------------------------------------------------------ WKV
def _wkv_case(B, T, C, seed, lo=-8.0):
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(B, T, C, generator=g)
    v = torch.randn(B, T, C, generator=g)
    w = -torch.exp(torch.rand(C, generator=g) * (1.0 - lo) + lo)
    u = torch.rand(C, generator=g) * 2 - 1
    return w, u, k, v


def _check_wkv_f32(ops, B, T, C, seed):
    w, u, k, v = _wkv_case(B, T, C, seed)
    aa = torch.zeros(B, C); bb = torch.zeros(B, C); pp = torch.full((B, C), -1e38)
    d = lambda t: t.cuda()
    aa_d, bb_d, pp_d = d(aa), d(bb), d(pp)
    y = ops.wkv_f32(d(w), d(u), d(k), d(v), aa_d, bb_d, pp_d).cpu()
    for b in range(B):
        yr, ar, br, _ = O.wkv_naive(w.double(), u.double(), k[b].double(), v[b].double(),
                                    aa[b].double(), bb[b].double(), pp[b].double())
        assert (y[b].double() - yr).abs().max() < 1e-4 * max(1.0, float(yr.abs().max()))
        an, bn = O.state_naive_from_stable(aa_d[b].cpu(), bb_d[b].cpu(), pp_d[b].cpu())
        # bb is a positive sum; aa is a signed sum of the same weights times v ~ N(0,1)
        assert ((bn - br).abs() <= 1e-4 * br).all()
        assert ((an - ar).abs() <= 1e-4 * torch.maximum(ar.abs(), br)).all()


def test_wkv_f32_small(ops):
    _say("wkv_f32 B=2 T=37 C=130")
    _check_wkv_f32(ops, 2, 37, 130, seed=3)


def test_wkv_f32_isolated_workload(ops):
    _say("wkv_f32 B=8 T=1024 C=2560")
    _check_wkv_f32(ops, 8, 1024, 2560, seed=2)


def test_wkv_f32_split_invariance_and_large_k(ops):
    """Carrying the state across two calls equals one call; k up to +-60 must not overflow float32."""
    w, u, k, v = _wkv_case(1, 64, 64, seed=9)
    k = k * 20
    d = lambda t: t.cuda()
    s1 = [torch.zeros(1, 64).cuda(), torch.zeros(1, 64).cuda(), torch.full((1, 64), -1e38).cuda()]
    y_all = ops.wkv_f32(d(w), d(u), d(k), d(v), *s1)
    s2 = [torch.zeros(1, 64).cuda(), torch.zeros(1, 64).cuda(), torch.full((1, 64), -1e38).cuda()]
    ya = ops.wkv_f32(d(w), d(u), d(k[:, :20].contiguous()), d(v[:, :20].contiguous()), *s2)
    yb = ops.wkv_f32(d(w), d(u), d(k[:, 20:].contiguous()), d(v[:, 20:].contiguous()), *s2)
    # the exponent is float64 inside a call and rounded to float32 at the call boundary
    assert torch.allclose(torch.cat([ya, yb], 1), y_all, rtol=2e-5, atol=2e-5)
    assert torch.isfinite(y_all).all()
    yr = O.wkv_stable(w.double(), u.double(), k[0].double(), v[0].double(),
                      torch.zeros(64).double(), torch.zeros(64).double(), torch.full((64,), -1e38).double())[0]
    assert (y_all[0].cpu().double() - yr).abs().max() < 1e-4 * max(1.0, float(yr.abs().max()))


@pytest.mark.parametrize("T", [256, 333, 1000])
def test_wkv_f32_long_sequences_carry_a_state_in_and_out(ops, T):
    """Sequences of 256 steps and more run as a two-pass scan inside a workgroup (ragged last chunks at 333 and
    1000): a state carried in from a first call, the outputs and the state carried out against the float64
    recurrence over both calls; large |k| must not overflow."""
    _say(f"wkv_f32 scan T={T}")
    B, C, T0 = 3, 96, 40
    w, u, k, v = _wkv_case(B, T0 + T, C, seed=11)
    k = k * 8
    d = lambda t: t.cuda()
    st = [torch.zeros(B, C).cuda(), torch.zeros(B, C).cuda(), torch.full((B, C), -1e38).cuda()]
    ya = ops.wkv_f32(d(w), d(u), d(k[:, :T0].contiguous()), d(v[:, :T0].contiguous()), *st)
    yb = ops.wkv_f32(d(w), d(u), d(k[:, T0:].contiguous()), d(v[:, T0:].contiguous()), *st)
    y = torch.cat([ya, yb], 1).cpu().double()
    assert torch.isfinite(y).all()
    for b in range(B):
        z = torch.zeros(C).double()
        yr, ar, br, _ = O.wkv_naive(w.double(), u.double(), k[b].double(), v[b].double(), z, z.clone(), torch.full((C,), -1e38).double())
        assert (y[b] - yr).abs().max() < 1e-4 * max(1.0, float(yr.abs().max()))
        ys, a_s, b_s, p_s = O.wkv_stable(w.double(), u.double(), k[b].double(), v[b].double(), z, z.clone(), torch.full((C,), -1e38).double())
        # the state in its shifted form: aa e^pp and bb e^pp are what the next call continues from
        got_a, got_b, got_p = st[0][b].cpu().double(), st[1][b].cpu().double(), st[2][b].cpu().double()
        scale = torch.exp(got_p - p_s)
        assert ((got_b * scale - b_s).abs() <= 1e-4 * b_s.abs()).all()
        assert ((got_a * scale - a_s).abs() <= 1e-4 * torch.maximum(a_s.abs(), b_s.abs())).all()


@pytest.mark.parametrize("T", [300, 1000])
def test_wkv_f32_one_read_scan_with_ragged_blocks_and_a_carried_state(ops, T):
    """With 512 and more groups of 32 channels the scan keeps each chunk's k and v in registers between its two passes
    and reads them once (blocks of 128 steps; 300 and 1000 end inside a block and inside a chunk): outputs and the
    state carried out, after a state carried in from a first call, against the float64 recurrence; large |k|."""
    _say(f"wkv_f32 one-read scan T={T}")
    B, C, T0 = 8, 2048, 30
    w, u, k, v = _wkv_case(B, T0 + T, C, seed=21)
    k = k * 6
    d = lambda t: t.cuda()
    st = [torch.zeros(B, C).cuda(), torch.zeros(B, C).cuda(), torch.full((B, C), -1e38).cuda()]
    ya = ops.wkv_f32(d(w), d(u), d(k[:, :T0].contiguous()), d(v[:, :T0].contiguous()), *st)
    yb = ops.wkv_f32(d(w), d(u), d(k[:, T0:].contiguous()), d(v[:, T0:].contiguous()), *st)
    y = torch.cat([ya, yb], 1).cpu().double()
    assert torch.isfinite(y).all()
    for b in (0, 3, 7):
        z = torch.zeros(C).double()
        ys, a_s, b_s, p_s = O.wkv_stable(w.double(), u.double(), k[b].double(), v[b].double(), z, z.clone(), torch.full((C,), -1e38).double())
        assert (y[b] - ys).abs().max() < 1e-4 * max(1.0, float(ys.abs().max()))
        got_a, got_b, got_p = st[0][b].cpu().double(), st[1][b].cpu().double(), st[2][b].cpu().double()
        scale = torch.exp(got_p - p_s)
        assert ((got_b * scale - b_s).abs() <= 1e-4 * b_s.abs()).all()
        assert ((got_a * scale - a_s).abs() <= 1e-4 * torch.maximum(a_s.abs(), b_s.abs())).all()


def test_wkv_forward_f64_reference_convention(ops):
    """Drop-in for torch.ops.rwkv.wkv_forward: naive state in/out, pp untouched."""
    B, T, C = 1, 50, 96
    w, u, k, v = _wkv_case(B, T, C, seed=4)
    w, u, k, v = (t.double() for t in (w, u, k, v))
    aa = torch.rand(C).double(); bb = torch.rand(C).double() + 0.5; pp = torch.full((C,), -1e30).double()
    yr, ar, br, pr = O.wkv_naive(w, u, k[0], v[0], aa, bb, pp)
    d = lambda t: t.cuda()
    aa_d, bb_d, pp_d = d(aa.clone()), d(bb.clone()), d(pp.clone())
    y = torch.empty(T, C, dtype=torch.float64, device="cuda")
    ops.wkv_forward(1, T, C, d(w), d(u), d(k[0].contiguous()), d(v[0].contiguous()), y, aa_d, bb_d, pp_d)
    assert torch.allclose(y.cpu(), yr, rtol=1e-11, atol=1e-12)
    assert torch.allclose(aa_d.cpu(), ar, rtol=1e-10) and torch.allclose(bb_d.cpu(), br, rtol=1e-10)
    assert torch.equal(pp_d.cpu(), pp)
    # from the empty state too
    z = torch.zeros(C).double()
    yr, ar, br, _ = O.wkv_naive(w, u, k[0], v[0], z, z.clone(), pp)
    aa_d, bb_d = d(z.clone()), d(z.clone())
    ops.wkv_forward(1, T, C, d(w), d(u), d(k[0].contiguous()), d(v[0].contiguous()), y, aa_d, bb_d, pp_d)
    assert torch.allclose(y.cpu(), yr, rtol=1e-11, atol=1e-12)
    assert torch.allclose(bb_d.cpu(), br, rtol=1e-10)


def test_argmax_first_maximum(ops):
    x = torch.randn(50277, dtype=torch.float64)
    x[40000] = 9.0; x[123] = 9.0
    assert int(ops.argmax(x.cuda())) == 123


def test_pack_m16_round_trip(ops):
    for n_in, n_out in [(64, 16), (130, 77), (2560, 2560)]:
        c = torch.randint(0, 256, (n_in, n_out), dtype=torch.uint8, device="cuda")
        p = ops.pack_m16(c)
        assert torch.equal(ops.unpack_m16(p, n_in, n_out), c)
    # block 0, lane 16*g + n, byte i  <->  codes[16*g + i][n] - 128
    c = torch.arange(64 * 16, dtype=torch.int64).reshape(64, 16).remainder(256).to(torch.uint8).cuda()
    p = ops.pack_m16(c).cpu().reshape(64, 16)
    for lane in (0, 5, 17, 63):
        g, n = divmod(lane, 16)
        want = (c[16 * g:16 * g + 16, n].cpu().to(torch.int16) - 128).to(torch.int8)
        assert torch.equal(p[lane].view(torch.int8), want)


# the last two run the 160-column workgroup variant (320 general workgroups would make 1.25 per compute unit),
# with ragged rows, ragged columns and a contraction that ends inside a round of the pipeline
@pytest.mark.parametrize("T,K,N", [(1, 64, 16), (5, 256, 100), (64, 2560, 2560), (130, 2560, 10240),
                                   (33, 10240, 2560), (8, 2560, 50277), (1000, 192, 2560), (1024, 320, 2500),
                                   (3, 20544, 32),      # a few long rows: the two-launch quantiser
                                   (4, 8320, 48),       # the same with parts that have to be rounded up to whole groups of 16 values
                                   (9, 20544, 32),      # rows too long for the register-resident quantiser
                                   (20, 2560, 2560), (32, 640, 5000),    # 9..32 rows: the few-row variant with LDS staging
                                   # 769..960 rows on a long contraction: the 160-column workgroups (208 of them)
                                   (800, 2560, 2560), (900, 2560, 5120),
                                   # the 128-column workgroups with the contraction split (80 workgroups x 2,
                                   # 20 x 4: integer slices added by the tail kernel), ragged rows
                                   (250, 2560, 2560), (60, 10240, 2560)])
def test_gemm8_matches_fp64_dense(ops, T, K, N):
    """Prompt GEMM (matmul.py:56-57 without its bfloat16 rounding) against the float64 dense product."""
    g = torch.Generator().manual_seed(T * 7 + K + N)
    w = torch.randn(N, K, generator=g) * 0.02
    codes, rng, off = O.quantize_matrix(w)
    x = torch.randn(T, K, generator=g, dtype=torch.float64)
    x[0, : K // 2] *= 50.0                                    # rows with very different scales
    want = O.mm8_naive(x, codes, rng, off, dtype=torch.float64)
    dev = "cuda"
    p16 = ops.pack_m16(codes.to(dev))
    got = ops.gemm8(x.to(dev), p16, rng.to(dev), off.to(dev), K, N).cpu()
    bound = ((x.abs() * rng.double()) @ codes.double()).max(dim=1, keepdim=True).values
    err = ((got - want).abs() / bound).max().item()
    print(f"gemm8 T={T} K={K} N={N}: max err / sum|terms| = {err:.2e}", flush=True)
    assert err < 2e-7                                         # float32 rounding of x*range, nothing else


def test_gemm8_rows_do_not_depend_on_batching(ops):
    """Integer accumulation: a row's result is bit-identical whether the contraction is split (few rows)
    or not (many rows), and wherever the row sits in its tile."""
    g = torch.Generator().manual_seed(3)
    K, N = 2560, 2560
    w = torch.randn(N, K, generator=g) * 0.02
    codes, rng, off = O.quantize_matrix(w)
    x = torch.randn(1024, K, generator=g, dtype=torch.float64).cuda()
    p16 = ops.pack_m16(codes.cuda())
    wide = ops.gemm8(x, p16, rng.cuda(), off.cuda(), K, N)            # 160-column workgroups
    full = ops.gemm8(x[:300].contiguous(), p16, rng.cuda(), off.cuda(), K, N)    # 128-column workgroups
    few = ops.gemm8(x[37:40].contiguous(), p16, rng.cuda(), off.cuda(), K, N)    # few-row variant, split contraction
    assert torch.equal(full[37:40], few) and torch.equal(wide[:300], full)
