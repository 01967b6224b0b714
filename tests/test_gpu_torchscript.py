"""The boundary as the reference uses it: its modules are TorchScript-compiled and call the three native operators
as torch.ops.rwkv.* from inside scripted code (matmul.py:42-49 mm8_one, :70-80 mm8_three, wkv.py:8-19 wkv_forward),
and the quantised model travels as a torch.jit archive (opt.py:89-92,112-117).  Here small stand-in modules with the
reference's attribute names (weight / range / offset [, 1, 2]; matmul.py:12,67-68) make the same calls; they are
scripted, saved as a .rwkv archive, loaded back (a file this test wrote itself) and run on the GPU against the
CPU oracle.  A second archive carries a whole quantised model under the reference's attribute tree; its
state_dict() rebuilds the HIP model without a second quantisation."""
from typing import List

import pytest
import torch

from oracle import rwkv_oracle as O
from rwkvstic_amd import synth

pytestmark = pytest.mark.gpu


class MM8Like(torch.nn.Module):
    """One quantised matrix, single-row call (the T == 1 branch of MM8.forward)."""

    def __init__(self, codes, rng, off):
        super().__init__()
        self.weight = codes                    # uint8 [in, out]
        self.range = rng                       # float32 [in]
        self.offset = off                      # float64 [in]
        self.M = int(codes.shape[0])           # in
        self.N = int(codes.shape[1])           # out

    def forward(self, y):
        y32 = y.to(torch.float32)
        zp = y.mul(self.offset).sum()
        out = torch.zeros(self.N, device=y.device, dtype=torch.float32)
        torch.ops.rwkv.mm8_one(self.M, self.N, y32[0], self.weight, out, self.range)
        return out.unsqueeze(0) + zp


class MM8x3Like(torch.nn.Module):
    """Three matrices of one shape in one operator call (MM8_3)."""

    def __init__(self, q0, q1, q2):
        super().__init__()
        self.weight, self.range, self.offset = q0
        self.weight1, self.range1, self.offset1 = q1
        self.weight2, self.range2, self.offset2 = q2
        self.M = int(self.weight.shape[0])
        self.N = int(self.weight.shape[1])

    def forward(self, y: List[torch.Tensor]):
        x0 = y[0].squeeze().contiguous().to(torch.float32)
        x1 = y[1].squeeze().contiguous().to(torch.float32)
        x2 = y[2].squeeze().contiguous().to(torch.float32)
        o0 = torch.zeros(self.N, device=x0.device, dtype=torch.float32)
        o1 = torch.zeros(self.N, device=x0.device, dtype=torch.float32)
        o2 = torch.zeros(self.N, device=x0.device, dtype=torch.float32)
        torch.ops.rwkv.mm8_three(self.M, self.N, x0, x1, x2, self.weight, self.weight1, self.weight2, o0, o1, o2,
                                 self.range, self.range1, self.range2)
        zp0 = y[0].mul(self.offset).sum()
        zp1 = y[1].mul(self.offset1).sum()
        zp2 = y[2].mul(self.offset2).sum()
        return o0.unsqueeze(0) + zp0, o1.unsqueeze(0) + zp1, o2.unsqueeze(0) + zp2


class WKVLike(torch.nn.Module):
    def forward(self, T: int, C: int, w, u, k, v, aa, bb, pp):
        # the matrix modules hand over float32 rows (a float32 tensor plus a 0-dim float64 stays float32); the
        # operator is float64, so the caller converts, as wkv.py:9-13 does
        w = w.contiguous().to(torch.float64)
        u = u.contiguous().to(torch.float64)
        k = k.contiguous().to(torch.float64)
        v = v.contiguous().to(torch.float64)
        y = torch.empty((T, C), device=w.device, dtype=torch.float64)
        torch.ops.rwkv.wkv_forward(1, T, C, w, u, k, v, y, aa, bb, pp)
        return y, aa, bb, pp


class TimeMixLike(torch.nn.Module):
    """k, v, r -> WKV -> output matrix, the operator sequence of block.py:69-80 for one row."""

    def __init__(self, att, attout, w, u):
        super().__init__()
        self.att, self.attout, self.wkv = att, attout, WKVLike()
        self.time_decay, self.time_first = w, u

    def forward(self, x, aa, bb, pp):
        k, v, r = self.att([x, x, x])
        y, aa, bb, pp = self.wkv(1, int(x.shape[1]), self.time_decay, self.time_first, k, v, aa, bb, pp)
        return self.attout(y * torch.sigmoid(r)), aa, bb, pp


def _quantised(n_out, n_in, seed):
    g = torch.Generator().manual_seed(seed)
    return O.quantize_matrix(torch.randn(n_out, n_in, generator=g) * 0.02)


def test_scripted_modules_call_the_operators_and_survive_an_archive(tmp_path):
    from rwkvstic_amd import ops
    ops.register_torch_ops()
    C = 192
    qs = [_quantised(C, C, s) for s in range(4)]
    g = torch.Generator().manual_seed(9)
    w = -torch.exp(torch.rand(C, generator=g, dtype=torch.float64) * 6 - 5)
    u = torch.rand(C, generator=g, dtype=torch.float64) * 2 - 1
    dev = lambda q: tuple(t.cuda() for t in q)
    mod = TimeMixLike(MM8x3Like(dev(qs[0]), dev(qs[1]), dev(qs[2])), MM8Like(*dev(qs[3])), w.cuda(), u.cuda())
    scripted = torch.jit.script(mod)          # resolves torch.ops.rwkv.* against the registered schemas
    path = str(tmp_path / "timemix.rwkv")
    torch.jit.save(scripted, path)
    loaded = torch.jit.load(path, map_location="cuda")      # written two lines above by this test
    # the tensors are plain module attributes, as in the reference's modules (matmul.py:12,67-68)
    assert loaded.att.weight.dtype == torch.uint8 and loaded.att.range1.dtype == torch.float32
    assert loaded.att.offset2.dtype == torch.float64 and torch.equal(loaded.attout.weight.cpu(), qs[3][0])
    x = torch.randn(1, C, generator=g, dtype=torch.float64)
    aa = torch.zeros(C, dtype=torch.float64); bb = torch.zeros(C, dtype=torch.float64)
    pp = torch.full((C,), -1e30, dtype=torch.float64)
    # the oracle: mm8_naive (matmul.py:124-142) with exact accumulation, wkv_naive (wkv.py:23-39)
    ref_state = (aa.clone(), bb.clone(), pp.clone())
    got_state = (aa.cuda(), bb.cuda(), pp.cuda())
    for step in range(3):
        k, v, r = (O.mm8_naive(x, *q, dtype=torch.float64) for q in qs[:3])
        y, a2, b2, p2 = O.wkv_naive(w, u, k, v, *ref_state)
        want = O.mm8_naive(y * torch.sigmoid(r), *qs[3], dtype=torch.float64)
        ref_state = (a2, b2, p2)
        for m in (scripted, loaded):
            st = tuple(t.clone() for t in got_state)
            out, a3, b3, p3 = m(x.cuda(), *st)
            assert (out.cpu() - want).abs().max() < 1e-4
            # (k and v reach the operator rounded to float32, as in the reference; aa is a signed sum, so it is
            # measured against the size of the sums, not element by element)
            assert ((b3.cpu() - b2).abs() <= 1e-4 * b2.abs() + 1e-30).all()
            assert ((a3.cpu() - a2).abs() <= 1e-4 * torch.maximum(a2.abs(), b2) + 1e-30).all()
        got_state = (a3, b3, p3)
        x = x + want * 0.5


def test_mm8_three_against_the_float64_product_directly():
    from rwkvstic_amd import ops
    n_in, n_out = 640, 523
    g = torch.Generator().manual_seed(12)
    ws = [torch.randint(0, 256, (n_in, n_out), generator=g, dtype=torch.uint8) for _ in range(3)]
    rs = [torch.rand(n_in, generator=g) * 1e-3 for _ in range(3)]
    xs = [torch.randn(n_in, generator=g) for _ in range(3)]
    ys = [torch.randn(n_out, generator=g) for _ in range(3)]
    got = [y.clone().cuda() for y in ys]
    ops.register_torch_ops()
    torch.ops.rwkv.mm8_three(n_in, n_out, *[x.cuda() for x in xs], *[w.cuda() for w in ws], *got, *[r.cuda() for r in rs])
    for i in range(3):
        want = ys[i].double() + (xs[i].double() * rs[i].double()) @ ws[i].double()       # accumulates into y
        scale = ((xs[i].abs().double() * rs[i].double()) @ ws[i].double()).max()
        assert (got[i].cpu().double() - want).abs().max() <= 2.0 ** -23 * 8 * scale + 1e-6 * ys[i].abs().max()


class _Holder(torch.nn.Module):
    """A module tree that only holds tensors under given attribute paths."""

    def __init__(self):
        super().__init__()


def _tree_module(tree):
    root = _Holder()
    for path, t in tree.items():
        node = root
        parts = path.split(".")
        for p in parts[:-1]:
            if not hasattr(node, p):
                node.add_module(p, _Holder())
            node = getattr(node, p)
        node.register_buffer(parts[-1], t.clone())
    return root


def test_archive_with_the_reference_attribute_tree_rebuilds_the_model(tmp_path):
    """A torch.jit archive whose state_dict() carries the quantised model under the reference's names
    (blocks.i.att.weights.0.{weight,range,offset}[1,2], ..., emb.w, emptyState) -> HipRWKV.from_quantized."""
    from rwkvstic_amd.model import HipRWKV
    sd = synth.make_state_dict(layers=2, C=64, V=300, seed=14, ln="random")
    hip = HipRWKV(sd)
    path = str(tmp_path / "model.rwkv")
    torch.jit.save(torch.jit.script(_tree_module(hip.quantized_tree())), path)
    loaded = torch.jit.load(path, map_location="cpu")       # this test's own file
    again = HipRWKV.from_quantized(dict(loaded.state_dict()))
    toks = synth.random_tokens(9, V=300, seed=3).tolist()
    l1, s1 = hip.forward(toks, hip.emptyState.clone())
    l2, s2 = again.forward(toks, again.emptyState.clone())
    assert torch.equal(l1, l2) and torch.equal(s1, s2)
    ref = O.OracleModel(sd)
    lr, _ = ref.forward(toks, ref.emptyState.clone())
    assert (l2.cpu() - lr).abs().max() < 1e-3


def test_rwkv_archive_is_read_without_running_its_code(tmp_path):
    """RWKV("model.rwkv") (load.py:42-47 -> opt.py:89-92): the archive's tensors are taken by attribute path with a
    restricted unpickler (no torch.jit.load), the codes are only repacked; same results as the model quantised here
    from the float checkpoint.  The archive is this test's own, with the reference's attribute tree held as plain
    tensor attributes; a real export of the reference does not exist here (parity with one: unpinned)."""
    from archive_standins import write_archive
    from rwkvstic_amd.master import RWKV, greedy
    from rwkvstic_amd.model import HipRWKV
    sd = synth.make_state_dict(layers=2, C=64, V=300, seed=14, ln="random")
    path = str(tmp_path / "model.rwkv")
    write_archive(sd, path)
    r = RWKV(path, sampler=greedy)
    hip = HipRWKV(sd)
    toks = synth.random_tokens(9, V=300, seed=3).tolist()
    l1, s1 = hip.forward(toks, hip.emptyState.clone())
    l2, s2 = r.model.forward(toks, r.emptyState.clone())
    # codes and ranges are bit-equal; the offsets hold a mean whose summation order differs in the last bits
    assert (l1 - l2).abs().max() < 1e-9 and (s1[:, :2] - s2[:, :2]).abs().max() < 1e-9
    ref = O.OracleModel(sd)
    lr, _ = ref.forward(toks, ref.emptyState.clone())
    assert (l2.cpu() - lr).abs().max() < 1e-3
    out = r.forward(number=3, stopTokens=[], end_adj=0.0)
    assert len(out["output"].split()) == 3
