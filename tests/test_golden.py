"""Frozen vectors (tests/golden/tiny_model.pt, written by tests/golden/make_golden.py from the pinned oracle): the
oracle must still reproduce them (CPU), and the HIP path must match them (GPU) to the parity bounds."""
import os

import pytest
import torch

from oracle import rwkv_oracle as O
from rwkvstic_amd import synth

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tiny_model.pt")
MATS = ("blocks.0.att.key.weight", "blocks.1.ffn.value.weight", "head.weight")


@pytest.fixture(scope="module")
def gold():
    g = torch.load(GOLD, map_location="cpu", weights_only=True)
    layers, C, F, V, seed, tseed, n = (int(x) for x in g["spec"])
    sd = synth.make_state_dict(layers=layers, C=C, F=F, V=V, seed=seed, ln="random")
    assert torch.equal(synth.random_tokens(n, V=V, seed=tseed), g["tokens"])
    return g, sd


def test_oracle_still_reproduces_the_frozen_vectors(gold):
    g, sd = gold
    for key in MATS:
        codes, rng, off = O.quantize_matrix(sd[key].float())
        assert torch.equal(codes, g[f"quant.{key}.codes"]) and torch.equal(rng, g[f"quant.{key}.range"])
        assert torch.allclose(off, g[f"quant.{key}.offset"], rtol=1e-13, atol=0)
    m = O.OracleModel(sd, matmul_dtype=torch.float64)
    st = m.emptyState.clone()
    for i, t in enumerate(g["tokens"].tolist()):
        lg, st = m.forward([t], st)
        assert (lg - g["logits.f64"][i]).abs().max() < 1e-9          # float64 throughout: order of sums only
    assert torch.allclose(st, g["state.f64"], rtol=1e-9, atol=1e-12)
    # the float32 path against its own frozen run: within float32 summation noise of this small model
    m32 = O.OracleModel(sd)
    st = m32.emptyState.clone()
    for i, t in enumerate(g["tokens"].tolist()):
        lg, st = m32.forward([t], st)
        assert (lg - g["logits.f32"][i]).abs().max() < 2e-5


@pytest.mark.gpu
def test_hip_path_matches_the_frozen_vectors(gold):
    from rwkvstic_amd import ops
    from rwkvstic_amd.model import HipRWKV, wkv_state_to_reference
    g, sd = gold
    for key in MATS:
        codes, rng, off = ops.quantize(sd[key].float().cuda().contiguous())
        assert torch.equal(codes.cpu(), g[f"quant.{key}.codes"]) and torch.equal(rng.cpu(), g[f"quant.{key}.range"])
        assert torch.allclose(off.cpu(), g[f"quant.{key}.offset"], rtol=1e-13, atol=0)
    hip = HipRWKV(sd)
    st = hip.emptyState.clone()
    for i, t in enumerate(g["tokens"].tolist()):
        lg, st = hip.forward([t], st)
        assert (lg.cpu() - g["logits.f32"][i]).abs().max() < 1e-3        # the parity bound against the float32 path
        assert (lg.cpu() - g["logits.f64"][i]).abs().max() < 1e-4        # and against exact accumulation
        assert int(lg.argmax()) == int(g["logits.f32"][i].argmax())
    s = wkv_state_to_reference(st).cpu()
    ref = g["state.f64"]
    assert (s[:, :2] - ref[:, :2]).abs().max() < 1e-4
    assert ((s[:, 3] - ref[:, 3]).abs() <= 1e-4 * ref[:, 3].abs() + 1e-30).all()
    assert ((s[:, 2] - ref[:, 2]).abs() <= 1e-4 * torch.maximum(ref[:, 2].abs(), ref[:, 3]) + 1e-30).all()
    # the prompt path on the same tokens
    lp, sp = hip.forward(g["tokens"].tolist(), hip.emptyState.clone())
    assert (lp.cpu() - g["logits.f64"][-1]).abs().max() < 1e-4
