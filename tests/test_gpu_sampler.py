"""The device-side sampler against the CPU restatement of the reference's `typical` (agnostic/samplers/typical.py:1-17):
the kept set, the distribution of 20,000 draws (chi-square), greedy mode, logit adjustment and stop tokens of the
device generation loop (rwkvMaster.py:28-56)."""
import pytest
import torch

from oracle import rwkv_oracle as O
from rwkvstic_amd import synth

pytestmark = pytest.mark.gpu


def _draws(ops, logits, n, **kw):
    out = torch.empty(n, dtype=torch.int64, device="cuda")
    lg = logits.cuda()
    for i in range(n):
        ops.sample_token(lg, counter=i, out=out[i:i + 1], **kw)
    torch.cuda.synchronize()
    return out.cpu()


@pytest.mark.parametrize("V,temp,tau", [(1000, 1.0, 0.8), (50277, 1.0, 0.8), (50277, 0.7, 0.95), (5000, 1.3, 0.5)])
def test_typical_draws_follow_the_reference_distribution(V, temp, tau):
    from rwkvstic_amd import ops
    g = torch.Generator().manual_seed(V + int(10 * temp))
    logits = (torch.randn(V, generator=g, dtype=torch.float64) * 2.5)
    logits[:5] += 4.0                                   # a few likely tokens on top of a long tail
    want = O.typical_distribution(logits, temp, tau)
    n = 20000
    got = _draws(ops, logits, n, temp=temp, tau=tau, seed=1234)
    assert int(got.min()) >= 0 and int(got.max()) < V
    # nothing outside the kept set is ever drawn (one borderline token may differ: the cut compares float32
    # running sums formed in different orders)
    outside = (want[got] == 0)
    assert int(outside.sum()) <= n * 2e-3
    # chi-square over the tokens with an expected count of at least 5, the rest pooled
    cnt = torch.bincount(got, minlength=V).double()
    exp = want * n
    big = exp >= 5
    chi = float((((cnt - exp) ** 2) / exp)[big].sum())
    rest_e, rest_c = float(exp[~big].sum()), float(cnt[~big].sum())
    if rest_e >= 5:
        chi += (rest_c - rest_e) ** 2 / rest_e
    dof = int(big.sum()) + (1 if rest_e >= 5 else 0) - 1
    print(f"V={V} temp={temp} tau={tau}: kept {int((want > 0).sum())} tokens, chi2 {chi:.1f} on {dof} dof", flush=True)
    assert chi < dof + 5.0 * (2 * dof) ** 0.5 + 10       # about five standard deviations


def test_tau_zero_and_a_vanishing_temperature_never_fall_back_to_token_0():
    """Probabilities (1/8, 1/4, 1/2, 1/8): distances of the surprises from the entropy are (1.25, 0.25, 0.75, 1.25) ln 2.
    tau = 0 keeps position #(cumulative < 0) = 0 of the sorted distances (typical.py:13-14): token 1, always.  With a
    temperature so small that every kept weight p^(1/temp) underflows the draw has nothing to draw from (the reference's
    multinomial raises there); the device sampler then returns the kept token with the largest logit, never token 0
    (which would read as end-of-text)."""
    from rwkvstic_amd import ops
    logits = torch.log(torch.tensor([0.125, 0.25, 0.5, 0.125], dtype=torch.float64)) - 1.5
    want = O.typical_distribution(logits, 1.0, 0.0)
    assert want.tolist() == [0.0, 1.0, 0.0, 0.0]
    got = _draws(ops, logits, 64, temp=1.0, tau=0.0, seed=5)
    assert got.tolist() == [1] * 64
    got = _draws(ops, logits, 64, temp=1e-3, tau=0.8, seed=5)          # kept: everything; 0.5 ** 1000 underflows
    assert got.tolist() == [2] * 64
    got = _draws(ops, logits, 64, temp=1e-3, tau=0.2, seed=5)          # kept: token 1 only
    assert got.tolist() == [1] * 64
    # the same on a real-sized vocabulary (the variant with keys in LDS and registers)
    g = torch.Generator().manual_seed(3)
    big = torch.randn(50277, generator=g, dtype=torch.float64) * 2.5
    want = O.typical_distribution(big, 1.0, 0.0)
    assert int((want > 0).sum()) == 1
    got = _draws(ops, big, 16, temp=1.0, tau=0.0, seed=9)
    assert got.tolist() == [int(want.argmax())] * 16


@pytest.mark.parametrize("spread,tau", [(0.02, 0.5), (0.3, 0.8)])
def test_typical_cut_on_a_nearly_flat_distribution(spread, tau):
    """Logits of a random-init model: 50277 tokens of almost equal probability, so tens of thousands of distances
    from the entropy share their leading bits (the search's list of undecided tokens overflows and it falls back to
    more passes over all tokens).  Tokens are grouped by their rank in distance; the draws per group must follow
    the oracle's kept mass per group - a cut too tight empties groups, one too wide fills groups that must stay empty."""
    from rwkvstic_amd import ops
    V, n, groups = 50277, 20000, 40
    g = torch.Generator().manual_seed(int(spread * 1000))
    logits = torch.randn(V, generator=g, dtype=torch.float64) * spread
    want = O.typical_distribution(logits, 1.0, tau)
    probs = torch.softmax(logits.float(), dim=-1)
    s = -torch.log(probs)
    d = (s - (s * probs).sum()).abs()
    rank = torch.argsort(torch.argsort(d))
    grp = (rank * groups // V).long()
    got = _draws(ops, logits, n, temp=1.0, tau=tau, seed=99)
    assert int((want[got] == 0).sum()) <= n * 2e-3
    exp = torch.zeros(groups, dtype=torch.float64).index_add_(0, grp, want) * n
    cnt = torch.bincount(grp[got], minlength=groups).double()
    big = exp >= 5
    chi = float((((cnt - exp) ** 2) / exp)[big].sum())
    dof = int(big.sum()) - 1
    print(f"spread={spread} tau={tau}: kept {int((want > 0).sum())} tokens, chi2 {chi:.1f} on {dof} dof", flush=True)
    assert float(cnt[~big].sum()) <= n * 2e-3 + float(exp[~big].sum()) * 3 + 5
    assert chi < dof + 5.0 * (2 * dof) ** 0.5 + 10


def test_greedy_mode_end_adj_and_determinism():
    from rwkvstic_amd import ops
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(777, generator=g, dtype=torch.float64)
    logits[0] = logits.max() + 1.0
    lg = logits.clone().cuda()
    assert int(ops.sample_token(lg, greedy=True)) == 0
    lg = logits.clone().cuda()
    t = int(ops.sample_token(lg, greedy=True, end_adj=-990.0))           # rwkvMaster.py:37
    assert t == int(logits[1:].argmax()) + 1 and float(lg[0]) == float(logits[0]) - 990.0
    a = _draws(ops, logits, 50, seed=9)
    b = _draws(ops, logits, 50, seed=9)
    c = _draws(ops, logits, 50, seed=10)
    assert torch.equal(a, b) and not torch.equal(a, c)


def test_device_generation_loop_matches_host_loop_and_stops_on_a_stop_token():
    from rwkvstic_amd import ops
    from rwkvstic_amd.model import HipRWKV
    sd = synth.make_state_dict(2, 1024, 4096, 1999, seed=5, ln="random")
    hip = HipRWKV(sd)
    assert hip.fused_step
    s0 = hip.emptyState.clone()
    _, s0 = hip.forward(synth.random_tokens(4, V=1999, seed=2).tolist(), s0)
    # device loop
    toks, logits, s1 = hip.decode_sample(17, 12, s0.clone(), temp=0.9, tau=0.8, end_adj=-990.0, seed=42)
    hip.check()
    assert toks.numel() == 12
    # the same loop from the host: forward, then one device draw with the same (seed, counter)
    s2, t, out = s0.clone(), 17, []
    for i in range(12):
        l2, s2 = hip.forward([t], s2)
        t = int(ops.sample_token(l2, temp=0.9, tau=0.8, end_adj=-990.0, seed=42, counter=i))
        out.append(t)
    assert toks.tolist() == out
    assert torch.equal(logits, l2) and torch.equal(s1, s2)
    # a stop token ends the loop on the device: state and logits are those of the stopping step
    stop_at = 5
    toks3, logits3, s3 = hip.decode_sample(17, 12, s0.clone(), temp=0.9, tau=0.8, end_adj=-990.0, seed=42,
                                           stop_tokens=[out[stop_at], 1998])
    hip.check()
    first = min(i for i, v in enumerate(out) if v in (out[stop_at], 1998))
    assert toks3.tolist() == out[:first + 1]
    s4, t = s0.clone(), 17
    for i in range(first + 1):
        l4, s4 = hip.forward([t], s4)
        t = int(ops.sample_token(l4, temp=0.9, tau=0.8, end_adj=-990.0, seed=42, counter=i))
    assert torch.equal(s3, s4) and torch.equal(logits3, l4)
    # the model keeps working after a stopped loop
    toks5, _, _ = hip.decode_sample(17, 3, s0.clone(), greedy=True)
    g2, _, _ = hip.decode_greedy(17, 3, s0.clone())
    assert toks5.tolist() == g2.tolist()


def test_master_forward_runs_the_loop_on_the_device():
    """RWKV(...).forward(number=n) (rwkvMaster.py:28-56) with the built-in samplers on a model the persistent kernel
    serves: same tokens as the explicit loops, state and lastToken updated as the reference does."""
    from rwkvstic_amd.master import RWKV, greedy, typical
    sd = synth.make_state_dict(2, 1024, 4096, 1999, seed=6, ln="random")
    r = RWKV(sd, sampler=greedy)
    hip = r.model
    assert hip.fused_step
    r.lastToken = [23]
    out = r.forward(number=7, stopTokens=[], end_adj=0.0)
    toks, logits, st = hip.decode_greedy(23, 7, hip.emptyState.clone())
    assert out["output"] == " ".join(str(int(t)) for t in toks)
    assert torch.equal(out["state"], st) and torch.equal(out["logits"], logits) and r.lastToken == [int(toks[-1])]
    assert torch.equal(r.myState, st)
    # typical: reproducible under torch.manual_seed, default end_adj keeps token 0 out
    outs = []
    for _ in range(2):
        torch.manual_seed(7)
        r2 = RWKV(sd, sampler=typical)
        r2.lastToken = [23]
        outs.append(r2.forward(number=9)["output"])
    assert outs[0] == outs[1] and len(outs[0].split()) == 9 and "0" not in outs[0].split()
    # a per-token callback falls back to the host loop and still works
    seen = []
    r3 = RWKV(sd, sampler=greedy)
    r3.lastToken = [23]
    o3 = r3.forward(number=4, stopTokens=[], end_adj=0.0, progressLambda=lambda d: seen.append(d["progress"]))
    assert seen == [0, 1, 2, 3] and o3["output"] == " ".join(str(int(t)) for t in toks[:4])
