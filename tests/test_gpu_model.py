"""GPU parity of the whole-model forward against the CPU oracle (the reference's CPU path restated)."""
import pytest
import torch

from oracle import rwkv_oracle as O
from rwkvstic_amd import synth

pytestmark = pytest.mark.gpu

LOGIT_TOL = 1e-3       # max-abs on logits against the float32 CPU path
STATE_TOL = 1e-4       # relative, WKV state in the reference convention, against exact accumulation
# The float32 CPU path is itself only reproducible to a few 1e-4 (its BLAS sums the all-positive
# relu^2 products of the F-long ffn value matvec in float32 and the total then cancels against the
# zero-point term; 1 vs 8 BLAS threads move its logits by 3e-4 at C=2560).  State rows are therefore
# compared at STATE_TOL against the same network with float64 accumulation (the reference's
# naivedtype=float64 configuration) and at NOISY_STATE_TOL against the float32 path.
NOISY_STATE_TOL = 2e-3


def _say(msg):
    print(msg, flush=True)


def _state_close(st_gpu, st_ref, tol=NOISY_STATE_TOL):
    from rwkvstic_amd.model import wkv_state_to_reference
    s = wkv_state_to_reference(st_gpu).cpu()
    # shift rows: LayerNorm outputs, O(1)
    assert (s[:, 0] - st_ref[:, 0]).abs().max() < 10 * tol
    assert (s[:, 1] - st_ref[:, 1]).abs().max() < 10 * tol
    bb_ref = st_ref[:, 3]
    assert ((s[:, 3] - bb_ref).abs() <= tol * bb_ref.abs() + 1e-30).all(), "bb"
    assert ((s[:, 2] - st_ref[:, 2]).abs() <= tol * torch.maximum(st_ref[:, 2].abs(), bb_ref) + 1e-30).all(), "aa"


@pytest.fixture(scope="module")
def tiny():
    from rwkvstic_amd.model import HipRWKV
    sd = synth.make_state_dict(layers=3, C=64, V=512, seed=5, ln="random")
    return O.OracleModel(sd), HipRWKV(sd)


def test_tiny_single_tokens(tiny):
    ref, hip = tiny
    assert hip.layers == 3 and hip.dims == 64 and hip.vocab == 512
    assert torch.equal(hip.emptyState.cpu(), ref.emptyState)
    toks = synth.random_tokens(12, V=512, seed=3).tolist()
    sr, sg = ref.emptyState.clone(), hip.emptyState.clone()
    for i, t in enumerate(toks):
        _say(f"tiny token {i}")
        lr, sr = ref.forward([t], sr)
        lg, sg = hip.forward([t], sg)
        assert (lg.cpu() - lr).abs().max() < LOGIT_TOL
        assert int(lg.argmax()) == int(lr.argmax())
    _state_close(sg, sr)


def test_tiny_chunked_prefill_matches_oracle_and_single_steps(tiny):
    ref, hip = tiny
    toks = synth.random_tokens(19, V=512, seed=4).tolist()
    lr, sr = ref.forward(toks, ref.emptyState.clone())
    lg, sg = hip.forward(toks, hip.emptyState.clone())
    assert (lg.cpu() - lr).abs().max() < LOGIT_TOL
    _state_close(sg, sr)
    # chunk-size invariance on the GPU path itself
    s2 = hip.emptyState.clone()
    l2, s2 = hip.forward(toks[:7], s2)
    l2, s2 = hip.forward(toks[7:], s2)
    assert (l2 - lg).abs().max() < 1e-5
    assert (s2[:, :2] - sg[:, :2]).abs().max() < 1e-6


def test_ragged_shape_model():
    """C not a multiple of 128, V not a multiple of 8, F != 4C."""
    from rwkvstic_amd.model import HipRWKV
    sd = synth.make_state_dict(layers=2, C=72, F=200, V=301, seed=8, ln="random")
    ref, hip = O.OracleModel(sd), HipRWKV(sd)
    toks = synth.random_tokens(6, V=301, seed=1).tolist()
    sr, sg = ref.emptyState.clone(), hip.emptyState.clone()
    for t in toks:
        lr, sr = ref.forward([t], sr)
        lg, sg = hip.forward([t], sg)
        assert (lg.cpu() - lr).abs().max() < LOGIT_TOL
    _state_close(sg, sr)


def test_decode_greedy_device_loop_matches_host_loop(tiny):
    ref, hip = tiny
    s1 = hip.emptyState.clone()
    toks, logits, s1 = hip.decode_greedy(17, 10, s1)
    s2 = hip.emptyState.clone()
    t, out = 17, []
    for _ in range(10):
        l2, s2 = hip.forward([t], s2)
        t = int(l2.argmax()); out.append(t)
    assert toks.tolist() == out
    assert torch.equal(logits, l2) and torch.equal(s1, s2)


def test_forward_rejects_bad_state(tiny):
    _, hip = tiny
    with pytest.raises(ValueError):
        hip.forward([1], hip.emptyState.clone().float())
    with pytest.raises(ValueError):
        hip.forward([1], hip.emptyState.clone()[:2])
    with pytest.raises(ValueError):
        hip.forward([], hip.emptyState.clone())
    # ids given on the host are checked there, as the reference's host-side table lookup is (emb.py:9)
    for bad in ([512], [3, -1], torch.tensor([0, 600])):
        with pytest.raises(IndexError):
            hip.forward(bad, hip.emptyState.clone())
    with pytest.raises(IndexError):
        hip.decode_greedy(512, 2, hip.emptyState.clone())
    with pytest.raises(IndexError):
        hip.forward_batch([1, 999], torch.stack([hip.emptyState.clone()] * 2))
    # ids already on the device are not read back; the kernels clamp them to the table
    lg, _ = hip.forward(torch.tensor([600], device="cuda"), hip.emptyState.clone())
    lc, _ = hip.forward([511], hip.emptyState.clone())
    assert torch.equal(lg, lc)


def test_169m_shape_greedy_128_tokens():
    """The plumbing configuration: 12 layers, C=768, F=3072, V=50277; 32-token prompt, 128 greedy tokens."""
    from rwkvstic_amd.model import HipRWKV
    L, C, F, V = synth.SHAPES["169M"]
    sd = synth.make_state_dict(L, C, F, V, seed=0)          # the configuration as stated: LayerNorm weight 1, bias 0
    ref, hip = O.OracleModel(sd), HipRWKV(sd)
    exact = O.OracleModel(sd, matmul_dtype=torch.float64)
    assert hip.weight_bytes() == 130_625_280
    prompt = synth.random_tokens(32, V=V, seed=0).tolist()
    _say("169M oracle greedy (CPU) ...")
    toks_r, logits_r, st_r = ref.greedy(prompt, 128)
    _say("169M GPU prefill + greedy ...")
    st = hip.emptyState.clone()
    lg, st = hip.forward(prompt, st)
    worst = 0.0
    toks_g = []
    for i in range(128):
        worst = max(worst, float((lg.cpu() - logits_r[i]).abs().max()))
        t = int(lg.argmax())
        toks_g.append(t)
        lg, st = hip.forward([t], st)
    worst = max(worst, float((lg.cpu() - logits_r[128]).abs().max()))
    _say(f"169M worst logit max-abs {worst:.3e}")
    assert toks_g == toks_r, "greedy tokens differ from the CPU oracle"
    assert worst <= LOGIT_TOL
    _state_close(st, st_r)
    # the 1e-4 bound on the state holds against the same network with exact (float64) accumulation: the float32
    # path above is itself only reproducible to NOISY_STATE_TOL
    _say("169M oracle with float64 accumulation, same tokens ...")
    st_e = exact.emptyState.clone()
    _, st_e = exact.forward(prompt, st_e)
    for t in toks_g:
        le, st_e = exact.forward([t], st_e)
    assert (lg.cpu() - le).abs().max() < 1e-4
    _state_close(st, st_e, tol=STATE_TOL)


# ------------------------------------------------------------------ persistent single-token kernel
@pytest.mark.parametrize("C,L,V", [(1024, 2, 1999), (2560, 2, 5003), (2048, 1, 1600), (4096, 1, 1777), (5120, 2, 1777)])
def test_fused_step_matches_oracle_and_phase_kernels(C, L, V):
    from rwkvstic_amd.model import HipRWKV
    _say(f"fused step C={C} L={L} V={V}")
    sd = synth.make_state_dict(L, C, 4 * C, V, seed=C + L, ln="random")
    ref = O.OracleModel(sd)
    exact = O.OracleModel(sd, matmul_dtype=torch.float64)
    hip = HipRWKV(sd)
    plain = HipRWKV(sd, fused=False)
    assert hip.fused_step and not plain.fused_step
    toks = synth.random_tokens(6, V=V, seed=5).tolist()
    sr, se = ref.emptyState.clone(), exact.emptyState.clone()
    sg, sp = hip.emptyState.clone(), plain.emptyState.clone()
    for i, t in enumerate(toks):
        lr, sr = ref.forward([t], sr)
        le, se = exact.forward([t], se)
        lg, sg = hip.forward([t], sg)
        hip.check()
        lp, sp = plain.forward([t], sp)
        e_ref = float((lg.cpu() - lr).abs().max())
        e_ex = float((lg.cpu() - le).abs().max())
        e_pl = float((lg - lp).abs().max())
        _say(f"  token {i}: |fused-fp32 oracle| {e_ref:.2e}  |fused-fp64 oracle| {e_ex:.2e}  |fused-phase| {e_pl:.2e}"
             f"  (|fp32 oracle-fp64 oracle| {float((lr - le).abs().max()):.2e})")
        # Against the float32 CPU path the bound is 1e-3, unless that path's own float32 summation noise (its
        # distance from the same network with exact accumulation, printed above) is already of that size, as at
        # C=4096 with LayerNorm weights up to 1.5: then the kernel must sit within 5e-4 of the noise, and the
        # comparison that binds is the 1e-4 one against exact accumulation.
        noise = float((lr - le).abs().max())
        assert e_ref < max(LOGIT_TOL, noise + 5e-4) and e_pl < LOGIT_TOL
        assert e_ex < 1e-4
        assert int(lg.argmax()) == int(lr.argmax())
    _state_close(sg, sr)
    _state_close(sg, se, tol=STATE_TOL)
    _state_close(sp, se, tol=STATE_TOL)
    # determinism: integer accumulation makes a replay bit-identical
    s2 = hip.emptyState.clone()
    for t in toks:
        l2, s2 = hip.forward([t], s2)
    assert torch.equal(l2, lg) and torch.equal(s2, sg)


def test_fused_kernel_128_greedy_tokens_match_both_oracles():
    """The kernel the benchmark times, held to the parity statement itself: after a 32-token prompt, 128 greedy
    tokens through the persistent single-token kernel are the oracle's tokens, every logits vector is within
    1e-3 of the float32 CPU path, and the final state within 1e-4 of the same network with exact accumulation
    (its WKV sums and sigmoids are float32 where block.py:72 and operators.cu:21-36 are float64: this is the run
    that bounds the drift)."""
    from rwkvstic_amd.model import HipRWKV
    L, C, V = 4, 1024, 2003
    sd = synth.make_state_dict(L, C, 4 * C, V, seed=321, ln="random")
    ref, exact, hip = O.OracleModel(sd), O.OracleModel(sd, matmul_dtype=torch.float64), HipRWKV(sd)
    assert hip.fused_step
    prompt = synth.random_tokens(32, V=V, seed=6).tolist()
    toks_r, logits_r, st_r = ref.greedy(prompt, 128)
    st = hip.emptyState.clone()
    for t in prompt:                                   # the prompt too goes token by token through the kernel
        lg, st = hip.forward([t], st)
    toks_g, worst = [], 0.0
    for i in range(128):
        worst = max(worst, float((lg.cpu() - logits_r[i]).abs().max()))
        t = int(lg.argmax())
        toks_g.append(t)
        lg, st = hip.forward([t], st)
    hip.check()
    worst = max(worst, float((lg.cpu() - logits_r[128]).abs().max()))
    _say(f"fused kernel, 160 tokens: worst logit max-abs vs float32 oracle {worst:.3e}")
    assert toks_g == toks_r
    assert worst <= LOGIT_TOL
    _state_close(st, st_r)
    st_e = exact.emptyState.clone()
    for t in prompt + toks_g:
        le, st_e = exact.forward([t], st_e)
    e_ex = float((lg.cpu() - le).abs().max())
    _say(f"fused kernel, 160 tokens: final logits vs float64-accumulation oracle {e_ex:.3e}")
    assert e_ex < 1e-4
    _state_close(st, st_e, tol=STATE_TOL)
    # the device-side greedy loop produces the same 128 tokens
    s2 = hip.emptyState.clone()
    for t in prompt[:-1]:
        _, s2 = hip.forward([t], s2)
    toks_d, _, s2 = hip.decode_greedy(prompt[-1], 128, s2)
    hip.check()
    assert toks_d.tolist() == toks_r


@pytest.mark.parametrize("kind", ["offset", "outliers"])
def test_fused_kernel_layernorm_with_large_mean(kind):
    """LayerNorm inputs whose mean dwarfs their spread (every channel of the residual stream shifted by +30
    through the ln0 bias) or with a few huge channels: the statistics travel between workgroups as partial sums,
    and a variance formed as E[x^2] - mean^2 from rounded partials would lose digits here (layernorm.py:11-20
    subtracts the mean first)."""
    from rwkvstic_amd.model import HipRWKV
    L, C, V = 2, 1024, 1500
    sd = synth.make_state_dict(L, C, 4 * C, V, seed=99, ln="random")
    if kind == "offset":
        sd["blocks.0.ln0.bias"] = sd["blocks.0.ln0.bias"] + 30.0
    else:
        sd["blocks.0.ln0.bias"][[3, 500, 1023]] += torch.tensor([300.0, -250.0, 400.0])
    exact, hip = O.OracleModel(sd, matmul_dtype=torch.float64), HipRWKV(sd)
    assert hip.fused_step
    toks = synth.random_tokens(8, V=V, seed=8).tolist()
    se, sg = exact.emptyState.clone(), hip.emptyState.clone()
    for t in toks:
        le, se = exact.forward([t], se)
        lg, sg = hip.forward([t], sg)
    hip.check()
    err = float((lg.cpu() - le).abs().max())
    _say(f"large-mean LayerNorm ({kind}): |dlogits| vs float64-accumulation oracle {err:.3e}")
    assert err < 1e-4
    _state_close(sg, se, tol=STATE_TOL)
    # the many-row path on the same model
    lp, sp = hip.forward(toks, hip.emptyState.clone())
    assert float((lp.cpu() - le).abs().max()) < 1e-4
    _state_close(sp, se, tol=STATE_TOL)


def test_fused_greedy_device_loop_matches_host_loop():
    """rwkv_model_decode_greedy on the persistent kernel: argmax and the preparation of the next step run in one
    launch between the token kernels; tokens, logits and state must equal forward() + host argmax, bit for bit
    (rwkvMaster.py:28-56 with the sampler replaced by argmax)."""
    from rwkvstic_amd.model import HipRWKV
    sd = synth.make_state_dict(2, 1024, 4096, 1999, seed=77, ln="random")
    hip = HipRWKV(sd)
    assert hip.fused_step
    s1 = hip.emptyState.clone()
    _, s1 = hip.forward(synth.random_tokens(3, V=1999, seed=9).tolist(), s1)      # a non-trivial starting state
    s2 = s1.clone()
    toks, logits, s1 = hip.decode_greedy(17, 9, s1)
    hip.check()
    t, out = 17, []
    for _ in range(9):
        l2, s2 = hip.forward([t], s2)
        t = int(l2.argmax()); out.append(t)
    hip.check()
    assert toks.tolist() == out
    assert torch.equal(logits, l2) and torch.equal(s1, s2)
    # the loop leaves the model usable for plain steps (its last launch prepared a step that is prepared again)
    l3, s3 = hip.forward([out[-1]], s2.clone())
    toks4, l4, s4 = hip.decode_greedy(out[-1], 1, s1.clone())
    assert torch.equal(l3, l4) and torch.equal(s3, s4)


@pytest.mark.parametrize("n_prompt", [23, 100])      # 100: the chunked WKV scan (3 full chunks + a partial one)
def test_prompt_gemm_path_matches_token_steps(tiny, n_prompt):
    """A prompt through the GEMM path leaves the same logits and state as the same tokens fed one at a time
    (chunk-size invariance; block.py:58-67 token shift, wkv.py:23-39 recurrence)."""
    ref, hip = tiny
    toks = synth.random_tokens(n_prompt, V=512, seed=11).tolist()
    lg, sg = hip.forward(toks, hip.emptyState.clone())
    s1 = hip.emptyState.clone()
    for t in toks:
        l1, s1 = hip.forward([t], s1)
    _say(f"prompt-vs-steps |dlogits| {(lg - l1).abs().max().item():.2e}")
    assert (lg - l1).abs().max() < 1e-5
    assert (sg[:, :2] - s1[:, :2]).abs().max() < 1e-6
    from rwkvstic_amd.model import wkv_state_to_reference
    a, b = wkv_state_to_reference(sg), wkv_state_to_reference(s1)
    assert ((a[:, 3] - b[:, 3]).abs() <= 1e-6 * b[:, 3].abs() + 1e-30).all()
    assert ((a[:, 2] - b[:, 2]).abs() <= 1e-6 * torch.maximum(b[:, 2].abs(), b[:, 3]) + 1e-30).all()


def test_prompt_longer_than_one_pass(tiny):
    """A prompt of more rows than one pass of the many-row kernels takes (1024): the state is carried from pass to
    pass inside one call; against the CPU oracle and against the same prompt fed as two calls."""
    ref, hip = tiny
    toks = synth.random_tokens(1100, V=512, seed=12).tolist()
    lr, sr = ref.forward(toks, ref.emptyState.clone())
    lg, sg = hip.forward(toks, hip.emptyState.clone())
    _say(f"1100-token prompt |dlogits| vs oracle {(lg.cpu() - lr).abs().max().item():.2e}")
    assert (lg.cpu() - lr).abs().max() < LOGIT_TOL and int(lg.argmax()) == int(lr.argmax())
    _state_close(sg, sr)
    _, s2 = hip.forward(toks[:700], hip.emptyState.clone())
    l2, s2 = hip.forward(toks[700:], s2)
    assert (lg - l2).abs().max() < 1e-5 and (sg[:, :2] - s2[:, :2]).abs().max() < 1e-6


def test_long_prompts_hold_the_state_bound_against_exact_accumulation():
    """2200 tokens on a model with slowly forgetting channels (time_decay down to -8: histories of thousands of
    tokens): the float32 sums of the chunked WKV scan, carried from pass to pass, stay within the 1e-4 state bound
    of the float64 recurrence (operators.cu:21-36), whether the prompt is one call or 1024-token chunks."""
    from rwkvstic_amd.model import HipRWKV
    sd = synth.make_state_dict(layers=3, C=64, V=512, seed=15, ln="random")
    for i in range(3):
        sd[f"blocks.{i}.att.time_decay"][: 32] = torch.linspace(-8.0, -5.0, 32)
    exact, hip = O.OracleModel(sd, matmul_dtype=torch.float64), HipRWKV(sd)
    toks = synth.random_tokens(2200, V=512, seed=13).tolist()
    le, se = exact.forward(toks, exact.emptyState.clone())
    lg, sg = hip.forward(toks, hip.emptyState.clone())
    _say(f"2200-token prompt |dlogits| vs float64-accumulation oracle {(lg.cpu() - le).abs().max().item():.2e}")
    assert (lg.cpu() - le).abs().max() < 1e-4 and int(lg.argmax()) == int(le.argmax())
    _state_close(sg, se, tol=STATE_TOL)
    s2 = hip.emptyState.clone()
    for i in range(0, len(toks), 1024):
        l2, s2 = hip.forward(toks[i:i + 1024], s2)
    assert (l2.cpu() - le).abs().max() < 1e-4
    _state_close(s2, se, tol=STATE_TOL)
    # and token by token through the per-phase kernels for the last stretch
    s3 = hip.emptyState.clone()
    _, s3 = hip.forward(toks[:2100], s3)
    for t in toks[2100:]:
        l3, s3 = hip.forward([t], s3)
    assert (l3.cpu() - le).abs().max() < 1e-4
    _state_close(s3, se, tol=STATE_TOL)


def test_prompt_gemm_path_mid_shape_vs_fp64_oracle():
    """C=256, F=1024, ragged vocabulary; 70 tokens (18 M-tiles: a partial 64-token workgroup tile)."""
    from rwkvstic_amd.model import HipRWKV
    sd = synth.make_state_dict(layers=2, C=256, F=1024, V=1203, seed=21, ln="random")
    ref, hip = O.OracleModel(sd, matmul_dtype=torch.float64), HipRWKV(sd)
    toks = synth.random_tokens(70, V=1203, seed=2).tolist()
    lr, sr = ref.forward(toks, ref.emptyState.clone())
    lg, sg = hip.forward(toks, hip.emptyState.clone())
    _say(f"prompt |dlogits| vs fp64 oracle {(lg.cpu() - lr).abs().max().item():.2e}")
    assert (lg.cpu() - lr).abs().max() < 1e-4
    _state_close(sg, sr, tol=STATE_TOL)


@pytest.mark.parametrize("B", [5, 20])      # 5: the products of at most 8 rows; 20: the 9..32-row variant
def test_forward_batch_matches_per_sequence_steps(tiny, B):
    ref, hip = tiny
    states, toks = [], []
    for b in range(B):
        s = hip.emptyState.clone()
        if b:                                     # sequence 0 starts from the empty state
            _, s = hip.forward(synth.random_tokens(3 + b % 7, V=512, seed=30 + b).tolist(), s)
        states.append(s)
        toks.append(int(synth.random_tokens(1, V=512, seed=40 + b)[0]))
    batch_state = torch.stack(states).contiguous()
    for step in range(3):
        lb, batch_state = hip.forward_batch(toks, batch_state)
        nxt = []
        for b in range(B):
            l1, states[b] = hip.forward([toks[b]], states[b])
            assert (lb[b] - l1).abs().max() < 1e-5, (step, b)
            assert (batch_state[b, :, :2] - states[b][:, :2]).abs().max() < 1e-6
            lr = None
            nxt.append(int(l1.argmax()))
            assert int(lb[b].argmax()) == nxt[-1]
        toks = nxt
    with pytest.raises(ValueError):
        hip.forward_batch(toks, batch_state[:2])


SWEEP = [  # layers, C, F, V, prompt length, chunking, batch sizes (None: widths the batch path does not take)
    (2, 72, 200, 301, 63, (31, 1, 31), None),
    (3, 128, 512, 1000, 130, (3, 31, 1, 95), (1, 2, 40, 127, 128, 131)),     # 128: where the batch path changes its row kernels
    (2, 192, 768, 777, 64, (64,), (3, 33)),
    (2, 448, 1000, 333, 130, (3, 7, 7, 64, 49), None),
    (2, 512, 2048, 50277, 257, (31, 31, 2, 16, 100, 16, 1, 60), (17,)),
    (1, 640, 2560, 4097, 64, (16, 31, 16, 1), (5, 40)),
    (1, 64, 64, 17, 257, (1, 31, 100, 2, 100, 23), (9,)),
    (1, 2048, 8192, 1234, 63, (7, 56), (5, 33)),
]


@pytest.mark.parametrize("L,C,F,V,T,cuts,batches", SWEEP)
@pytest.mark.parametrize("fused", [True, False])
def test_shapes_chunkings_and_batches_against_the_exact_oracle(L, C, F, V, T, cuts, batches, fused):
    """Widths that are and are not multiples of 64 / 128 / 512, ffn widths other than 4 C, small and full
    vocabularies: a prompt in one pass and cut into uneven pieces against the float64-accumulating oracle, the greedy
    device loop against the host loop, and batch steps against the same sequences stepped one by one.  With
    ``fused`` the products accumulate exactly (logits within 2e-5 of the oracle, measured 5e-7); without it the
    single-token steps follow the reference's float32 kernels."""
    from rwkvstic_amd.model import HipRWKV
    sd = synth.make_state_dict(layers=L, C=C, F=F, V=V, seed=100 + C, ln="random")
    ref, hip = O.OracleModel(sd, matmul_dtype=torch.float64), HipRWKV(sd, fused=fused)
    toks = synth.random_tokens(T, V=V, seed=C + 1).tolist()
    assert sum(cuts) == T
    lr, sr = ref.forward(toks, ref.emptyState.clone())
    lg, sg = hip.forward(toks, hip.emptyState.clone())
    tol = 2e-5 if fused else 2e-4
    _say(f"C={C} fused={fused}: one pass |dlogits| {(lg.cpu() - lr).abs().max().item():.2e}")
    assert (lg.cpu() - lr).abs().max() < tol
    _state_close(sg, sr, tol=STATE_TOL)
    s2, i = hip.emptyState.clone(), 0
    for n in cuts:
        l2, s2 = hip.forward(toks[i:i + n], s2)
        i += n
    assert (l2.cpu() - lr).abs().max() < tol
    _state_close(s2, sr, tol=STATE_TOL)
    hip.check()
    # greedy loop on the device == host loop
    t0 = int(lg.argmax())
    sa, sb = sg.clone(), sg.clone()
    tk, la, sa = hip.decode_greedy(t0, 4, sa)
    cur, host = t0, []
    for _ in range(4):
        lb, sb = hip.forward([cur], sb)
        cur = int(lb.argmax())
        host.append(cur)
    assert tk.tolist() == host and (la - lb).abs().max() < 1e-9
    if not (fused and batches):
        return
    for B in batches:
        states = torch.stack([hip.emptyState.clone() for _ in range(B)])
        for b in range(B):                        # every sequence with its own history
            hip.forward(synth.random_tokens(1 + b % 3, V=V, seed=C + 11 + b).tolist(), states[b])
        singles = states.clone()
        btoks = synth.random_tokens(B, V=V, seed=C + 7).tolist()
        lbt, states = hip.forward_batch(btoks, states)
        for b in range(B):
            l1, _ = hip.forward([btoks[b]], singles[b])
            assert (lbt[b] - l1).abs().max() < 1e-5, (B, b)
            assert (states[b][:, :2] - singles[b][:, :2]).abs().max() < 1e-6, (B, b)
    hip.check()


def test_rwkv_shell_loads_checkpoint_file_and_generates(tmp_path, tiny):
    """RWKV(path) -> RWKVMaster surface (load.py:18,42-47; rwkvMaster.py:28-105) over the HIP model."""
    from rwkvstic_amd.master import RWKV, greedy
    ref, hip = tiny
    sd = synth.make_state_dict(layers=3, C=64, V=512, seed=5, ln="random")
    path = str(tmp_path / "tiny.pth")
    torch.save(sd, path)
    r = RWKV(path, sampler=greedy)
    assert torch.equal(r.emptyState, hip.emptyState)
    prompt = synth.random_tokens(9, V=512, seed=12).tolist()
    ids, st = r.loadContext(newctx=prompt, ctx=[int(prompt[-1])])
    assert ids == prompt and r.lastToken == [prompt[-1]]
    # the reference feeds lastToken again after loadContext (rwkvMaster.py:31-33); mirror that here
    out = r.forward(number=6, stopTokens=[], end_adj=0.0)
    s2 = hip.emptyState.clone()
    _, s2 = hip.forward(prompt, s2)
    toks, _, s2 = hip.decode_greedy(prompt[-1], 6, s2)
    assert out["output"] == " ".join(str(int(t)) for t in toks)
    assert torch.equal(out["state"], s2)


def test_rwkv_shell_takes_the_reference_loader_options(tmp_path, tiny):
    """opt.py:15-19,112-116: ``export`` writes the quantised model and ends the program; ``config`` names the GPU and
    may ask for host-resident codes; what is loaded back from the export gives the same logits bit for bit."""
    import os
    from rwkvstic_amd.master import RWKV, greedy
    _, hip = tiny
    sd = synth.make_state_dict(layers=3, C=64, V=512, seed=5, ln="random")
    path, stem = str(tmp_path / "tiny.pth"), str(tmp_path / "exported")
    torch.save(sd, path)
    with pytest.raises(SystemExit):
        RWKV(path, jit=False, export=stem)
    assert os.path.exists(stem + ".rwkvq")
    toks = synth.random_tokens(7, V=512, seed=2).tolist()
    want, _ = hip.forward(toks, hip.emptyState.clone())
    cfg = {"devices": [{"device": "cuda:0", "dtype": torch.uint8, "stream": True}]}
    for r in (RWKV(stem + ".rwkvq", sampler=greedy), RWKV(stem + ".rwkvq", sampler=greedy, config=cfg),
              RWKV(path, sampler=greedy, config=cfg)):
        got, _ = r.model.forward(toks, r.emptyState.clone())
        assert torch.equal(got, want)
    assert not RWKV(path, config=cfg).model.blocks[0]["att_k"].packed.is_cuda        # the codes stayed on the host


def test_quantized_tree_round_trip_and_oracle_layout(tmp_path, tiny):
    """The quantised model under the reference's attribute names (what its .rwkv export holds, opt.py:89-92;
    names from matmul.py:12,67-68, block.py:13-47, opt.py:31-48): the codes and ranges equal the CPU oracle's
    quantiser output bit for bit (offsets to the last bits), and a model rebuilt from the tree (no second quantisation) gives identical results."""
    from rwkvstic_amd.master import RWKV, greedy
    from rwkvstic_amd.model import HipRWKV
    ref, hip = tiny
    sd = synth.make_state_dict(layers=3, C=64, V=512, seed=5, ln="random")
    tree = hip.quantized_tree()
    assert tree["emptyState"].shape == (3, 5, 64) and tree["emb.w"].shape == (512, 64)
    assert tree["blocks.0.attmix"].shape == (3, 1, 64) and tree["blocks.2.ffnmix"].shape == (2, 1, 64)
    names = {"blocks.1.att.weights.0.": ("blocks.1.att.key.weight", "blocks.1.att.value.weight", "blocks.1.att.receptance.weight"),
             "blocks.1.attout.weights.0.": ("blocks.1.att.output.weight",), "blocks.1.ffnkey.weights.0.": ("blocks.1.ffn.key.weight",),
             "blocks.1.ffnvalue.weights.0.": ("blocks.1.ffn.value.weight",),
             "blocks.1.ffnreceptance.weights.0.": ("blocks.1.ffn.receptance.weight",), "head.weights.0.": ("head.weight",)}
    for prefix, keys in names.items():
        for suffix, key in zip(("", "1", "2"), keys):
            codes, rng, off = O.quantize_matrix(sd[key].float())
            assert tree[prefix + "weight" + suffix].dtype == torch.uint8
            assert torch.equal(tree[prefix + "weight" + suffix], codes), (prefix, suffix)       # [in, out]
            assert torch.equal(tree[prefix + "range" + suffix], rng) and rng.dtype == torch.float32
            # (the offset holds a mean of fractions: equal up to the order of that one sum)
            assert torch.allclose(tree[prefix + "offset" + suffix], off, rtol=1e-13, atol=1e-300) and off.dtype == torch.float64
    assert torch.equal(tree["blocks.1.time_decay"], sd["blocks.1.att.time_decay"].reshape(-1).double().exp().neg())
    again = HipRWKV.from_quantized(tree)
    toks = synth.random_tokens(7, V=512, seed=31).tolist()
    l1, s1 = hip.forward(toks, hip.emptyState.clone())
    l2, s2 = again.forward(toks, again.emptyState.clone())
    assert torch.equal(l1, l2) and torch.equal(s1, s2)
    # through a file and the loader shell
    path = str(tmp_path / "tiny.rwkvq")
    hip.save_quantized(path)
    r = RWKV(path, sampler=greedy)
    l3, s3 = r.model.forward(toks, r.emptyState.clone())
    assert torch.equal(l1, l3) and torch.equal(s1, s3)
    with pytest.raises(ValueError):
        bad = dict(tree)
        bad["head.weights.0.weight"] = bad["head.weights.0.weight"].float()
        HipRWKV.from_quantized(bad)


def test_host_resident_weights_give_identical_results():
    """stream=True (matmul.py:21,186: the codes stay in host memory): the kernels read the pinned host copies in
    place; logits and state are bit-identical to the device-resident model, on the prompt path, the persistent
    single-token kernel and the per-phase kernels."""
    from rwkvstic_amd.model import HipRWKV
    sd = synth.make_state_dict(2, 1024, 4096, 1999, seed=31, ln="random")
    dev, host = HipRWKV(sd), HipRWKV(sd, stream=True)
    assert host.fused_step and not host.blocks[0]["att_k"].packed16.is_cuda and host.blocks[0]["att_k"].packed16.is_pinned()
    toks = synth.random_tokens(9, V=1999, seed=4).tolist()
    l1, s1 = dev.forward(toks, dev.emptyState.clone())
    l2, s2 = host.forward(toks, host.emptyState.clone())
    assert torch.equal(l1, l2) and torch.equal(s1, s2)
    for t in (5, 77):
        l1, s1 = dev.forward([t], s1)
        l2, s2 = host.forward([t], s2)
        host.check()
        assert torch.equal(l1, l2) and torch.equal(s1, s2)
    tiny_sd = synth.make_state_dict(layers=2, C=72, F=200, V=301, seed=8, ln="random")
    a, b = HipRWKV(tiny_sd), HipRWKV(tiny_sd, stream=True)
    la, sa = a.forward([3, 4], a.emptyState.clone())
    lb, sb = b.forward([3, 4], b.emptyState.clone())
    assert torch.equal(la, lb) and torch.equal(sa, sb)


@pytest.mark.parametrize("C,L", [(1024, 2), (2560, 1), (5120, 1)])
def test_a_token_step_that_never_gets_its_input_drains_and_is_reported(C, L):
    """The failure path of the persistent kernel, forced from the host without anything that could hang: a token
    step is launched whose input is never published and whose waits give up after a few hundred polls.  Every
    workgroup must leave (the launch ends), the state must be untouched, check() must report the step once, and
    the steps after it must give exactly what a model that never saw the failure gives."""
    from rwkvstic_amd.model import HipRWKV
    V = 1500
    sd = synth.make_state_dict(L, C, 4 * C, V, seed=77 + C, ln="random")
    hip, clean = HipRWKV(sd), HipRWKV(sd)
    assert hip.fused_step
    toks = synth.random_tokens(4, V=V, seed=3).tolist()
    s, sc = hip.emptyState.clone(), clean.emptyState.clone()
    for t in toks[:2]:
        _, s = hip.forward([t], s)
        _, sc = clean.forward([t], sc)
    before = s.clone()
    _say(f"unfed token step, C={C}")
    hip.selftest_timeout(s)
    with pytest.raises(RuntimeError, match="gave up waiting"):
        hip.check()
    assert torch.equal(s, before)
    hip.check()                                        # reported once, then clear
    for t in toks[2:]:
        lg, s = hip.forward([t], s)
        lc, sc = clean.forward([t], sc)
    hip.check()
    assert torch.equal(lg, lc) and torch.equal(s, sc)


def test_timed_token_steps_advance_the_state_like_forward():
    """rwkv_model_time_token_kernel: n steps with events around the persistent kernel only; the state it leaves is
    the one n forward() calls leave, and the duration is a plausible positive number."""
    from rwkvstic_amd.model import HipRWKV
    L, C, V = 2, 1024, 1200
    sd = synth.make_state_dict(L, C, 4 * C, V, seed=12, ln="random")
    hip = HipRWKV(sd)
    assert hip.fused_step
    s1, s2 = hip.emptyState.clone(), hip.emptyState.clone()
    us = hip.time_token_kernel(17, 5, s1)
    for _ in range(5):
        _, s2 = hip.forward([17], s2)
    hip.check()
    assert torch.equal(s1, s2)
    assert 1.0 < us < 5000.0
