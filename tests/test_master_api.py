"""Behaviour of the RWKVMaster-compatible shell (reference rwkvMaster.py:14-125) with a stub model; no GPU."""
import pytest
import torch

from rwkvstic_amd.master import RWKV, RWKVMaster, TokenIds, greedy, typical


class StubModel:
    """logits favour (last token + 1) mod V; the state counts the tokens it has seen."""
    V = 16

    def __init__(self):
        self.calls = []

    def forward(self, tokens, state):
        tokens = [int(t) for t in tokens]
        self.calls.append(tokens)
        state += len(tokens)                       # in place, like the real model
        logits = torch.zeros(self.V, dtype=torch.float64)
        logits[(tokens[-1] + 1) % self.V] = 5.0
        return logits, state


def _master(sampler=greedy):
    m = StubModel()
    return m, RWKVMaster(m, torch.zeros(1, dtype=torch.float64), sampler)


def test_defaults_and_state_api():
    m, r = _master()
    assert r.lastToken == [187] and float(r.myState) == 0.0
    r.setState((torch.full((1,), 7.0, dtype=torch.float64), [3]))
    st, last = r.getState()
    assert float(st) == 7.0 and last == [3]
    st += 1                                          # a clone: the master's own state is untouched
    assert float(r.myState) == 7.0
    r.resetState()
    assert float(r.myState) == 0.0 and r.lastToken == [187]


def test_forward_generates_until_number_and_updates_last_token():
    m, r = _master()
    r.lastToken = [2]
    out = r.forward(number=4, stopTokens=[])
    assert m.calls == [[2], [3], [4], [5]]
    assert out["output"] == "3 4 5 6" and r.lastToken == [6]
    assert float(out["state"]) == 4.0 and float(r.myState) == 4.0
    assert out["logits"][0] == -990.0               # end_adj lands on logit 0


def test_forward_stops_on_stop_token_and_stop_string():
    m, r = _master()
    r.lastToken = [2]
    assert r.forward(number=10, stopTokens=[5])["output"] == "3 4 5"
    m, r = _master()
    r.lastToken = [2]
    assert r.forward(number=10, stopTokens=[], stopStrings=["4"])["output"] == "3 4"
    # end_adj can pull the end token up as well as push it down
    m, r = _master()
    r.lastToken = [2]
    assert r.forward(number=3, end_adj=100.0)["output"] == "0"      # token 0 wins, and it is a stop token


class DeviceLoopStub(StubModel):
    """A model that offers the device-side loop: records whether it was used."""
    fused_step = True
    vocab = 16

    def decode_sample(self, token, n, state, **kw):
        self.device_calls = getattr(self, "device_calls", 0) + 1
        self.seeds = getattr(self, "seeds", []) + [kw["seed"]]
        toks = torch.tensor([(int(token) + 1 + i) % self.V for i in range(n)])
        return toks, torch.zeros(self.V, dtype=torch.float64), state


def test_device_loop_is_taken_only_when_it_cannot_change_the_result():
    """The whole-loop call is an optimisation of rwkvMaster.py:28-56: it must step aside for a vocabulary the device
    sampler cannot hold, and for stop strings that the decoded text could end with (ids decode to digits and spaces)."""
    def run(model, **kw):
        r = RWKVMaster(model, torch.zeros(1, dtype=torch.float64), greedy)
        r.lastToken = [2]
        out = r.forward(number=3, stopTokens=[], **kw)
        return getattr(model, "device_calls", 0), out["output"]
    assert run(DeviceLoopStub()) == (1, "3 4 5")                                   # the default stop string cannot match ids
    assert run(DeviceLoopStub(), stopStrings=[]) == (1, "3 4 5")
    assert run(DeviceLoopStub(), stopStrings=["4"]) == (0, "3 4")                  # host loop, and it stops as the reference does
    assert run(DeviceLoopStub(), stopStrings=["<|endoftext|>", "3 4"]) == (0, "3 4")
    assert run(DeviceLoopStub(), stopStrings=[""]) == (0, "3")                     # every text ends with the empty string
    big = DeviceLoopStub()
    big.vocab = 65536
    assert run(big) == (0, "3 4 5")
    # seeds: reproducible under torch.manual_seed, different from call to call and from master to master
    seeds = []
    for _ in range(2):
        torch.manual_seed(11)
        a, b = DeviceLoopStub(), DeviceLoopStub()
        run(a), run(a), run(b)
        seeds.append(a.seeds + b.seeds)
    assert seeds[0] == seeds[1] and len(set(seeds[0])) == 3


def test_forward_progress_callback_payload():
    m, r = _master()
    r.lastToken = [0]
    seen = []
    r.forward(number=2, stopTokens=[], progressLambda=seen.append)
    assert [s["progress"] for s in seen] == [0, 1] and seen[1]["tokens"] == [1, 2] and seen[1]["total"] == 2
    assert seen[1]["current"] == "2"


def test_load_context_chunks_and_does_not_touch_callers_state():
    m, r = _master()
    mine = torch.full((1,), 10.0, dtype=torch.float64)
    ids, st = r.loadContext(newctx=list(range(1, 8)), ctx=[9, 11], statex=mine, batch=3)
    assert m.calls == [[1, 2, 3], [4, 5, 6], [7]] and ids == list(range(1, 8))
    assert float(mine) == 10.0 and float(st) == 17.0 and float(r.myState) == 17.0
    assert r.lastToken == [11]                       # the reference keeps the last token of ctx, not newctx
    st += 1
    assert float(r.myState) == 17.0


def test_typical_sampler_stays_in_the_typical_set():
    g = torch.Generator().manual_seed(0)
    logits = torch.tensor([0.0, 0.1, 8.0, 0.2, -3.0], dtype=torch.float64)
    assert all(typical(logits, 1.0, 0.5, generator=g) == 2 for _ in range(20))
    flat = torch.zeros(50, dtype=torch.float64)
    draws = {typical(flat, 1.0, 0.8, generator=g) for _ in range(200)}
    assert len(draws) > 10 and all(0 <= d < 50 for d in draws)
    assert typical(logits, 0.5, 0.95, generator=g) in range(5)


def test_token_id_tokenizer_round_trip():
    t = TokenIds()
    assert t.encode("3 4 5") == [3, 4, 5] and t.decode([3, 4, 5]) == "3 4 5" and t.encode([1, 2]) == [1, 2]


def test_rwkv_rejects_unknown_modes_and_files():
    with pytest.raises(ValueError):
        RWKV("model.pth", mode="jax")
    with pytest.raises(ValueError):
        RWKV("model.onnx")
    with pytest.raises((ValueError, FileNotFoundError)):
        RWKV("no_such_model.rwkv")
    with pytest.raises(TypeError):
        RWKV({}, strategy="cuda fp16")


def test_rwkv_reads_the_reference_loader_options():
    """opt.py:15-19, matmul.py:177-199: ``jit`` means nothing here, ``config`` may name the one GPU and ask for
    host-resident codes, everything this backend does not provide is refused before any weight is touched."""
    from rwkvstic_amd.master import _loader_options
    assert _loader_options("cuda", {}) == {"device": "cuda", "stream": False, "export": False}
    assert _loader_options("cuda", {"jit": False, "export": "out"})["export"] == "out"
    one = {"devices": [{"device": "cuda:0", "dtype": torch.uint8, "stream": True}], "custom": True}
    assert _loader_options("cuda", {"config": one}) == {"device": "cuda:0", "stream": True, "export": False}
    assert _loader_options("cuda:0", {"config": one})["device"] == "cuda:0"
    for bad in ({"devices": []},
                {"devices": [{"device": "cuda:0"}, {"device": "cuda:1"}]},          # the reference's split over devices
                {"devices": [{"device": "cpu", "dtype": torch.uint8}]},
                {"devices": [{"device": "cuda", "dtype": torch.float16}]},
                {"devices": [{"device": "cuda", "naive": True}]}):
        with pytest.raises(ValueError):
            _loader_options("cuda", {"config": bad})
    with pytest.raises(ValueError):
        _loader_options("cuda:1", {"config": one})
    with pytest.raises(TypeError):
        _loader_options("cuda", {"export": True})
    with pytest.raises(TypeError):
        _loader_options("cuda", {"strategy": "cuda fp16"})
    with pytest.raises(ValueError):                     # refused before the (missing) file is opened
        RWKV("no_such_model.pth", config={"devices": [{"device": "cpu"}]})


def test_post_contract_and_state_json_round_trip():
    """server.py:56-86: state in and out as nested float lists, "input" loaded as context, the rest passed to forward."""
    import json
    from rwkvstic_amd import serving
    m, r = _master()
    r.emptyState = torch.zeros(2, 3, dtype=torch.float64)
    r.resetState()
    reply = serving.post(r, {"input": "4 5 6", "number": 2, "stopTokens": [], "end_adj": 0.0})
    assert m.calls[0] == [4, 5, 6] and len(m.calls) == 3            # the prompt, then two single-token steps
    assert reply["output"] == "188 189" or len(reply["output"].split()) == 2
    assert isinstance(reply["logits"], list) and len(reply["logits"]) == StubModel.V
    assert isinstance(reply["state"], list) and len(reply["state"]) == 2 and len(reply["state"][0]) == 3
    wire = json.loads(json.dumps(reply))                             # survives the wire format
    # the returned state fed back continues where the first request stopped
    before = len(m.calls)
    reply2 = serving.post(r, {"state": wire["state"], "number": 1, "stopTokens": [], "end_adj": 0.0})
    assert len(m.calls) == before + 1
    assert float(torch.tensor(reply2["state"]).flatten()[0]) == float(torch.tensor(wire["state"]).flatten()[0]) + 1
    # a state of the wrong shape is refused
    import pytest as _pytest
    with _pytest.raises(ValueError):
        serving.post(r, {"state": [[0.0]], "number": 1})
    # float32 on the wire: the empty WKV row's -1e30 survives, finer digits do not
    st = torch.tensor([[-1e30, 1.0 + 2 ** -30, 0.5]], dtype=torch.float64)
    back = serving.state_from_json(serving.state_to_json(st), st)
    assert back.dtype == torch.float64 and float(back[0, 0]) == float(torch.tensor(-1e30, dtype=torch.float32))
    assert float(back[0, 1]) == 1.0 and float(back[0, 2]) == 0.5


def test_http_handler_speaks_the_wire_format():
    import json
    import threading
    import urllib.request
    import socketserver
    from rwkvstic_amd import serving
    m, r = _master()
    with socketserver.TCPServer(("127.0.0.1", 0), serving.make_handler(r)) as httpd:
        port = httpd.server_address[1]
        t = threading.Thread(target=httpd.handle_request)
        t.start()
        req = urllib.request.Request(f"http://127.0.0.1:{port}/", data=json.dumps({"number": 1, "stopTokens": []}).encode(),
                                     headers={"Content-Type": "application/json"})
        reply = json.loads(urllib.request.urlopen(req, timeout=10).read())
        t.join()
    assert set(reply) >= {"logits", "state", "output"}
