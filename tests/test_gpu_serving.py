"""The request contract of the reference's HTTP front end (server.py:56-86) over the real model: prompt ->
loadContext -> forward on the GPU, the state out and back in as JSON, through ``serving.post`` and once over the wire."""
import json
import threading
import urllib.request
import socketserver

import pytest
import torch

from rwkvstic_amd import synth

pytestmark = pytest.mark.gpu


def _ids(text):
    return [int(t) for t in text.split()]


@pytest.mark.parametrize("C,V", [(1024, 1999), (64, 512)])      # persistent single-token kernel / per-phase kernels
def test_post_over_the_hip_model(C, V):
    from rwkvstic_amd import serving
    from rwkvstic_amd.master import RWKV, greedy
    sd = synth.make_state_dict(2, C, 4 * C, V, seed=41, ln="random")
    r = RWKV(sd, sampler=greedy)
    hip = r.model
    prompt = synth.random_tokens(37, V=V, seed=5).tolist()
    print(f"post: prompt of {len(prompt)} tokens, C={C}", flush=True)
    reply = serving.post(r, {"input": prompt, "number": 6, "stopTokens": [], "end_adj": 0.0})
    # what the request means: empty state, the prompt as context, then six tokens starting from lastToken = [187]
    # (resetState, rwkvMaster.py:23; the prompt's own last token is not fed again, :58-105)
    st = hip.emptyState.clone()
    _, st = hip.forward(prompt, st)
    toks, logits, st = hip.decode_greedy(187, 6, st)
    hip.check()
    assert _ids(reply["output"]) == toks.tolist()
    assert reply["logits"] == logits.cpu().float().numpy().tolist()
    assert len(reply["state"]) == hip.layers and len(reply["state"][0]) == 5 and len(reply["state"][0][0]) == C
    assert torch.equal(torch.tensor(reply["state"], dtype=torch.float32), st.cpu().float())
    # the state survives the wire format and continues the sequence: same as continuing from its float32 rounding
    wire = json.loads(json.dumps(reply))
    reply2 = serving.post(r, {"state": wire["state"], "number": 4, "stopTokens": [], "end_adj": 0.0})
    back = serving.state_from_json(wire["state"], hip.emptyState)
    assert back.dtype == torch.float64 and back.is_cuda
    toks2, logits2, st2 = hip.decode_greedy(int(toks[-1]), 4, back.clone())
    hip.check()
    assert _ids(reply2["output"]) == toks2.tolist()
    assert torch.equal(torch.tensor(reply2["state"], dtype=torch.float32), st2.cpu().float())
    # float32 on the wire costs little: the continuation from the unrounded state gives nearly the same logits
    toks3, logits3, _ = hip.decode_greedy(int(toks[-1]), 4, st.clone())
    assert float((logits3 - logits2).abs().max()) < 1e-3
    # a stop token ends the request early and is part of the output (rwkvMaster.py:49-50)
    reply4 = serving.post(r, {"input": prompt, "number": 6, "stopTokens": [int(toks[2])], "end_adj": 0.0})
    assert _ids(reply4["output"]) == toks.tolist()[:toks.tolist().index(int(toks[2])) + 1]


def test_post_over_http_with_the_typical_sampler():
    """The same contract over a socket, with the default sampler (typical, on the device): the reply is well formed,
    reproducible under torch.manual_seed, and never holds the end token with the default end_adj."""
    from rwkvstic_amd import serving
    from rwkvstic_amd.master import RWKV
    sd = synth.make_state_dict(2, 1024, 4096, 1999, seed=42, ln="random")
    r = RWKV(sd)
    body = json.dumps({"input": "5 6 7 8 9 10 11", "number": 12}).encode()
    outs = []
    for _ in range(2):
        torch.manual_seed(3)
        with socketserver.TCPServer(("127.0.0.1", 0), serving.make_handler(r)) as httpd:
            port = httpd.server_address[1]
            t = threading.Thread(target=httpd.handle_request)
            t.start()
            req = urllib.request.Request(f"http://127.0.0.1:{port}/", data=body, headers={"Content-Type": "application/json"})
            reply = json.loads(urllib.request.urlopen(req, timeout=60).read())
            t.join()
        assert set(reply) >= {"logits", "state", "output"} and len(reply["logits"]) == 1999
        ids = _ids(reply["output"])
        assert len(ids) == 12 and 0 not in ids and all(0 <= i < 1999 for i in ids)
        outs.append(ids)
    assert outs[0] == outs[1]
