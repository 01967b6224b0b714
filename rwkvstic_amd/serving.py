"""The request contract of the reference's HTTP front end (reference src/rwkvstic/server.py:56-86) without the
server around it: ``post(master, body)`` takes the decoded JSON body of a POST and returns the dict the reference
serialises back.

    body:  {"state": nested list | absent, "input": text | absent, ...keyword arguments of forward()}
      - "state" given  -> turned into a tensor (server.py:66-67); absent -> resetState() and the empty state (:68-70)
      - "input" given  -> loadContext(newctx=input, statex=state), its returned state replaces "state" (:72-75)
      - everything left goes to forward(**body) (:78)
    reply: forward()'s dict with "state" as one nested float list per layer and "logits" as a float list, both
           passed through float32 as the reference does (:79-81) - a state that went through JSON is therefore the
           float32 rounding of the one that was sent (the -1e30 of an empty WKV row survives it).

``make_handler(master)`` wraps it into an ``http.server`` request handler for callers that want the wire format
too; nothing here starts a server.
"""
from __future__ import annotations

import json
from typing import Dict

import torch


def state_to_json(state: torch.Tensor):
    """server.py:79-80: one float32 nested list per layer."""
    return [x.cpu().float().numpy().tolist() for x in state]


def state_from_json(obj, like: torch.Tensor) -> torch.Tensor:
    """server.py:66-67 (``initTensor``): the nested list back as a tensor of the model's state dtype, on its device."""
    t = torch.tensor(obj, dtype=torch.float32).to(dtype=like.dtype, device=like.device).contiguous()
    if t.shape != like.shape:
        raise ValueError(f"state of shape {tuple(t.shape)}, the model's is {tuple(like.shape)}")
    return t


def post(master, body: Dict) -> Dict:
    body = dict(body)
    if body.get("state", None) is not None:
        body["state"] = state_from_json(body["state"], master.emptyState)
    else:
        master.resetState()
        body["state"] = master.getState()[0]
    if body.get("input", None) is not None:
        body["state"] = master.loadContext(newctx=body["input"], statex=body.get("state", None))[1]
        del body["input"]
    out = dict(master.forward(**body))
    out["state"] = state_to_json(out["state"])
    out["logits"] = out["logits"].cpu().float().numpy().tolist()
    return out


def make_handler(master):
    import http.server

    class Handler(http.server.BaseHTTPRequestHandler):
        def do_POST(self):                               # server.py:58-86
            n = int(self.headers["Content-Length"])
            reply = json.dumps(post(master, json.loads(self.rfile.read(n))))
            self.send_response(200)
            self.send_header("Content-type", "text/json")
            self.end_headers()
            self.wfile.write(reply.encode("utf-8"))

        def log_message(self, *args):
            pass

    return Handler
