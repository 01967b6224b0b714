"""User-facing shell with the reference's surface: ``RWKV(path, ...)`` returns an object that behaves like
``RWKVMaster`` (reference src/rwkvstic/rwkvMaster.py:14-125) over the HIP FASTQUANT model
(reference load.py:18,42-47 picks ``OptRWKV`` + the ``typical`` sampler for this mode).

Kept from the reference, because callers rely on it: ``forward`` adds ``end_adj`` to logit 0 before
sampling and stops on ``stopTokens`` / ``stopStrings``; ``lastToken`` starts at ``[187]``; ``loadContext``
sets ``lastToken`` to the last token of ``ctx`` (not of ``newctx``) and leaves the caller's state untouched;
``getState``/``setState`` exchange ``(state, lastToken)`` pairs.  Changed: prompts are fed in chunks of 1024
tokens (the reference's default is 20) because they run as GEMMs here, and with the built-in samplers, no
per-token callback and no stop strings that could match, ``forward(number=n)`` runs as one device-side loop
(token kernel, sampler, stop-token test, next embedding) instead of n host round trips.
"""
from __future__ import annotations

from typing import Callable, Dict, Iterable, List, Optional, Sequence, Union

import torch

MODE = "hip-fastquant"
DEVICE_SAMPLER_MAX_VOCAB = 53248        # rwkv_sample_token: 1024 threads x 52 values in registers


def _clone(x):
    return x.clone() if hasattr(x, "clone") else x


def typical(logits: torch.Tensor, temp: float = 1.0, tau: float = 0.95, generator=None, **_unused) -> int:
    """Locally typical sampling (reference agnostic/samplers/typical.py:1-17): keep the tokens whose surprise
    is closest to the entropy until their mass reaches ``tau``, then sample; float32, on the logits' device."""
    probs = torch.softmax(logits.float(), dim=-1)
    surprise = -torch.log(probs)
    ent = torch.nansum(surprise * probs, dim=-1, keepdim=True)
    dist = (surprise - ent).abs()
    order = torch.argsort(dist)
    cum = torch.cumsum(probs[order], dim=-1)
    cutoff = int((cum < tau).sum())
    cutoff = min(cutoff, order.numel() - 1)
    probs = torch.where(dist > dist[order[cutoff]], torch.zeros_like(probs), probs)
    if temp != 1.0:
        probs = probs ** (1.0 / temp)
    return int(torch.multinomial(probs, num_samples=1, generator=generator)[0])


def greedy(logits: torch.Tensor, *_args, **_kw) -> int:
    return int(torch.argmax(logits))


class TokenIds:
    """Stand-in tokenizer for callers that work in token ids: ``encode`` accepts a sequence of ints (or a
    string of whitespace-separated ints), ``decode`` joins ids with spaces."""

    def encode(self, x) -> List[int]:
        if isinstance(x, str):
            return [int(t) for t in x.split()]
        return [int(t) for t in x]

    def decode(self, ids: Iterable[int]) -> str:
        return " ".join(str(int(i)) for i in ids)


def load_tokenizer(spec):
    """``None`` -> :class:`TokenIds`; a path -> a ``tokenizers`` JSON file (the reference ships the GPT-NeoX 20B
    vocabulary, tokenizer/__init__.py:3-8); anything with ``encode``/``decode`` is used as is."""
    if spec is None:
        return TokenIds()
    if isinstance(spec, str):
        from tokenizers import Tokenizer
        tk = Tokenizer.from_file(spec)

        class _Wrap:
            def encode(self, s):
                return tk.encode(s).ids

            def decode(self, ids):
                return tk.decode([int(i) for i in ids])
        return _Wrap()
    return spec


def _no_progress(x):
    return x


class RWKVMaster:
    logging = False

    def __init__(self, model, emptyState, sampler: Optional[Callable] = typical, tokenizer=None):
        self.model = model
        self.tokenizer = load_tokenizer(tokenizer)
        self.emptyState = _clone(emptyState)
        self.myState = _clone(emptyState)
        self.lastToken = [187]                   # rwkvMaster.py:23
        self.sampler = sampler

    # ------------------------------------------------------------------ generation (rwkvMaster.py:28-56)
    def _device_loop(self, number, stopStrings, progressLambda, kwargs) -> bool:
        """Whether the whole generation loop can run on the device (``HipRWKV.decode_sample``): the built-in
        samplers, no per-token callback, and stop strings that cannot occur (no stop strings, or a tokenizer
        that only ever yields token ids)."""
        m = self.model
        if not (callable(getattr(m, "decode_sample", None)) and getattr(m, "fused_step", False)):
            return False
        if self.sampler not in (typical, greedy) or progressLambda is not _no_progress or number < 1:
            return False
        if len(self.lastToken) != 1 or set(kwargs) - {"temp", "top_p_usual"}:
            return False
        if getattr(m, "vocab", 0) > DEVICE_SAMPLER_MAX_VOCAB:
            return False                         # the device sampler keeps the whole distribution in one workgroup
        if not stopStrings:
            return True
        # decoded ids are digits and spaces: a stop string of only those (or an empty one) can end the text
        # (rwkvMaster.py:53), every other one never can
        return isinstance(self.tokenizer, TokenIds) and all(s.strip("0123456789 ") != "" for s in stopStrings)

    def forward(self, state=None, number: int = 1, stopStrings: Sequence[str] = ("<|endoftext|>",),
                stopTokens: Sequence[int] = (0,), progressLambda: Callable[[Dict], None] = _no_progress,
                end_adj: float = -990.0, **kwargs):
        ostate = self.myState if state is None else state
        if self._device_loop(number, stopStrings, progressLambda, kwargs):
            # one call: token kernel, sampler, stop test and the next embedding all stay on the GPU
            # the seed of a call comes from torch's global generator: reproducible under torch.manual_seed, and two
            # masters in one process do not repeat each other's draws
            seed = int(torch.randint(0, 2 ** 62, (1,)))
            toks, logits, ostate = self.model.decode_sample(
                self.lastToken[0], number, ostate, greedy=self.sampler is greedy, temp=kwargs.get("temp", 1.0),
                tau=kwargs.get("top_p_usual", 0.8), end_adj=end_adj,
                seed=seed, stop_tokens=list(stopTokens))
            tokens = [int(t) for t in toks.tolist()]
            self.myState = ostate
            self.lastToken = [tokens[-1]]
            self._raise_if_aborted()
            return {"logits": logits, "state": ostate, "output": self.tokenizer.decode(tokens)}
        tokens: List[int] = []
        logits, text = None, ""
        for i in range(number):
            logits, ostate = self.model.forward(self.lastToken, ostate)
            logits[0] += end_adj
            self.myState = ostate
            sampled = self.sample(logits, **kwargs) if self.sampler is not None else int(torch.argmax(logits))
            self.lastToken = [int(sampled)]
            tokens.append(self.lastToken[0])
            text = self.tokenizer.decode(tokens)
            progressLambda({"logits": logits, "state": ostate, "output": text, "progress": i, "tokens": tokens,
                            "total": number, "current": self.tokenizer.decode([tokens[-1]])})
            if tokens[-1] in stopTokens:
                break
            if stopStrings and text.endswith(tuple(stopStrings)):
                break
        self._raise_if_aborted()
        return {"logits": logits, "state": ostate, "output": text}

    def _raise_if_aborted(self):
        """A model whose token kernel can give up waiting (bounded waits) reports it here, once the results
        have been pulled to the host anyway: nothing computed since the last check is valid then."""
        check = getattr(self.model, "check", None)
        if callable(check):
            check()

    # ------------------------------------------------------------------ prompt (rwkvMaster.py:58-105)
    def loadContext(self, newctx="", ctx="\n\n", statex=None, progressCallBack: Callable = lambda x: x,
                    batch: int = 1024):
        state = _clone(self.myState if statex is None else statex)
        ctx_ids = self.tokenizer.encode(ctx)
        new_ids = list(self.tokenizer.encode(newctx))
        if ctx_ids:
            self.lastToken = [int(ctx_ids[-1])]
        for i in range(0, len(new_ids), max(1, batch)):
            chunk = new_ids[i:i + max(1, batch)]
            _, state = self.model.forward(chunk, state)
            progressCallBack(chunk)
        self._raise_if_aborted()
        self.myState = _clone(state)
        return new_ids, _clone(state)

    # ------------------------------------------------------------------ small API (rwkvMaster.py:107-125)
    def sample(self, logits, temp: float = 1.0, top_p_usual: float = 0.8, **kw) -> int:
        return self.sampler(logits, temp, top_p_usual, **kw)

    def decode(self, x):
        return self.tokenizer.decode(x)

    def encode(self, x):
        return self.tokenizer.encode(x)

    def setState(self, state):
        self.myState = _clone(state[0])
        self.lastToken = state[1]

    def getState(self):
        return _clone(self.myState), self.lastToken

    def resetState(self):
        self.myState = _clone(self.emptyState)
        self.lastToken = [187]


def _loader_options(device: str, kwargs: Dict) -> Dict:
    """The options ``OptRWKV`` reads (opt.py:15-19, matmul.py:177-199) turned into this backend's: ``jit`` means
    nothing here (there is no script compiler in the path); ``config["devices"]`` must name one GPU holding uint8
    weights - the reference's split over several devices, its CPU / MPS fallbacks and its unquantised dtypes are not
    part of this backend - and its ``stream`` entry keeps the codes in pinned host memory (matmul.py:21,186);
    ``config["custom"]`` (which WKV operator, wkv.py:56-60) has one answer here.  ``export`` is returned for the
    caller to act on.  Anything else raises: ``strategy`` would select another loader in the reference (load.py:48)."""
    opts = dict(kwargs)
    opts.pop("jit", None)
    out = {"device": device, "stream": False, "export": opts.pop("export", False)}
    config = opts.pop("config", None)
    if opts:
        raise TypeError(f"unsupported options for mode {MODE!r}: {sorted(opts)}")
    if config is not None:
        devices = config.get("devices") if isinstance(config, dict) else None
        if not isinstance(devices, (list, tuple)) or len(devices) != 1 or not isinstance(devices[0], dict):
            raise ValueError("config['devices'] must hold exactly one device entry: this backend runs on one GPU")
        entry = devices[0]
        name = str(entry.get("device", "cuda"))
        if not name.startswith("cuda"):
            raise ValueError(f"device {name!r}: this backend has no CPU / MPS path")
        if entry.get("dtype", torch.uint8) != torch.uint8 or entry.get("naive", False):
            raise ValueError("this backend holds uint8 (fp32i8) weights and runs its own kernels only")
        if device in ("cuda", name):
            out["device"] = name
        else:
            raise ValueError(f"device={device!r} and config['devices'][0]['device']={name!r} disagree")
        out["stream"] = bool(entry.get("stream", False))
    if out["export"] is not False and not isinstance(out["export"], str):
        raise TypeError("export must be a file name stem (opt.py:112-113)")
    return out


def RWKV(path: Union[str, Dict[str, torch.Tensor]], mode: str = MODE, *, tokenizer=None, device: str = "cuda",
         sampler: Optional[Callable] = typical, **kwargs) -> RWKVMaster:
    """``path``: a BlinkDL ``.pth`` checkpoint, a file written by ``HipRWKV.save_quantized`` (the quantised
    attribute tree of the reference's .rwkv export as plain tensors; by convention ``.rwkvq``), both loaded with
    ``weights_only=True``; a TorchScript ``.rwkv`` archive (opt.py:89-92), of which only the tensors are read, by
    attribute path, without compiling or running the code stored in it (``rwkvstic_amd.archive``); or an already
    loaded dict of either kind.  Only the FASTQUANT mode exists in this backend (load.py:42-47); other modes raise.
    Of ``OptRWKV``'s options (opt.py:15-19) ``jit`` is accepted and means nothing, ``config`` may name the one GPU and
    ask for host-resident weights (``{"devices": [{"device": "cuda:0", "dtype": torch.uint8, "stream": True}]}``),
    and ``export="stem"`` writes the quantised model to ``stem.rwkvq`` and then ends the program, as the reference
    does after writing ``stem.rwkv`` (opt.py:112-116)."""
    if mode != MODE:
        raise ValueError(f"mode {mode!r} is not provided by this backend (only {MODE!r})")
    opts = _loader_options(device, kwargs)
    device = opts["device"]
    from .model import HipRWKV
    if isinstance(path, str):
        if path.endswith(".rwkv"):
            from .archive import read_archive_tensors
            weights = read_archive_tensors(path)
            if "emb.w" not in weights or "head.weights.0.weight" not in weights:
                raise ValueError(f"{path}: no FASTQUANT attribute tree (emb.w, head.weights.0.weight, ...) in the archive")
        elif path.endswith(".pth") or path.endswith(".rwkvq"):
            weights = torch.load(path, map_location="cpu", weights_only=True)
        else:
            raise ValueError("only .pth checkpoints, .rwkvq quantised trees and .rwkv archives are supported")
    else:
        weights = path
    if "emb.w" in weights:
        model = HipRWKV.from_quantized(weights, device=device, stream=opts["stream"])
    else:
        model = HipRWKV(weights, device=device, stream=opts["stream"])
    if opts["export"] is not False:
        model.save_quantized(opts["export"] + ".rwkvq")
        raise SystemExit(0)                      # opt.py:115
    return RWKVMaster(model, model.emptyState.clone(), sampler, tokenizer)
