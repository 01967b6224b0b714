"""FASTQUANT RWKV-4 model on the HIP backend.

``HipRWKV`` plays the role of the reference's ``myRWKV`` module
(reference src/rwkvstic/agnostic/backends/opt.py:27-84): same constructor
inputs (a BlinkDL ``.pth`` state dict), same ``forward(tokens, state) ->
(logits[V], state[L,5,C])`` contract, same ``emptyState``.  Loading quantises
every matrix on the GPU with the reference scheme (matmul.py:18-40) and repacks
it into the streaming block layout; the forward pass is one C-ABI call.
"""
from __future__ import annotations

import ctypes as C
from typing import Dict, Iterable, List, Optional, Tuple, Union

import torch

from . import _native as N
from . import ops


class QuantMatrix:
    """Device-resident quantised matrix: packed codes + per-input-channel range/offset."""

    def __init__(self, packed: torch.Tensor, rng: torch.Tensor, off: torch.Tensor, n_in: int, n_out: int,
                 packed16: Optional[torch.Tensor] = None):
        self.packed, self.range, self.offset, self.n_in, self.n_out = packed, rng, off, n_in, n_out
        self.packed16 = packed16

    @classmethod
    def from_weight(cls, weight: torch.Tensor, device, m16: bool = True, stream: bool = False) -> "QuantMatrix":
        """``weight[out, in]`` in any float dtype, on any device."""
        w = weight.to(device=device, dtype=torch.float32).contiguous()
        codes, rng, off = ops.quantize(w)
        n_in, n_out = codes.shape
        return cls(ops.pack(codes), rng, off, n_in, n_out, ops.pack_m16(codes) if m16 else None)._placed(stream)

    @classmethod
    def from_codes(cls, codes: torch.Tensor, rng: torch.Tensor, off: torch.Tensor, device, stream: bool = False) -> "QuantMatrix":
        """From the reference/.rwkv layout: ``codes[in, out]`` uint8, ``range[in]``, ``offset[in]``."""
        codes = codes.to(device)
        n_in, n_out = codes.shape
        return cls(ops.pack(codes), rng.to(device=device, dtype=torch.float32).contiguous(),
                   off.to(device=device, dtype=torch.float64).contiguous(), n_in, n_out, ops.pack_m16(codes))._placed(stream)

    def _placed(self, stream: bool) -> "QuantMatrix":
        """``stream=True`` (the reference's per-device ``stream`` option, matmul.py:21,186: codes stay in host
        memory, range and offset on the device): the packed codes move to pinned host memory, which the GPU
        reads in place over the host link while the kernels run; nothing else changes."""
        if stream:
            def pinned(t):
                h = torch.empty(t.shape, dtype=t.dtype, pin_memory=True)
                h.copy_(t)
                return h
            self.packed = pinned(self.packed)
            if self.packed16 is not None:
                self.packed16 = pinned(self.packed16)
        self.stream = stream
        return self

    def codes(self) -> torch.Tensor:
        packed = self.packed.to(self.range.device) if not self.packed.is_cuda else self.packed
        return ops.unpack(packed, self.n_in, self.n_out)

    def desc(self) -> N.QMat:
        return N.QMat(self.packed.data_ptr(), self.packed16.data_ptr() if self.packed16 is not None else None,
                      self.range.data_ptr(), self.offset.data_ptr(), self.n_in, self.n_out)

    def nbytes(self) -> int:
        return self.n_in * self.n_out


class HipRWKV:
    def __init__(self, weights: Union[Dict[str, torch.Tensor], Iterable[Tuple[str, torch.Tensor]]],
                 device: str = "cuda", fused: bool = True, stream: bool = False):
        """``fused=False`` skips the second weight layout, so single-token steps run as one launch per
        phase (the path every shape supports) instead of the persistent kernel.  ``stream=True`` keeps the
        quantised codes of every matrix in pinned host memory (models larger than the GPU's memory; the
        reference's ``stream`` option, matmul.py:21,186) - the same kernels then read them over the host link."""
        if not torch.cuda.is_available():
            raise RuntimeError("HipRWKV needs a ROCm GPU (gfx950); there is no CPU path in this backend")
        N.lib()
        self.device = torch.device(device)
        f64 = dict(device=self.device, dtype=torch.float64)
        items = weights.items() if isinstance(weights, dict) else weights
        vec: Dict[str, torch.Tensor] = {}
        mats: Dict[str, QuantMatrix] = {}
        self.emb: Optional[torch.Tensor] = None
        for key, t in items:
            if key == "emb.weight":
                self.emb = t.to(device=self.device, dtype=torch.float32).contiguous()
            elif key.endswith(".weight") and t.dim() == 2:
                mats[key] = QuantMatrix.from_weight(t, self.device, m16=fused, stream=stream)
            else:
                vec[key] = t
        if self.emb is None:
            raise KeyError("emb.weight")
        # opt.py:96-98
        layers = len([k for k in vec if "blocks" in k and "ln1.bias" in k])

        def v64(key):
            return vec[key].reshape(-1).to(**f64).contiguous()

        blocks: List[dict] = []
        for i in range(layers):
            p = f"blocks.{i}."
            blocks.append(dict(
                ln1_w=v64(p + "ln1.weight"), ln1_b=v64(p + "ln1.bias"),
                ln2_w=v64(p + "ln2.weight"), ln2_b=v64(p + "ln2.bias"),
                # block.py:35-47
                att_mix=torch.stack([v64(p + "att.time_mix_k"), v64(p + "att.time_mix_v"),
                                     v64(p + "att.time_mix_r")]).contiguous(),
                ffn_mix=torch.stack([v64(p + "ffn.time_mix_k"), v64(p + "ffn.time_mix_r")]).contiguous(),
                time_first=v64(p + "att.time_first"),
                time_decay=v64(p + "att.time_decay").exp().neg().contiguous(),
                att_k=mats[p + "att.key.weight"], att_v=mats[p + "att.value.weight"],
                att_r=mats[p + "att.receptance.weight"], att_o=mats[p + "att.output.weight"],
                ffn_k=mats[p + "ffn.key.weight"], ffn_r=mats[p + "ffn.receptance.weight"],
                ffn_v=mats[p + "ffn.value.weight"],
            ))
        self._finish_init((v64("blocks.0.ln0.weight"), v64("blocks.0.ln0.bias")),
                          (v64("ln_out.weight"), v64("ln_out.bias")), mats["head.weight"], blocks)

    def _finish_init(self, ln0, ln_out, head: QuantMatrix, blocks: List[dict]) -> None:
        self.ln0, self.ln_out, self.head, self.blocks = ln0, ln_out, head, blocks
        self.layers = len(blocks)
        self.dims = blocks[0]["att_k"].n_out
        self.ffn = blocks[0]["ffn_k"].n_out
        self.vocab = self.emb.shape[0]
        self._keep: List[torch.Tensor] = []
        # opt.py:31-32,80
        es = torch.zeros((self.layers, 5, self.dims), device=self.device, dtype=torch.float64)
        es[:, 4] = -1e30
        self.emptyState = es
        self._build_handle()

    # ------------------------------------------------------------------
    # The quantised model as the reference keeps it (and exports it in a .rwkv archive, opt.py:89-92,112-117):
    # a tree of module attributes.  Names: matmul.py:12,67-68,175,254 (weights.0.{weight,range,offset}[1,2]),
    # block.py:13-47 (ln1, ln2, att, ffnkey, ffnvalue, attout, ffnreceptance, attmix, ffnmix, time_first,
    # time_decay), opt.py:31-48 (emptyState, emb.w, ln_in, ln_out, head).  Codes are uint8 [in, out], range
    # float32 [in], offset float64 [in]; time_decay is stored as -exp(raw) (block.py:41).
    _MAT_ATTRS = (("att_k", "att.weights.0.", ""), ("att_v", "att.weights.0.", "1"), ("att_r", "att.weights.0.", "2"),
                  ("att_o", "attout.weights.0.", ""), ("ffn_k", "ffnkey.weights.0.", ""),
                  ("ffn_r", "ffnreceptance.weights.0.", ""), ("ffn_v", "ffnvalue.weights.0.", ""))

    def quantized_tree(self) -> Dict[str, torch.Tensor]:
        """Flat ``{attribute path: tensor}`` (on the CPU) of the quantised model under the reference's names."""
        out: Dict[str, torch.Tensor] = {}

        def put_mat(prefix: str, suffix: str, m: QuantMatrix) -> None:
            out[f"{prefix}weight{suffix}"] = m.codes().cpu()
            out[f"{prefix}range{suffix}"] = m.range.cpu()
            out[f"{prefix}offset{suffix}"] = m.offset.cpu()

        out["emptyState"] = self.emptyState.cpu()
        out["emb.w"] = self.emb.cpu()
        out["ln_in.weight"], out["ln_in.bias"] = self.ln0[0].cpu(), self.ln0[1].cpu()
        out["ln_out.weight"], out["ln_out.bias"] = self.ln_out[0].cpu(), self.ln_out[1].cpu()
        put_mat("head.weights.0.", "", self.head)
        for i, b in enumerate(self.blocks):
            p = f"blocks.{i}."
            for name in ("ln1", "ln2"):
                out[p + name + ".weight"], out[p + name + ".bias"] = b[name + "_w"].cpu(), b[name + "_b"].cpu()
            for key, prefix, suffix in self._MAT_ATTRS:
                put_mat(p + prefix, suffix, b[key])
            out[p + "attmix"] = b["att_mix"].cpu().unsqueeze(1)        # [3, 1, C] (block.py:35-36)
            out[p + "ffnmix"] = b["ffn_mix"].cpu().unsqueeze(1)        # [2, 1, C]
            out[p + "time_first"] = b["time_first"].cpu()
            out[p + "time_decay"] = b["time_decay"].cpu()
        return out

    @classmethod
    def from_quantized(cls, tree: Dict[str, torch.Tensor], device: str = "cuda", stream: bool = False) -> "HipRWKV":
        """From ``quantized_tree()`` (or the same attributes taken from a reference model): nothing is
        quantised again, the codes are only repacked into the streaming layouts (``stream``: kept in pinned host
        memory, as in the constructor)."""
        if not torch.cuda.is_available():
            raise RuntimeError("HipRWKV needs a ROCm GPU (gfx950); there is no CPU path in this backend")
        N.lib()
        self = cls.__new__(cls)
        self.device = torch.device(device)
        f64 = dict(device=self.device, dtype=torch.float64)

        def v64(key):
            return tree[key].reshape(-1).to(**f64).contiguous()

        def mat(prefix: str, suffix: str = "") -> QuantMatrix:
            codes = tree[f"{prefix}weight{suffix}"]
            if codes.dtype != torch.uint8 or codes.dim() != 2:
                raise ValueError(f"{prefix}weight{suffix}: expected uint8 codes [in, out]")
            return QuantMatrix.from_codes(codes.contiguous(), tree[f"{prefix}range{suffix}"].reshape(-1),
                                          tree[f"{prefix}offset{suffix}"].reshape(-1), self.device, stream=stream)

        self.emb = tree["emb.w"].to(device=self.device, dtype=torch.float32).contiguous()
        layers = len([k for k in tree if k.startswith("blocks.") and k.endswith(".ln1.bias")])
        blocks: List[dict] = []
        for i in range(layers):
            p = f"blocks.{i}."
            blk = dict(ln1_w=v64(p + "ln1.weight"), ln1_b=v64(p + "ln1.bias"),
                       ln2_w=v64(p + "ln2.weight"), ln2_b=v64(p + "ln2.bias"),
                       att_mix=tree[p + "attmix"].reshape(3, -1).to(**f64).contiguous(),
                       ffn_mix=tree[p + "ffnmix"].reshape(2, -1).to(**f64).contiguous(),
                       time_first=v64(p + "time_first"), time_decay=v64(p + "time_decay"))
            for key, prefix, suffix in cls._MAT_ATTRS:
                blk[key] = mat(p + prefix, suffix)
            blocks.append(blk)
        self._finish_init((v64("ln_in.weight"), v64("ln_in.bias")), (v64("ln_out.weight"), v64("ln_out.bias")),
                          mat("head.weights.0."), blocks)
        return self

    def save_quantized(self, path: str) -> None:
        """``torch.save`` of ``quantized_tree()``: plain tensors, loadable with ``weights_only=True``."""
        torch.save(self.quantized_tree(), path)

    # ------------------------------------------------------------------
    def _build_handle(self) -> None:
        L = N.lib()
        self._layer_arr = (N.LayerDesc * self.layers)()
        for i, b in enumerate(self.blocks):
            d = self._layer_arr[i]
            for name in ("ln1_w", "ln1_b", "ln2_w", "ln2_b", "att_mix", "ffn_mix", "time_decay", "time_first"):
                setattr(d, name, b[name].data_ptr())
            for name in ("att_k", "att_v", "att_r", "att_o", "ffn_k", "ffn_r", "ffn_v"):
                setattr(d, name, b[name].desc())
        desc = N.ModelDesc(self.layers, self.dims, self.ffn, self.vocab, self.emb.data_ptr(),
                           self.ln0[0].data_ptr(), self.ln0[1].data_ptr(),
                           self.ln_out[0].data_ptr(), self.ln_out[1].data_ptr(),
                           self.head.desc(), self._layer_arr)
        handle = C.c_void_p()
        with torch.cuda.device(self.device):
            N.check(L.rwkv_model_create(C.byref(desc), C.byref(handle)))
        self._handle = handle
        self.fused_step = bool(L.rwkv_model_has_fused_step(handle))
        self._ws: Optional[torch.Tensor] = None
        self._ws_tokens = 0
        self._bws: Optional[torch.Tensor] = None

    def __del__(self):
        h = getattr(self, "_handle", None)
        if h:
            try:
                N.lib().rwkv_model_destroy(h)
            except Exception:
                pass
            self._handle = None

    def _workspace(self, T: int) -> torch.Tensor:
        if self._ws is None or T > self._ws_tokens:
            nbytes = N.lib().rwkv_model_workspace_bytes(self._handle, T)
            self._ws = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
            self._ws_tokens = T
        return self._ws

    def check(self) -> None:
        """Synchronise and raise if a single-token launch gave up waiting (diagnostics)."""
        N.check(N.lib().rwkv_model_check(self._handle))

    def selftest_timeout(self, state: torch.Tensor) -> None:
        """Launch one token step whose input never arrives and whose waits give up after a few hundred polls: the
        launch ends normally, ``state`` is untouched, and the next ``check()`` raises (self-test of the failure path)."""
        self._check_state(state)
        logits = torch.empty(self.vocab, dtype=torch.float64, device=self.device)
        with torch.cuda.device(self.device):
            N.check(N.lib().rwkv_model_selftest_timeout(self._handle, torch.cuda.current_stream().cuda_stream,
                                                        state.data_ptr(), logits.data_ptr()))

    def time_token_kernel(self, token: int, n: int, state: torch.Tensor) -> float:
        """Feed ``token`` ``n`` times (``state`` advances) and return the persistent kernel's own average duration
        in microseconds, from events recorded on the stream around each of its launches (measurement aid)."""
        import ctypes
        self._check_state(state)
        tok = torch.tensor([int(token)], dtype=torch.int64, device=self.device)
        logits = torch.empty(self.vocab, dtype=torch.float64, device=self.device)
        us = ctypes.c_float(0.0)
        with torch.cuda.device(self.device):
            N.check(N.lib().rwkv_model_time_token_kernel(self._handle, torch.cuda.current_stream().cuda_stream, tok.data_ptr(),
                                                         state.data_ptr(), logits.data_ptr(), int(n), ctypes.byref(us)))
        return float(us.value)

    def weight_bytes(self) -> int:
        """uint8 weight bytes streamed per decoded token: L*13*C^2 + V*C."""
        n = self.head.nbytes()
        for b in self.blocks:
            n += sum(b[k].nbytes() for k in ("att_k", "att_v", "att_r", "att_o", "ffn_k", "ffn_r", "ffn_v"))
        return n

    # ------------------------------------------------------------------
    def _check_state(self, state: torch.Tensor) -> None:
        if (not isinstance(state, torch.Tensor) or state.device.type != "cuda" or state.dtype != torch.float64
                or tuple(state.shape) != (self.layers, 5, self.dims) or not state.is_contiguous()):
            raise ValueError(f"state must be a contiguous CUDA float64 tensor of shape "
                             f"({self.layers}, 5, {self.dims})")

    def _tokens(self, tokens) -> torch.Tensor:
        """Token ids as an int64 vector on the device.  Ids that arrive on the host are range-checked there, as the
        reference's host-side table lookup does (emb.py:9 raises IndexError); ids already on the device are not read
        back: the kernels clamp them to the table."""
        tok = torch.as_tensor(tokens, dtype=torch.int64).reshape(-1)
        if tok.device.type == "cpu" and tok.numel() and (int(tok.min()) < 0 or int(tok.max()) >= self.vocab):
            raise IndexError(f"token id out of range for a vocabulary of {self.vocab}")
        return tok.to(self.device)

    def forward(self, tokens, state: torch.Tensor):
        """``(logits[V] float64, state)``; ``state`` is updated in place and returned (opt.py:61-76)."""
        tok = self._tokens(tokens)
        if tok.numel() == 0:
            raise ValueError("forward needs at least one token")
        self._check_state(state)
        T = tok.numel()
        ws = self._workspace(T)
        logits = torch.empty(self.vocab, dtype=torch.float64, device=self.device)
        with torch.cuda.device(self.device):
            N.check(N.lib().rwkv_model_forward(self._handle, torch.cuda.current_stream().cuda_stream,
                                               tok.data_ptr(), T, state.data_ptr(), logits.data_ptr(),
                                               ws.data_ptr(), ws.numel()))
        return logits, state

    __call__ = forward

    def forward_batch(self, tokens, states: torch.Tensor):
        """One token for each of B independent sequences: ``tokens[B]``, ``states[B, L, 5, C]`` float64
        (updated in place) -> ``(logits[B, V] float64, states)``."""
        tok = self._tokens(tokens)
        B = tok.numel()
        if (not isinstance(states, torch.Tensor) or states.device.type != "cuda" or states.dtype != torch.float64
                or tuple(states.shape) != (B, self.layers, 5, self.dims) or not states.is_contiguous()):
            raise ValueError(f"states must be a contiguous CUDA float64 tensor of shape "
                             f"({B}, {self.layers}, 5, {self.dims})")
        L = N.lib()
        nbytes = L.rwkv_model_batch_workspace_bytes(self._handle, B)
        if nbytes == 0:
            raise RuntimeError("forward_batch needs the model built with fused=True and n_embd, n_ffn multiples of 64")
        if self._bws is None or self._bws.numel() < nbytes:
            self._bws = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
        logits = torch.empty((B, self.vocab), dtype=torch.float64, device=self.device)
        with torch.cuda.device(self.device):
            N.check(L.rwkv_model_forward_batch(self._handle, torch.cuda.current_stream().cuda_stream,
                                               tok.data_ptr(), B, states.data_ptr(), logits.data_ptr(),
                                               self._bws.data_ptr(), self._bws.numel()))
        return logits, states

    def decode_greedy(self, token: int, n: int, state: torch.Tensor):
        """Feed ``token`` then greedily generate: returns ``(tokens[n] int64 on device, last logits, state)``
        where ``tokens[i] = argmax(forward(previous token))``.  No host round trip per token."""
        self._check_state(state)
        if not 0 <= int(token) < self.vocab:
            raise IndexError(f"token id out of range for a vocabulary of {self.vocab}")
        toks = torch.empty(n + 1, dtype=torch.int64, device=self.device)
        toks[0] = int(token)
        ws = self._workspace(1)
        logits = torch.empty(self.vocab, dtype=torch.float64, device=self.device)
        with torch.cuda.device(self.device):
            N.check(N.lib().rwkv_model_decode_greedy(self._handle, torch.cuda.current_stream().cuda_stream,
                                                     toks.data_ptr(), n, state.data_ptr(), logits.data_ptr(),
                                                     ws.data_ptr(), ws.numel()))
        return toks[1:], logits, state


    def decode_sample(self, token: int, n: int, state: torch.Tensor, *, greedy: bool = False, temp: float = 1.0,
                      tau: float = 0.8, end_adj: float = 0.0, seed: int = 0, stop_tokens=()):
        """``RWKVMaster.forward(number=n)`` (rwkvMaster.py:28-56) without a host round trip per token: feed
        ``token``, then ``n`` times choose the next token on the device (locally typical sampling,
        agnostic/samplers/typical.py:1-17, or argmax), with ``end_adj`` added to logit 0 before every choice
        and the loop ending at the first chosen stop token (which is part of the output).  Returns
        ``(tokens int64 on the device, logits, state)``; ``state`` and ``logits`` are those of the last step
        that ran.  Needs the persistent single-token kernel (``fused_step``)."""
        self._check_state(state)
        if not self.fused_step:
            raise RuntimeError("decode_sample needs the persistent single-token kernel (fused_step)")
        if not 0 <= int(token) < self.vocab:
            raise IndexError(f"token id out of range for a vocabulary of {self.vocab}")
        toks = torch.empty(n + 1, dtype=torch.int64, device=self.device)
        toks[0] = int(token)
        stops = torch.as_tensor(list(stop_tokens), dtype=torch.int64, device=self.device)
        flag = torch.zeros(1, dtype=torch.int32, device=self.device)
        done = torch.zeros(1, dtype=torch.int64, device=self.device)
        ws = self._workspace(1)
        logits = torch.empty(self.vocab, dtype=torch.float64, device=self.device)
        with torch.cuda.device(self.device):
            N.check(N.lib().rwkv_model_decode_sample(
                self._handle, torch.cuda.current_stream().cuda_stream, toks.data_ptr(), n, state.data_ptr(),
                logits.data_ptr(), ws.data_ptr(), ws.numel(), 1 if greedy else 0, float(temp), float(tau), float(end_adj),
                int(seed) & (2 ** 64 - 1), stops.data_ptr() if stops.numel() else None, int(stops.numel()),
                flag.data_ptr(), done.data_ptr()))
        return toks[1:1 + int(done)], logits, state


def wkv_state_to_reference(state: torch.Tensor) -> torch.Tensor:
    """Rows 2-4 hold the max-shifted triple ``(aa', bb', pp')``; the reference's naive kernel keeps
    ``aa = aa' e^{pp'}``, ``bb = bb' e^{pp'}`` and never touches ``pp`` (cuda/operators.cu:21-36).
    Returns a copy in the reference convention (pp reset to -1e30)."""
    out = state.clone()
    e = torch.exp(state[:, 4])
    out[:, 2] = state[:, 2] * e
    out[:, 3] = state[:, 3] * e
    out[:, 4] = -1e30
    return out


def wkv_state_from_reference(state: torch.Tensor) -> torch.Tensor:
    """Inverse of :func:`wkv_state_to_reference`: a naive ``(aa, bb)`` is the shifted triple with ``pp' = 0``
    (or the empty state where ``bb == 0``)."""
    out = state.clone()
    empty = ~(state[:, 3] > 0)
    out[:, 4] = torch.where(empty, torch.full_like(state[:, 4], -1e30), torch.zeros_like(state[:, 4]))
    return out
