"""Seeded random-init RWKV-4 checkpoints in the BlinkDL ``.pth`` key layout.

There are no pretrained weights offline, so every test and benchmark runs on
models drawn here: matrices and embedding ~N(0, 0.02), ``time_decay`` ~U(-5, 1),
``time_first`` ~U(-1, 1), every ``time_mix_*`` ~U(0, 1); LayerNorm gamma=1 beta=0 with
``ln="identity"`` (the benchmark configurations), or gamma ~U(0.5, 1.5), beta ~N(0, 0.1)
drawn separately for every LayerNorm with ``ln="random"`` (what a trained checkpoint looks like
to the kernels: every weight and bias path carries a non-trivial value).
The key names and shapes are the ones ``OptRWKV`` reads
(reference src/rwkvstic/agnostic/backends/opt.py:34-48, modules/block.py:13-47).
"""
from __future__ import annotations

from typing import Dict, Iterator, Tuple

import torch

SHAPES = {
    # name: (layers, C, F, V)
    "169M": (12, 768, 3072, 50277),
    "3B": (32, 2560, 10240, 50277),
    "14B": (40, 5120, 20480, 50277),
}


def iter_tensors(layers: int, C: int, F: int, V: int, seed: int = 0,
                 device: str = "cpu", ln: str = "identity") -> Iterator[Tuple[str, torch.Tensor]]:
    """Yield ``(key, tensor)`` pairs one at a time (large shapes never need the
    whole float32 checkpoint resident)."""
    if ln not in ("identity", "random"):
        raise ValueError("ln must be 'identity' or 'random'")
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    # LayerNorm parameters come from a generator of their own, so that the matrices of a seed are the same
    # in both modes
    gl = torch.Generator(device=device)
    gl.manual_seed(seed + 104729)

    def normal(*shape):
        return torch.randn(*shape, generator=g, device=device, dtype=torch.float32) * 0.02

    def uniform(lo, hi, *shape):
        return torch.rand(*shape, generator=g, device=device, dtype=torch.float32) * (hi - lo) + lo

    def ones():
        if ln == "random":
            return torch.rand(C, generator=gl, device=device, dtype=torch.float32) + 0.5
        return torch.ones(C, dtype=torch.float32, device=device)

    def zeros():
        if ln == "random":
            return torch.randn(C, generator=gl, device=device, dtype=torch.float32) * 0.1
        return torch.zeros(C, dtype=torch.float32, device=device)

    yield "emb.weight", normal(V, C)
    yield "blocks.0.ln0.weight", ones()
    yield "blocks.0.ln0.bias", zeros()
    for i in range(layers):
        p = f"blocks.{i}."
        yield p + "ln1.weight", ones()
        yield p + "ln1.bias", zeros()
        yield p + "ln2.weight", ones()
        yield p + "ln2.bias", zeros()
        yield p + "att.time_decay", uniform(-5.0, 1.0, C)
        yield p + "att.time_first", uniform(-1.0, 1.0, C)
        yield p + "att.time_mix_k", uniform(0.0, 1.0, 1, 1, C)
        yield p + "att.time_mix_v", uniform(0.0, 1.0, 1, 1, C)
        yield p + "att.time_mix_r", uniform(0.0, 1.0, 1, 1, C)
        yield p + "att.key.weight", normal(C, C)
        yield p + "att.value.weight", normal(C, C)
        yield p + "att.receptance.weight", normal(C, C)
        yield p + "att.output.weight", normal(C, C)
        yield p + "ffn.time_mix_k", uniform(0.0, 1.0, 1, 1, C)
        yield p + "ffn.time_mix_r", uniform(0.0, 1.0, 1, 1, C)
        yield p + "ffn.key.weight", normal(F, C)
        yield p + "ffn.receptance.weight", normal(C, C)
        yield p + "ffn.value.weight", normal(C, F)
    yield "ln_out.weight", ones()
    yield "ln_out.bias", zeros()
    yield "head.weight", normal(V, C)


def make_state_dict(layers: int, C: int, F: int | None = None, V: int = 50277,
                    seed: int = 0, device: str = "cpu", ln: str = "identity") -> Dict[str, torch.Tensor]:
    F = 4 * C if F is None else F
    return dict(iter_tensors(layers, C, F, V, seed, device, ln))


def random_tokens(n: int, V: int = 50277, seed: int = 0) -> torch.Tensor:
    g = torch.Generator()
    g.manual_seed(seed + 7919)
    return torch.randint(0, V, (n,), generator=g, dtype=torch.int64)
