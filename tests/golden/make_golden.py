#!/usr/bin/env python3
"""Writes tests/golden/tiny_model.pt: frozen vectors of the CPU oracle on a tiny seeded model (L=2, C=64, F=256,
V=512, LayerNorm weights and biases drawn at random), so that neither the oracle nor the GPU path can drift
unnoticed.  The oracle itself is pinned by mathematics (tests/test_oracle_pins.py); the reference ships no
vectors for this path and was not run to make these.

    python tests/golden/make_golden.py

Contents (plain tensors, loadable with weights_only=True): the quantiser's output (codes, range, offset) for three
matrices, the logits after each of 8 tokens fed one at a time, the final state, the same with exact (float64)
accumulation, and the inputs' seeds.
"""
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import rwkv_oracle as O          # noqa: E402
from rwkvstic_amd import synth               # noqa: E402

SPEC = dict(layers=2, C=64, F=256, V=512, seed=2024, ln="random")
TOKENS_SEED, N_TOKENS = 77, 8
MATS = ("blocks.0.att.key.weight", "blocks.1.ffn.value.weight", "head.weight")


def build():
    torch.set_num_threads(1)                  # the float32 sums of the CPU path depend on the BLAS blocking
    sd = synth.make_state_dict(**SPEC)
    out = {"spec": torch.tensor([SPEC["layers"], SPEC["C"], SPEC["F"], SPEC["V"], SPEC["seed"], TOKENS_SEED, N_TOKENS])}
    for key in MATS:
        codes, rng, off = O.quantize_matrix(sd[key].float())
        out[f"quant.{key}.codes"], out[f"quant.{key}.range"], out[f"quant.{key}.offset"] = codes, rng, off
    toks = synth.random_tokens(N_TOKENS, V=SPEC["V"], seed=TOKENS_SEED)
    out["tokens"] = toks
    for tag, dtype in (("f32", torch.float32), ("f64", torch.float64)):
        m = O.OracleModel(sd, matmul_dtype=dtype)
        st = m.emptyState.clone()
        logits = []
        for t in toks.tolist():
            lg, st = m.forward([t], st)
            logits.append(lg.clone())
        out[f"logits.{tag}"] = torch.stack(logits)
        out[f"state.{tag}"] = st
    return out


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tiny_model.pt")
    torch.save(build(), path)
    print(path, os.path.getsize(path), "bytes")
