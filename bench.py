#!/usr/bin/env python3
"""Headline benchmark: batch-1 greedy decode of a random-init RWKV-4 in fp32i8 on one MI355X.

    python bench.py [--gpus 1] [--steps 512] [--warmup 16] [--shape 3B] [--prefill 1024]

A step is one decoded token (one pass of the FASTQUANT forward path at batch 1).
Before the timed region the model prefills a --prefill token random prompt; then
--warmup untimed and --steps timed greedy tokens run in a device-side loop
(argmax and embedding gather on the GPU, no host round trip per token).
Prints one JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E vendor peak

# HBM bytes per launch of the single-token kernel from rocprofv3 counters (FETCH_SIZE x 2 KiB + WRITE_SIZE x 1 KiB,
# both scaled by a 1 GiB device copy in the same run): a measured constant per shape, not something this script
# can read live.  Shapes without a counter run report null.
PMC_TRAFFIC_BYTES = {"3B": 2_964_600_000}


def cpu_baseline(shape, threads: int):
    """The CPU oracle (the reference's torch CPU path restated) on this box's host cores, on a
    bounded sample: the shape's embedding + 2 layers + head, decoding 6 tokens at batch 1; the per-layer
    time is scaled to the full layer count."""
    import torch
    from oracle import rwkv_oracle as O
    from rwkvstic_amd import synth
    L, C, F, V = shape
    torch.set_num_threads(threads)
    Ls = min(2, L)
    sd = synth.make_state_dict(Ls, C, F, V, seed=1)
    m = O.OracleModel(sd)
    del sd
    state = m.emptyState.clone()
    toks = synth.random_tokens(7, V=V, seed=2).tolist()
    m.forward([toks[0]], state)                       # warm-up
    t_layers = t_rest = 0.0
    n = 0
    for t in toks[1:]:
        t0 = time.perf_counter()
        x = m.emb[torch.tensor([t])].to(torch.float64)
        x = O.layernorm(x, *m.ln_in)
        t1 = time.perf_counter()
        for i, blk in enumerate(m.blocks):
            x = m.block_forward(blk, x, state[i])
        t2 = time.perf_counter()
        x = O.layernorm(x, *m.ln_out)
        m.head(x[-1:]).squeeze()
        t3 = time.perf_counter()
        t_layers += t2 - t1
        t_rest += (t1 - t0) + (t3 - t2)
        n += 1
    per_token = (t_layers / n) * (L / Ls) + t_rest / n
    return {
        "value": round(1.0 / per_token, 3), "unit": "tokens/s", "cores": threads, "kind": "port",
        "sample": f"oracle (torch CPU fp32 matmul on uint8->fp32 cast, fp64 elementwise), shape C={C} F={F} V={V}: "
                  f"{Ls} of {L} layers + head timed over {n} decode tokens at batch 1, layer time scaled x{L // Ls}",
    }


def phase_trace(model, L: int, C: int) -> int:
    """Where a token step of the persistent kernel spends its time: every workgroup stamps its phase boundaries
    (100 MHz wall clock); the table gives, per boundary, the spread over the workgroups relative to the earliest
    workgroup's start of the layer."""
    import numpy as np
    import torch
    from rwkvstic_amd import _native as N
    if not model.fused_step:
        print("phase trace: this shape does not run the persistent kernel", file=sys.stderr)
        return 2
    G, per = C // 16, 24
    st = model.emptyState.clone()
    for t in range(5):
        _, st = model.forward([t + 3], st)
    buf = torch.zeros(G * L * per, dtype=torch.int64, device="cuda")
    N.check(N.lib().rwkv_model_set_trace(model._handle, buf.data_ptr()))
    model.forward([77], st)
    torch.cuda.synchronize()
    model.check()
    N.check(N.lib().rwkv_model_set_trace(model._handle, None))
    t = buf.cpu().numpy().astype("float64").reshape(G, L, per) * 0.01          # microseconds
    names = {0: "start", 16: "A:polled", 1: "A:stats", 2: "A:digits", 3: "A:mfma", 20: "A:sums", 4: "finA",
             17: "B:polled", 5: "B:scale", 6: "B:digits", 7: "B:mfma", 21: "B:sums", 8: "finB",
             18: "C:polled", 9: "C:stats", 10: "C:digits", 11: "C:mfma", 12: "finC",
             19: "D:polled", 13: "D:scale", 14: "D:digits", 15: "D:mfma", 22: "D:sums"}
    print("phases: A = att k, v, r   B = att output   C = ffn key + receptance   D = ffn value   (microseconds)")
    print("X:polled = the polling wave holds every workgroup's first records; X:stats / X:scale = all records reduced "
          "(workgroup barrier); X:digits = gathered and written as digit planes; X:mfma = tile sums parked by the "
          "weight-streaming waves; X:sums = the owner wave has combined them; finX = results published")
    for l in sorted({min(L - 1, 1), L // 2, L - 2 if L > 2 else L - 1}):
        base = t[:, l, 0].min()
        print(f"layer {l}")
        prev = 0.0
        for i, name in names.items():
            v = t[:, l, i] - base
            med = float(np.median(v))
            print(f"  {name:9s} min {v.min():6.2f}  med {med:6.2f}  max {v.max():6.2f}   (+{med - prev:5.2f} after the previous boundary)")
            prev = med
    if L > 3:
        print(f"per layer, workgroup 0, layers 1..{L - 2}: {(t[0, L - 1, 0] - t[0, 1, 0]) / (L - 2):.2f} us")
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    one = torch.tensor([5], device="cuda")
    e0.record()
    for _ in range(50):
        model.forward(one, st)
    e1.record()
    torch.cuda.synchronize()
    model.check()
    print(f"token step without stamps: {e0.elapsed_time(e1) / 50 * 1e3:.1f} us")
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=512)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--shape", default="3B", choices=["169M", "3B", "14B"])
    ap.add_argument("--prefill", type=int, default=1024)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate-copy-mib", type=int, default=0,
                    help="before the workload, copy this many MiB device to device once (a kernel of known HBM "
                         "traffic: the yardstick for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--phase-trace", action="store_true",
                    help="instead of the benchmark: one token step of the persistent kernel with its 100 MHz phase "
                         "stamps switched on (rwkv_model_set_trace), printed as a table of min / median / max over "
                         "the workgroups per phase boundary, for three layers")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (batch-1 decode of one model replica); "
              "--gpus must be 1", file=sys.stderr)
        return 2

    import torch
    from rwkvstic_amd import synth
    from rwkvstic_amd.model import HipRWKV

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    shape = synth.SHAPES[args.shape]
    L, C, F, V = shape
    torch.cuda.set_device(0)
    t0 = time.perf_counter()
    model = HipRWKV(synth.iter_tensors(L, C, F, V, seed=0, device="cuda"), device="cuda:0")
    torch.cuda.synchronize()
    load_s = time.perf_counter() - t0
    wbytes = model.weight_bytes()

    stream = torch.cuda.current_stream()
    ev = lambda: torch.cuda.Event(enable_timing=True)

    if args.phase_trace:
        return phase_trace(model, L, C)

    if args.calibrate_copy_mib > 0:
        n = args.calibrate_copy_mib << 20
        src = torch.full((n,), 3, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)                    # one elementwise copy kernel: reads n bytes, writes n bytes
        torch.cuda.synchronize()
        del src, dst

    # ---- prefill -------------------------------------------------------------
    prompt = synth.random_tokens(args.prefill, V=V, seed=0).cuda()
    model.forward(prompt, model.emptyState.clone())      # untimed pass: allocates the prompt workspace
    state = model.emptyState.clone()
    e0, e1 = ev(), ev()
    torch.cuda.synchronize()
    e0.record(stream)
    logits, state = model.forward(prompt, state)
    e1.record(stream)
    torch.cuda.synchronize()
    prefill_ms = e0.elapsed_time(e1)
    tok = int(logits.argmax())

    # ---- decode --------------------------------------------------------------
    if args.warmup > 0:
        toks, logits, state = model.decode_greedy(tok, args.warmup, state)
        tok = int(toks[-1])
    torch.cuda.synchronize()
    e0, e1 = ev(), ev()
    w0 = time.perf_counter()
    e0.record(stream)
    toks, logits, state = model.decode_greedy(tok, args.steps, state)
    e1.record(stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - w0) * 1e3
    dev_ms = e0.elapsed_time(e1)
    ms_per_step = wall_ms / args.steps
    tok_s = args.steps / (wall_ms / 1e3)
    assert bool(torch.isfinite(logits).all()), "non-finite logits"

    # ---- the dominant kernel on its own: single-token forward calls, HIP events on the launch stream
    nk = min(64, args.steps)
    st2 = state.clone()
    one = toks[-1:].clone()
    model.forward(one, st2)
    torch.cuda.synchronize()
    e0, e1 = ev(), ev()
    e0.record(stream)
    for _ in range(nk):
        model.forward(one, st2)
    e1.record(stream)
    torch.cuda.synchronize()
    step_us = e0.elapsed_time(e1) / nk * 1e3
    achieved = wbytes / (step_us * 1e-6) / 1e9
    out = {
        "metric": "decode tokens/s @ RWKV-4 3B-shape fp32i8 B=1" if args.shape == "3B"
                  else f"decode tokens/s @ RWKV-4 {args.shape}-shape fp32i8 B=1",
        "value": round(tok_s, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f64 elementwise, u8 weights x fixed-point activations accumulated exactly in i32 (int8 MFMA)", "data": "synthetic",
        "config": {"workload": f"RWKV-4 {args.shape}-shape (L={L}, C={C}, F={F}, V={V}) fp32i8, random-init seed 0; "
                               f"{args.prefill}-token random prompt prefilled, then {args.steps} greedy tokens at batch 1",
                   "weight_bytes_per_token": wbytes, "load_seconds": round(load_s, 2)},
        "prefill_tokens_per_s": round(args.prefill / (prefill_ms / 1e3), 1),
        "roofline": {"bound": "hbm",
                     "kernel": "rwkv::decode_kernel (persistent, one launch per token; launch_us includes the prep_kernel in front of it)"
                               if model.fused_step
                               else "decode token step (all phase kernels of one token)",
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": PMC_TRAFFIC_BYTES.get(args.shape) if model.fused_step else None,
                     "launch_us": round(step_us, 2), "decode_loop_us_per_token": round(dev_ms / args.steps * 1e3, 2)},
    }
    if not args.no_cpu_baseline:
        threads = min(16, os.cpu_count() or 1)
        out["cpu_baseline"] = cpu_baseline(shape, threads)
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
