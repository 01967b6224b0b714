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
# both scaled by a 1 GiB device copy in the same run; profiles/decode_kernel_3B_b1_hbm_traffic.md): a measured
# constant per shape, not something this script can read live.  It is tied to the kernel sources it was measured on
# by their digest (csrc_digest() below): with any other sources the bench reports null instead of a stale figure.
PMC_TRAFFIC = {"3B": {"bytes": 2_974_128_334, "csrc_digest": "1d0f2145494a3c09"}}


DECODE_SOURCES = ("gen_decode_back.py", "rwkv_common.h", "rwkv_decode.h", "rwkv_decode.hip", "rwkv_decode_back.inc")


def csrc_digest() -> str:
    """sha256 over the sources of the single-token kernel (what `traffic` was measured on): the kernel, its
    generated weight-streaming program and the generator, and the common header they include."""
    import hashlib
    d = os.path.join(ROOT, "rwkvstic_amd", "csrc")
    h = hashlib.sha256()
    for name in DECODE_SOURCES:
        h.update(name.encode())
        h.update(open(os.path.join(d, name), "rb").read())
    return h.hexdigest()[:16]


kCpuTokens = 12     # timed decode tokens of the CPU leg: about 10 s at the 3B shape on 16 host threads


def cpu_baseline(shape, threads: int, layers_timed: int):
    """The CPU oracle (the reference's torch CPU path restated: float32 matmul on a per-call uint8 -> float32 cast,
    float64 element-wise, Python WKV step) on this box's host cores, decoding at batch 1 on a bounded sample:
    `layers_timed` of the shape's layers (0 = all, the default) + embedding + head, 1 untimed and `kCpuTokens` timed
    tokens; with fewer layers the layer time is scaled to the full depth.  The matrices are drawn directly as codes (oracle QMat.synthetic): the cost of the
    path does not depend on their values and running the quantiser over the model would take longer than the
    sample itself."""
    import torch
    from oracle import rwkv_oracle as O
    from rwkvstic_amd import synth
    L, C, F, V = shape
    torch.set_num_threads(threads)
    Ls = L if layers_timed <= 0 else min(layers_timed, L)
    m = O.OracleModel.synthetic(Ls, C, F, V, seed=1)
    state = m.emptyState.clone()
    toks = synth.random_tokens(1 + kCpuTokens, V=V, seed=2).tolist()
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
    scaled = "" if Ls == L else f", layer time scaled x{L / Ls:g}"
    return {
        "value": round(1.0 / per_token, 3), "unit": "tokens/s", "cores": threads, "kind": "port",
        "sample": f"oracle (torch CPU fp32 matmul on uint8->fp32 cast, fp64 elementwise), shape C={C} F={F} V={V}: "
                  f"{Ls} of {L} layers + head timed over {n} decode tokens at batch 1{scaled}",
    }


def calibrate_copy(mib: int) -> None:
    """One device-to-device copy of `mib` MiB (a kernel of known HBM traffic: the yardstick for rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE readings of the same run)."""
    if mib <= 0:
        return
    import torch
    n = mib << 20
    src = torch.full((n,), 3, dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    dst.copy_(src)                    # one copy kernel: reads n bytes, writes n bytes
    torch.cuda.synchronize()
    del src, dst


def isolated_matvec(device="cuda"):
    """BASELINE configuration 1: the quantised matrix-vector product on its own (rwkv_mm8_packed, general
    four-vector form) at the three 3B shapes, batch 1 and 8.  Each call reads a different matrix out of a pool
    of at least 512 MB, so no matrix is served from L2 or the 256 MB memory-side cache: GB/s = in x out bytes
    per call / time per call over HIP events."""
    import torch
    from rwkvstic_amd import _native, ops
    N_ws = _native.lib().rwkv_mm8_m16_workspace_bytes
    out = []
    pool = torch.randint(0, 256, (640 << 20,), dtype=torch.uint8, device=device)       # random bytes are valid packed codes
    g = torch.Generator(device=device).manual_seed(3)
    for n_in, n_out in ((2560, 2560), (2560, 10240), (10240, 2560)):
        nbytes = n_in * n_out
        n_mats = pool.numel() // nbytes
        r_row = torch.rand(n_in, generator=g, device=device) * 9e-4 + 1e-4
        m_row = (torch.randn(n_in, generator=g, device=device) * 0.01).double()
        r_col = torch.rand(n_out, generator=g, device=device) * 9e-4 + 1e-4
        m_col = torch.randn(n_out, generator=g, device=device) * 0.01
        for B in (1, 8):
            x = torch.randn(B, n_in, generator=g, device=device)
            y = torch.empty(B, n_out, dtype=torch.float64, device=device)
            calls = 2 * n_mats

            def run(k):
                for i in range(k):
                    off = (i % n_mats) * nbytes
                    ops.mm8_packed(x, pool[off:off + nbytes], n_in, n_out, r_row, m_row, r_col, m_col, out=y)
            run(n_mats)
            torch.cuda.synchronize()
            # the calls are recorded into a HIP graph and replayed, so that the time is the kernels' and not
            # the host's launch rate (about 10 us per call from Python, more than the smaller products take)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                run(calls)
            graph.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            graph.replay()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) / calls * 1e3
            out.append({"shape": f"{n_in}x{n_out}", "batch": B, "kernel": "mm8_packed", "us_per_call": round(us, 2),
                        "GB_per_s": round(nbytes / us / 1e3, 1), "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                        "distinct_matrices": n_mats})
            # the matrix-core route (rwkv_mm8_m16: digits once, then int8 MFMA on the M16 layout); random bytes
            # are valid M16 blocks too
            ws = torch.empty(N_ws(B, n_in), dtype=torch.uint8, device=device)

            def run16(k):
                for i in range(k):
                    off = (i % n_mats) * nbytes
                    ops.mm8_m16(x, pool[off:off + nbytes], n_in, n_out, r_row, m_row, r_col, m_col, out=y, workspace=ws)
            run16(n_mats)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                run16(calls)
            graph.replay()
            torch.cuda.synchronize()
            e0.record()
            graph.replay()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) / calls * 1e3
            out.append({"shape": f"{n_in}x{n_out}", "batch": B, "kernel": "mm8_m16", "us_per_call": round(us, 2),
                        "GB_per_s": round(nbytes / us / 1e3, 1), "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                        "distinct_matrices": n_mats})
    return out


def isolated_wkv(device="cuda"):
    """BASELINE configuration 2: rwkv_wkv_f32 at B=8, T=1024, C=2560 (k, v read and y written once: 251.7 MB)."""
    import torch
    from rwkvstic_amd import ops
    B, T, C = 8, 1024, 2560
    g = torch.Generator(device=device).manual_seed(4)
    k = torch.randn(B, T, C, generator=g, device=device)
    v = torch.randn(B, T, C, generator=g, device=device)
    w = -torch.exp(torch.rand(C, generator=g, device=device) * 9 - 8)
    u = torch.rand(C, generator=g, device=device) * 2 - 1
    us = []
    for _ in range(4):
        aa, bb = torch.zeros(B, C, device=device), torch.zeros(B, C, device=device)
        pp = torch.full((B, C), -1e38, device=device)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        ops.wkv_f32(w, u, k, v, aa, bb, pp)
        e1.record()
        torch.cuda.synchronize()
        us.append(e0.elapsed_time(e1) * 1e3)
    best = sorted(us[1:])[len(us[1:]) // 2]
    nbytes = 3 * B * T * C * 4
    return {"shape": f"B={B} T={T} C={C}", "us": round(best, 1), "GB_per_s": round(nbytes / best / 1e3, 1),
            "bytes": nbytes}


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
    G, per = (C // 32 if C > 4096 else C // 16), 24          # owner workgroups of the persistent kernel
    GA = N.lib().rwkv_model_trace_workgroups(model._handle)  # ... and the helper workgroups behind them
    st = model.emptyState.clone()
    for t in range(5):
        _, st = model.forward([t + 3], st)
    buf = torch.zeros(GA * L * per, dtype=torch.int64, device="cuda")
    N.check(N.lib().rwkv_model_set_trace(model._handle, buf.data_ptr()))
    model.forward([77], st)
    torch.cuda.synchronize()
    model.check()
    N.check(N.lib().rwkv_model_set_trace(model._handle, None))
    t_all = buf.cpu().numpy().astype("float64").reshape(GA, L, per) * 0.01     # microseconds
    t, th = t_all[:G], t_all[G:]
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
        if GA > G:
            print("  helper workgroups (ffn key), same time base:")
            prev = float(np.median(t[:, l, 8] - base))
            print(f"    (owners' finB, the input of this phase: med {prev:6.2f})")
            for i, name in enumerate(("records", "stats", "digits", "parked", "published", "next weights")):
                v = th[:, l, i] - base
                med = float(np.median(v))
                print(f"    {name:12s} min {v.min():6.2f}  med {med:6.2f}  max {v.max():6.2f}   (+{med - prev:5.2f})")
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


def batch_decode(model, args, shape) -> int:
    """B independent sequences (own state, own seeded 64-token prompt), greedy decode by batch steps."""
    import torch
    from rwkvstic_amd import synth
    L, C, F, V = shape
    B = args.batch
    states = []
    toks = []
    for b in range(B):
        lg, s = model.forward(synth.random_tokens(64, V=V, seed=100 + b).cuda(), model.emptyState.clone())
        states.append(s)
        toks.append(lg.argmax())
    st = torch.stack(states).contiguous()
    tok = torch.stack(toks)
    for _ in range(max(args.warmup, 1)):
        lg, st = model.forward_batch(tok, st)
        tok = lg.argmax(dim=1)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        lg, st = model.forward_batch(tok, st)
        tok = lg.argmax(dim=1)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / args.steps
    assert bool(torch.isfinite(lg).all())
    wbytes = model.weight_bytes()
    print(json.dumps({
        "metric": f"decode tokens/s @ RWKV-4 {args.shape}-shape fp32i8 B={B}", "value": round(B / (ms / 1e3), 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "data": "synthetic",
        "config": {"workload": f"RWKV-4 {args.shape}-shape (L={L}, C={C}, F={F}, V={V}) fp32i8, {B} independent states, "
                               f"seeded 64-token prompts, greedy batch steps", "weight_bytes_per_step": wbytes},
        "roofline": {"bound": "hbm", "achieved": round(wbytes / (ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(wbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "note": "one batch step streams the weights once for all sequences"}}), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=512)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--shape", default="3B", choices=["169M", "3B", "14B"])
    ap.add_argument("--prefill", type=int, default=1024)
    ap.add_argument("--prefill-chunk", type=int, default=0,
                    help="feed the prompt in chunks of this many tokens (0 = one call); the 14B configuration uses 256")
    ap.add_argument("--batch", type=int, default=1,
                    help="instead of the batch-1 benchmark: this many independent sequences, each prefilled with its own "
                         "64-token random prompt, decoded greedily one batch step at a time (the 14B configuration's "
                         "batch-32 decode); prints its own JSON line")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-baseline-layers", type=int, default=0,
                    help="layers of the shape the CPU baseline times (0 = all of them, the default; fewer: scaled to the full depth)")
    ap.add_argument("--no-isolated", action="store_true", help="skip the isolated matvec / WKV measurements")
    ap.add_argument("--isolated-only", action="store_true",
                    help="only the isolated matvec and WKV kernels (for profiling them on their own)")
    ap.add_argument("--calibrate-copy-mib", type=int, default=0,
                    help="before the workload, copy this many MiB device to device once (a kernel of known HBM "
                         "traffic: the yardstick for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--phase-trace", action="store_true",
                    help="instead of the benchmark: one token step of the persistent kernel with its 100 MHz phase "
                         "stamps switched on (rwkv_model_set_trace), printed as a table of min / median / max over "
                         "the workgroups per phase boundary, for three layers")
    ap.add_argument("--lib", default=None,
                    help="load this build of the library instead of the in-tree one (a diagnostic build made with "
                         "`python -m rwkvstic_amd.build --define NAME --output FILE`)")
    args = ap.parse_args()
    if args.lib:
        from rwkvstic_amd import _native
        _native.LIB_PATH = os.path.abspath(args.lib)
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (batch-1 decode of one model replica); "
              "--gpus must be 1", file=sys.stderr)
        return 2

    import torch
    from rwkvstic_amd import synth
    from rwkvstic_amd.model import HipRWKV

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    if args.isolated_only:
        torch.cuda.set_device(0)
        calibrate_copy(args.calibrate_copy_mib)
        print(json.dumps({"isolated_matvec": isolated_matvec(), "isolated_wkv": isolated_wkv()}), flush=True)
        return 0
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
    if args.batch > 1:
        return batch_decode(model, args, shape)

    calibrate_copy(args.calibrate_copy_mib)

    # ---- prefill -------------------------------------------------------------
    prompt = synth.random_tokens(args.prefill, V=V, seed=0).cuda()
    model.forward(prompt, model.emptyState.clone())      # untimed pass: allocates the prompt workspace
    state = model.emptyState.clone()
    e0, e1 = ev(), ev()
    torch.cuda.synchronize()
    e0.record(stream)
    chunk = args.prefill_chunk if args.prefill_chunk > 0 else args.prefill
    for c0 in range(0, args.prefill, chunk):
        logits, state = model.forward(prompt[c0:c0 + chunk], state)
    e1.record(stream)
    torch.cuda.synchronize()
    prefill_ms = e0.elapsed_time(e1)
    tok = int(logits.argmax())
    # the same prompt in 256-token chunks (the chunk size the 14B configuration prescribes): its own key of the line
    chunked_tok_s = None
    if chunk > 256 and args.prefill >= 512:
        st256 = model.emptyState.clone()
        model.forward(prompt[:256], st256.clone())
        f0, f1 = ev(), ev()
        torch.cuda.synchronize()
        f0.record(stream)
        for c0 in range(0, args.prefill, 256):
            lg256, st256 = model.forward(prompt[c0:c0 + 256], st256)
        f1.record(stream)
        torch.cuda.synchronize()
        chunked_tok_s = round(args.prefill / (f0.elapsed_time(f1) / 1e3), 1)
        # (chunking changes the order of float operations only in the WKV scan: same token, close logits)
        assert int(lg256.argmax()) == tok and float((lg256 - logits).abs().max()) < 1e-4, "256-token chunks disagree with the whole prompt"

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
    model.check()            # raises if a token step gave up waiting (its results would be stale): no number then

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
    model.check()
    # the persistent kernel alone: the library records events on the launch stream right before and after each of
    # its launches (the per-token preparation launch stays outside); the phase kernels have no such single launch
    kernel_us = model.time_token_kernel(int(one[0]), nk, st2) if model.fused_step else step_us
    model.check()
    achieved = wbytes / (kernel_us * 1e-6) / 1e9
    traffic = PMC_TRAFFIC.get(args.shape)
    digest = csrc_digest()
    traffic_now = traffic["bytes"] if (traffic and model.fused_step and traffic["csrc_digest"] == digest) else None
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
        "prefill_chunk": chunk,
        "prefill_tokens_per_s_chunk256": chunked_tok_s,
        "roofline": {"bound": "hbm",
                     "kernel": "rwkv::decode_kernel (persistent, one launch per token; kernel_us = its own duration, launch_us = one "
                               "single-token forward call = prep_kernel + decode_kernel)"
                               if model.fused_step
                               else "decode token step (all phase kernels of one token)",
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": traffic_now, "traffic_measured_on_csrc": traffic["csrc_digest"] if traffic else None,
                     "csrc_digest": digest,
                     "kernel_us": round(kernel_us, 2), "launch_us": round(step_us, 2), "decode_loop_us_per_token": round(dev_ms / args.steps * 1e3, 2)},
    }
    # the kept API: RWKV(...).forward(number=n) with the built-in samplers (device-side loop) next to the raw loop
    from rwkvstic_amd.master import RWKVMaster, greedy, typical
    api = {}
    n_api = min(256, max(args.steps, 8))
    for name, smp in (("typical", typical), ("greedy", greedy)):
        shell = RWKVMaster(model, model.emptyState, smp)
        shell.myState = state.clone()
        shell.lastToken = [int(toks[-1])]
        shell.forward(number=4, stopTokens=[])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        shell.forward(number=n_api, stopTokens=[])
        torch.cuda.synchronize()
        api[name] = round(n_api / (time.perf_counter() - t0), 1)
    out["api_forward_tokens_per_s"] = dict(api, tokens=n_api, note="RWKVMaster.forward(number=n): sampler, end_adj and stop test on the device")
    if not args.no_isolated:
        out["isolated_matvec"] = isolated_matvec()
        out["isolated_wkv"] = isolated_wkv()
    if not args.no_cpu_baseline:
        threads = min(16, os.cpu_count() or 1)
        out["cpu_baseline"] = cpu_baseline(shape, threads, args.cpu_baseline_layers)
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
