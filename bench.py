#!/usr/bin/env python3
"""Benchmark of the quantized matmul hot path on one MI355X.

Workload (the configuration the headline metric is quoted on): batch-1 decode GEMVs of a
Llama-3-8B feed-forward block in Q4_K -- gate and up 4096 -> 14336 and down 14336 -> 4096 --
on seeded synthetic weights and N(0,1) activations.  One step is one pass over that block: the
activation quantizer and one GEMV launch over gate and up (they read the same input), then the
quantizer and the GEMV for down, through the library's C ABI with inputs and outputs resident in HBM.  Steps rotate over enough distinct weight copies that
every pass streams from HBM rather than from the last-level cache.

Prints ONE JSON line: whole-step throughput in algorithmic GB/s, a roofline object for the
dominant kernel (the Q4_K GEMV over gate+up, timed with HIP events over batches of back-to-back
launches: median and fastest batch; beside it a launch that only reads the same bytes, as the measured
streaming peak for this footprint) and the CPU path (the C oracle, all host cores) timed on a bounded
sample.  The same line carries the other legs: the 512-token prefill GEMM, the host-pointer (trait)
path, the sweep over the other benchmark configurations and the 8B-shaped decode step; `--only-*`,
`--sweep` and `--only-row` run single legs, which is what the profiles under profiles/ were taken over.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import numpy as np  # noqa: E402

Q4_K = 12
HIDDEN, FFN = 4096, 14336
HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
# HBM bytes per launch of the dominant kernel, from `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE`
# runs of `bench.py --only-roofline`, calibrated on that run's 64 MiB copy (profiles/).
GEMV_Q4K_GATE_UP_TRAFFIC = 66248100
# The same kernel's duration by `rocprofv3 --kernel-trace --stats` on `bench.py --only-roofline`, condensed by
# `bench.py --trace-summary` (profiles/gemv_q4k_gate_up_4096x14336_kernel_trace.md): mean over all dispatches,
# median, and mean of the dispatches that started within 500 ns of their predecessor's end.  Under the profiler
# one dispatch in five starts on an idle device and runs longer; the events of an unprofiled run see none such.
GEMV_Q4K_GATE_UP_ROCPROF = {"avg_us": 11.878, "median_us": 11.759, "back_to_back_avg_us": 11.809, "dispatches": 1250}


def gemv_bytes(in_dim: int, out_dim: int, t: int = 1) -> int:
    """Algorithmic bytes of one Q4_K GEMV: raw GGUF rows + f32 x + f32 y."""
    return out_dim * (in_dim // 256 * 144) + 4 * in_dim * t + 4 * out_dim * t


# Untimed calls before a matrix-core GEMM of 32 tokens or more is timed.  A run of such calls speeds up over its
# first hundred or so (4096 -> 14336 at 2048 tokens, batches of 30 calls back to back: 385, 334, 327, 326 us a
# call; at 512 tokens 115, 110, 103, 99): the device's clock settles under the load.  A prefill pass is 224 such
# calls in a row, so the steady figure is the one that prices it; the GEMV legs show no such drift.
GEMM_WARM = 100


def batched_us(hiprt, stream, launch, batches: int, per_batch: int, warm: int = 10, many=None) -> dict:
    """Times `batches` runs of `per_batch` back-to-back launches with HIP events on the launch stream;
    the figures are microseconds per launch: the fastest batch, the median batch and the mean.
    `launch(i)` enqueues launch number i; `many(i, n)`, where given, enqueues launches i .. i + n - 1 from
    compiled code instead (no interpreter between two launches)."""
    if many is not None:
        many(0, warm)
    else:
        for i in range(warm):
            launch(i)
    stream.synchronize()
    ev = [(hiprt.Event(), hiprt.Event()) for _ in range(batches)]
    k = warm
    for e0, e1 in ev:
        e0.record(stream)
        if many is not None:
            many(k, per_batch)
            k += per_batch
        else:
            for _ in range(per_batch):
                launch(k)
                k += 1
        e1.record(stream)
    ev[-1][1].synchronize()
    us = [e0.elapsed_ms(e1) * 1e3 / per_batch for e0, e1 in ev]
    if os.environ.get("OGM_BENCH_DEBUG"):
        print("batches:", [round(u, 1) for u in us], file=sys.stderr)
    us = sorted(us)
    return {"min": round(us[0], 3), "median": round(us[len(us) // 2], 3), "mean": round(sum(us) / len(us), 3),
            "launches": batches * per_batch}


def trace_summary(path: str, period: int = 0) -> dict:
    """Condenses a `rocprofv3 --kernel-trace --output-format csv` trace (the *_kernel_trace.csv file, or a
    folder searched for one) per kernel name: dispatch count, mean / median / min / max duration from the
    dispatches' own start and end stamps, and -- over runs of consecutive dispatches of the same kernel with
    no gap above 20 us between them -- (last end - first start) / dispatches and the mean gap from one
    dispatch's end to the next one's start, how many of those gaps exceed 500 ns (the device sat idle: the
    host, slowed by the profiler's hooks, did not keep up) and the mean duration of the dispatches that started
    within 500 ns of their predecessor's end (back to back, as in an unprofiled run)."""
    import csv
    import glob
    if os.path.isdir(path):
        found = sorted(glob.glob(os.path.join(path, "**", "*kernel_trace.csv"), recursive=True))
        if not found:
            raise SystemExit(f"no *kernel_trace.csv under {path}")
        path = found[0]
    rows = []
    with open(path, newline="") as f:
        for r in csv.DictReader(f):
            rows.append((int(r["Start_Timestamp"]), int(r["End_Timestamp"]), r["Kernel_Name"]))
    rows.sort()
    per = {}
    i = 0
    while i < len(rows):
        j = i
        while j + 1 < len(rows) and rows[j + 1][2] == rows[i][2] and rows[j + 1][0] - rows[j][1] <= 20000:
            j += 1
        k = per.setdefault(rows[i][2], {"dur": [], "span_ns": 0, "span_n": 0, "gaps": [], "b2b": [], "seq": []})
        k["dur"] += [e - b for b, e, _ in rows[i:j + 1]]
        k["seq"] += [e - b for b, e, _ in rows[i:j + 1]]   # in dispatch order (dur is sorted below)
        if j > i:   # a run of at least two
            k["span_ns"] += rows[j][1] - rows[i][0]
            k["span_n"] += j - i + 1
            k["gaps"] += [rows[n + 1][0] - rows[n][1] for n in range(i, j)]
            # dispatches that started within 500 ns of their predecessor's end: the device was not left idle
            k["b2b"] += [rows[n + 1][1] - rows[n + 1][0] for n in range(i, j) if rows[n + 1][0] - rows[n][1] <= 500]
        i = j + 1
    out = {"file": path, "kernels": []}
    for name, k in sorted(per.items(), key=lambda kv: -sum(kv[1]["dur"])):
        d = sorted(k["dur"])
        row = {"kernel": name[:120], "dispatches": len(d), "mean_ns": round(sum(d) / len(d), 1),
               "median_ns": d[len(d) // 2], "min_ns": d[0], "max_ns": d[-1]}
        if k["span_n"]:
            row.update({"dispatches_in_runs": k["span_n"],
                        "span_ns_per_dispatch": round(k["span_ns"] / k["span_n"], 1),
                        "mean_gap_ns": round(sum(k["gaps"]) / len(k["gaps"]), 1),
                        "gaps_over_500ns": sum(1 for g in k["gaps"] if g > 500)})
            if k["b2b"]:
                row.update({"back_to_back_dispatches": len(k["b2b"]),
                            "back_to_back_mean_ns": round(sum(k["b2b"]) / len(k["b2b"]), 1)})
        if period > 1 and len(k["seq"]) >= 2 * period:
            # mean duration by dispatch number modulo the rotation's length: one entry per weight copy
            row["mean_ns_by_dispatch_mod_%d" % period] = [
                round(sum(k["seq"][i::period]) / len(k["seq"][i::period]), 1) for i in range(period)]
        out["kernels"].append(row)
    return out


def sweep(be, helpers, hiprt, only: str = "", light: bool = False) -> dict:
    """Kernel timings at the full size of every benchmark configuration: device-resident inputs,
    back-to-back calls over weight copies totalling more than the 256 MB last-level cache, HIP events
    on the launch stream.  Each figure covers the whole call (activation quantizer + matmul kernels)."""
    Q8_0, Q6_K, Q5_1, IQ4_XS = 8, 14, 7, 23
    blk = {Q8_0: (34, 32), Q4_K: (144, 256), Q6_K: (210, 256), Q5_1: (24, 32), IQ4_XS: (136, 256)}
    names = {Q8_0: "Q8_0", Q4_K: "Q4_K", Q6_K: "Q6_K", Q5_1: "Q5_1", IQ4_XS: "IQ4_XS"}
    stream = hiprt.Stream()
    out = {"device": be.device_name(),
           "unit": "us per call (activation quantizer + matmul kernels), median and fastest of 8 batches of "
                   "back-to-back calls, HIP events on the launch stream; GB/s and TFLOP/s are algorithmic, "
                   "from the median", "rows": []}

    uploaded = {}   # (type, in, out) -> device copies, shared by the rows of one matrix and freed at the end

    def run(t, in_dim, out_dim, T, decode, label, n=256):
        if only and only not in label:
            return
        w_bytes = out_dim * (in_dim // blk[t][1]) * blk[t][0]
        copies = max(2, min(24, (300 << 20) // w_bytes + 1))
        if (t, in_dim, out_dim) not in uploaded:
            raw = helpers.synth_weights(t, in_dim, out_dim, 11)
            uploaded[(t, in_dim, out_dim)] = [be.upload_raw(raw, t, in_dim, out_dim) for _ in range(copies)]
        hs = uploaded[(t, in_dim, out_dim)]
        x = hiprt.DeviceBuffer.from_numpy(helpers.synth_x(T, in_dim, 5))
        y = hiprt.DeviceBuffer(4 * T * out_dim)
        if light:
            n = max(32, n // 2)
        # (the tiled GEMMs are timed in their steady state, GEMM_WARM calls in: see the constant)
        st = batched_us(hiprt, stream, lambda i: be.matmul_dev(hs[i % copies], x.ptr, T, y.ptr, decode, stream.ptr),
                        8, max(4, n // 8), warm=GEMM_WARM if T >= 32 else 5)
        us = st["median"]
        nbytes = w_bytes + 4 * T * (in_dim + out_dim)
        flops = 2.0 * T * in_dim * out_dim
        out["rows"].append({"config": label, "type": names[t], "in": in_dim, "out": out_dim, "tokens": T,
                            "us": round(us, 2), "us_min": round(st["min"], 2), "launches": st["launches"],
                            "GBps": round(nbytes / us / 1e3, 1),
                            "frac_hbm": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                            "TFLOPs": round(flops / us / 1e6, 2), "kernel": be.last_kernel()})
        x.free()
        y.free()

    run(Q8_0, 4096, 4096, 1, False, "C1 GEMV")
    run(Q4_K, HIDDEN, FFN, 1, False, "C2 gate/up GEMV")
    run(Q4_K, FFN, HIDDEN, 1, False, "C2 down GEMV")
    for T in (1, 4, 8):
        run(Q6_K, 4096, 128256, T, False, f"C3 vocab batch {T}", n=64)
        run(Q4_K, 4096, 4096, T, False, f"C3 q/o batch {T}")
        run(Q4_K, 4096, 1024, T, False, f"C3 k/v batch {T}")
        if T > 1:   # the other two projections of a verify batch (their single-token rows are C2 and C5)
            run(Q4_K, HIDDEN, FFN, T, False, f"C3 gate/up batch {T}")
            run(Q6_K, FFN, HIDDEN, T, False, f"C3 ffn_down batch {T}")
    for T in (128, 512, 2048):
        run(Q4_K, HIDDEN, FFN, T, False, f"C4 prefill GEMM M={T}", n=64)
    # the 8B shapes' other projections at 512 tokens: grids that leave the 128-row plane kernel half empty
    run(Q4_K, 4096, 4096, 512, False, "C4 wo-sized GEMM 4096->4096 M=512", n=64)
    run(Q4_K, 4096, 6144, 512, False, "C4 q+k+v-sized GEMM 4096->6144 M=512", n=64)
    run(Q6_K, FFN, HIDDEN, 512, False, "C4 ffn_down GEMM 14336->4096 M=512", n=64)
    run(Q6_K, FFN, HIDDEN, 1, False, "C5 ffn_down GEMV")
    # the types beside the K-quants at batch sizes of a verify batch and a prompt (C1's matrix, and the FFN's)
    for T in (16, 32, 128, 512):
        run(Q8_0, 4096, 4096, T, False, f"C1-type Q8_0 4096->4096 batch {T}", n=64)
    run(Q8_0, FFN, HIDDEN, 32, False, "Q8_0 ffn_down-sized 14336->4096 batch 32", n=64)
    run(Q8_0, HIDDEN, FFN, 512, False, "Q8_0 gate-sized 4096->14336 batch 512", n=64)
    run(IQ4_XS, HIDDEN, FFN, 32, False, "IQ4_XS gate-sized 4096->14336 batch 32", n=64)
    run(IQ4_XS, HIDDEN, FFN, 512, False, "IQ4_XS gate-sized 4096->14336 batch 512", n=64)
    run(Q5_1, HIDDEN, FFN, 512, False, "Q5_1 gate-sized 4096->14336 batch 512", n=32)
    for hs in uploaded.values():
        for h in hs:
            be.free_weight(h)
    return out


DECODE_MODELS = {   # n_layer, n_embd, n_head, n_kv, head_dim, n_ff, n_vocab
    "8b": (32, 4096, 32, 8, 128, 14336, 128256),
    # Llama-3.1-405B's layer shapes (16 query heads per K/V head); run on a few of its 126 layers (--decode-layers)
    "405b": (126, 16384, 128, 8, 128, 53248, 128256),
}


def decode_leg(be, helpers, hiprt, steps: int, warmup: int, ctx: int, check: bool, only_prefill: int = 0,
               with_prefill: bool = True, only_verify: int = 0, attn_timeline: bool = False, attn_chunks_per_wg: int = 0, model: str = "8b",
               layers_run: int = 0) -> dict:
    """Batch-1 decode of an 8B-shaped Llama (32 layers: wq, wo 4096x4096, wk, wv 4096->1024, gate, up
    4096->14336 in Q4_K; down 14336->4096 and the 128256-row output in Q6_K; f16 KV cache holding `ctx`
    random positions): tokens per second of ogm_llama_decode_dev with the embedding row, the logits and
    the greedy token resident in HBM.  Every layer has its own device copy of the weights."""
    from orangu_amd import LlamaDecoder, QuantMatrix
    Q6_K = 14
    n_layer_model, n_embd, n_head, n_kv, hd, n_ff, n_vocab = DECODE_MODELS[model]
    n_layer = layers_run if layers_run > 0 else n_layer_model
    seed = 515
    rng = np.random.default_rng(seed)
    shapes = {"wq": (Q4_K, n_embd, n_embd), "wk": (Q4_K, n_embd, n_kv * hd), "wv": (Q4_K, n_embd, n_kv * hd),
              "wo": (Q4_K, n_embd, n_embd), "w_gate": (Q4_K, n_embd, n_ff), "w_up": (Q4_K, n_embd, n_ff),
              "w_down": (Q6_K, n_ff, n_embd)}
    # two distinct byte patterns per matrix kind, alternating over layers; one device copy per layer
    raws = {k: [helpers.synth_weights(t, i, o, seed + 17 * n + j) for j in range(2)]
            for n, (k, (t, i, o)) in enumerate(shapes.items())}
    out_raw = helpers.synth_weights(Q6_K, n_embd, n_vocab, seed + 999)
    norms = [(1 + 0.05 * rng.standard_normal(n_embd)).astype(np.float32) for _ in range(2 * n_layer + 1)]
    mats = {}

    def up(key):  # key = (kind, layer) or "output"
        if key not in mats:
            if key == "output":
                mats[key] = be.upload_raw(out_raw, Q6_K, n_embd, n_vocab)
            else:
                t, i, o = shapes[key[0]]
                mats[key] = be.upload_raw(raws[key[0]][key[1] % 2], t, i, o)
        return mats[key]

    layers = [{**{k: (k, l) for k in shapes}, "attn_norm": norms[2 * l], "ffn_norm": norms[2 * l + 1]}
              for l in range(n_layer)]
    dec = LlamaDecoder(be, n_embd=n_embd, n_head=n_head, n_head_kv=n_kv, head_dim=hd, n_ff=n_ff, n_vocab=n_vocab,
                       max_ctx=ctx + max(16, warmup + 2 * steps + 2), rms_eps=1e-5, rope_freq_base=500000.0, layers=layers,
                       output_norm=norms[-1], output="output", upload=up)
    kvs = []
    for l in range(n_layer):
        k = rng.standard_normal((ctx, n_kv * hd)).astype(np.float32)
        v = rng.standard_normal((ctx, n_kv * hd)).astype(np.float32)
        dec.kv_write(l, 0, k, v)
        if check and l < 2:
            kvs.append((k, v))
    if only_prefill:   # for profiles: nothing but prompts of this length (one warm-up, three timed)
        prompt = rng.integers(0, n_vocab, only_prefill).astype(np.uint32)
        dec.prefill_tokens(up("output"), prompt, 0)
        t0 = time.perf_counter()
        for _ in range(3):
            dec.prefill_tokens(up("output"), prompt, 0)
        dt_pre = (time.perf_counter() - t0) / 3
        dec.close()
        for h in mats.values():
            be.free_weight(h)
        return {"workload": f"configs[4] model, prefill of {only_prefill} tokens from an empty cache",
                "prefill_ms": round(dt_pre * 1e3, 2), "prefill_tok_per_s": round(only_prefill / dt_pre, 1)}
    if only_verify:    # for profiles: nothing but verify batches of this size appended at position `ctx`
        xv = rng.standard_normal((only_verify, n_embd)).astype(np.float32)
        dec.forward_all_logits(xv, ctx, want_logits=False)
        t0 = time.perf_counter()
        for _ in range(10):
            dec.forward_all_logits(xv, ctx, want_logits=False)
        dt_v = (time.perf_counter() - t0) / 10
        dec.close()
        for h in mats.values():
            be.free_weight(h)
        return {"workload": f"configs[4] model, verify batch of {only_verify} tokens at context {ctx}",
                "ms": round(dt_v * 1e3, 3), "tokens_verified_per_s": round(only_verify / dt_v, 1)}
    x_h = rng.standard_normal(n_embd).astype(np.float32)
    x_d = hiprt.DeviceBuffer.from_numpy(x_h)
    tok_d = hiprt.DeviceBuffer(4)
    stream = hiprt.Stream()
    pos = ctx
    if attn_timeline:
        # A variant of the library built with -DOGM_ATTN_STAMPS=1 (`--lib`): the wall-clock stamps of the last
        # layer's attention launch of each of `steps` decode steps, phase by phase, medians over steps.
        # (the launcher's rule for the chunks of 128 positions a workgroup takes in a row: ogm_launch_attn_decode)
        n_chunks = ctx // 128 + 1
        sub = attn_chunks_per_wg or max(-(-n_chunks * n_kv // 264), 2 if n_chunks * n_kv >= 256 else 1)
        n_wg = n_kv * -(-n_chunks // min(sub, n_chunks))
        phases = ["start -> q rotated, new K/V row written", "scores of the chunk", "weighted V sum",
                  "partial results stored and acknowledged", "ticket drawn",
                  "merging workgroup: chunks merged", "merging workgroup: row quantized"]
        if min(sub, n_chunks) > 1:
            phases[1:3] = ["the workgroup's chunks, one after the other", "its waves' results joined"]
        rows = {k: [] for k in phases}
        spans = []
        for i in range(warmup + steps):
            dec.decode_dev(x_d.ptr, pos, 0, tok_d.ptr, stream.ptr)
            stream.synchronize()
            st = dec.attn_stamps(n_wg).astype(np.int64)
            pos += 1
            if i < warmup:
                continue
            d = np.diff(st, axis=1) * 10.0 / 1e3          # 100 MHz ticks -> us
            merging = (st[:, 6] > st[:, 5]) & (st[:, 7] >= st[:, 6])   # (stamps of an earlier layer's merge are older)
            for j, k in enumerate(phases):
                sel = d[:, j] if j < 5 else d[merging, j]
                rows[k].append(float(np.median(sel)))
            spans.append((max(st[:, 5].max(), st[merging, 7].max()) - st[:, 0].min()) * 10.0 / 1e3)
        dec.close()
        for h in mats.values():
            be.free_weight(h)
        return {"workload": f"attention kernel of a decode step at context {ctx}: {n_wg} workgroups of "
                            f"{min(sub, n_chunks)} chunks, 100 MHz stamps, "
                            f"median over workgroups, then over {steps} steps",
                "us": {k: round(float(np.median(v)), 2) for k, v in rows.items()},
                "first start -> last end": round(float(np.median(spans)), 2)}
    for _ in range(warmup):
        dec.decode_dev(x_d.ptr, pos, 0, tok_d.ptr, stream.ptr)
        pos += 1
    stream.synchronize()
    hiprt.device_synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        dec.decode_dev(x_d.ptr, pos, 0, tok_d.ptr, stream.ptr)
        pos += 1
    stream.synchronize()
    hiprt.device_synchronize()
    dt = (time.perf_counter() - t0) / steps
    # the closed loop: each token's embedding row (tied to the output matrix) is read on the device
    # from the previous step's argmax; one synchronization after `steps` tokens
    t0 = time.perf_counter()
    toks = dec.generate(up("output"), 1, pos, steps)
    dt_gen = (time.perf_counter() - t0) / steps
    pos += steps
    # speculative-decode verify (generate.rs:1618-1674): the last accepted token plus a draft of 3 or 7 go
    # through the whole model as one batch appended at position `ctx`; host embedding rows in, and out
    # (a) the greedy token of EVERY position (ogm_llama_forward_all_logits: what the verify step compares the
    # draft with; the logits of all positions stay on the device), (b) the last position's logits alone
    # (ogm_llama_prefill).  Wall clock per call, the first call of a size untimed.
    verify = {}
    for n_v in (4, 8):
        xv = rng.standard_normal((n_v, n_embd)).astype(np.float32)
        reps_v = max(3, min(20, steps // 10))
        row = {"calls": reps_v}
        for key, call in (("all_positions", lambda: dec.forward_all_logits(xv, ctx, want_logits=False)),
                          ("last_position", lambda: dec.prefill(xv, ctx))):
            call()
            t0 = time.perf_counter()
            for _ in range(reps_v):
                call()
            dt_v = (time.perf_counter() - t0) / reps_v
            row[key] = {"ms": round(dt_v * 1e3, 3), "tokens_verified_per_s": round(n_v / dt_v, 1)}
        row["ms"] = row["all_positions"]["ms"]
        row["tokens_verified_per_s"] = row["all_positions"]["tokens_verified_per_s"]
        verify[f"verify_batch_{n_v}"] = row
    # prefill of a 512-token prompt from position 0 (GEMM matmuls, batch attention); the first
    # call allocates the batch buffers
    dt_pre = dt_pre_long = dt_pre_long_one = None
    if with_prefill:
        prompt = rng.integers(0, n_vocab, 512).astype(np.uint32)
        dec.prefill_tokens(up("output"), prompt, 0)
        t0 = time.perf_counter()
        for _ in range(3):
            dec.prefill_tokens(up("output"), prompt, 0)
        dt_pre = (time.perf_counter() - t0) / 3
        long_prompt = rng.integers(0, n_vocab, 2048).astype(np.uint32)
        dec.prefill_tokens(up("output"), long_prompt, 0)
        t0 = time.perf_counter()
        dec.prefill_tokens(up("output"), long_prompt, 0)
        dt_pre_long = time.perf_counter() - t0
        # the same 2048-token prompt with the Q4_K GEMMs' min pass folded into the super-block step (an option,
        # off by default: f32 results not the reference's bits)
        be.set_tuning("gemm_one_pass", 1)
        try:
            dec.prefill_tokens(up("output"), long_prompt, 0)
            t0 = time.perf_counter()
            dec.prefill_tokens(up("output"), long_prompt, 0)
            dt_pre_long_one = time.perf_counter() - t0
        finally:
            be.set_tuning("gemm_one_pass", 0)
    weights = n_layer * sum(o * (i // 256) * (144 if t == Q4_K else 210) for t, i, o in shapes.values()) \
        + n_vocab * (n_embd // 256) * 210
    kv_bytes = 2 * n_layer * ctx * n_kv * hd * 2
    what = "configs[4]: 8B-shaped Llama Q4_K_M-like" if model == "8b" else \
        f"{n_layer} of the {n_layer_model} layers of a {model.upper()}-shaped Llama Q4_K_M-like (and its output matrix)"
    res = {"workload": f"{what}, batch-1 greedy decode at context {ctx}",
           "tok_per_s": round(1.0 / dt, 1), "ms_per_token": round(dt * 1e3, 4),
           "generate_tok_per_s": round(1.0 / dt_gen, 1), "generated": [int(t) for t in toks[:4]],
           "prefill_512_ms": round(dt_pre * 1e3, 2) if dt_pre else None,
           "prefill_tok_per_s": round(512 / dt_pre, 1) if dt_pre else None,
           "prefill_2048_ms": round(dt_pre_long * 1e3, 2) if dt_pre_long else None,
           "prefill_2048_tok_per_s": round(2048 / dt_pre_long, 1) if dt_pre_long else None,
           "prefill_2048_ms_one_pass_option": round(dt_pre_long_one * 1e3, 2) if dt_pre_long_one else None,
           **verify,
           "bytes_per_token": weights + kv_bytes,
           "GBps": round((weights + kv_bytes) / dt / 1e9, 1),
           "frac_of_hbm_peak": round((weights + kv_bytes) / dt / 1e9 / HBM_PEAK_GBS, 4)}
    if check:
        # the same two-layer prefix of the model on the CPU restatement, same cache rows, one token
        from oracle import llama_ref as R
        small = LlamaDecoder(be, n_embd=n_embd, n_head=n_head, n_head_kv=n_kv, head_dim=hd, n_ff=n_ff,
                             n_vocab=n_vocab, max_ctx=ctx + 1, rms_eps=1e-5, rope_freq_base=500000.0,
                             layers=layers[:2], output_norm=norms[-1], output="output", upload=up)
        ref_layers = []
        for l in range(2):
            w = {k: (shapes[k][0], raws[k][l % 2], shapes[k][1], shapes[k][2]) for k in shapes}
            ref_layers.append(R.Layer(w["wq"], w["wk"], w["wv"], w["wo"], w["w_gate"], w["w_up"], w["w_down"],
                                      norms[2 * l], norms[2 * l + 1]))
        ref = R.Model(n_embd, n_head, n_kv, hd, n_ff, n_vocab, hd, 1e-5, 500000.0, ref_layers, norms[-1],
                      (Q6_K, out_raw, n_embd, n_vocab))
        ref.reset()
        for l, (k, v) in enumerate(kvs):
            small.kv_write(l, 0, k, v)
            ref.k_cache[l] = list(k.astype(np.float16))
            ref.v_cache[l] = list(v.astype(np.float16))
        want, _ = R.decode_step(ref, x_h, ctx)
        got, tok = small.decode(x_h, ctx)
        err = float(np.abs(got.astype(np.float64) - want).max() / (np.abs(want).max() + 1e-30))
        res["parity_vs_cpu"] = {"layers_checked": 2, "max_logit_error_over_max_logit": err,
                                "greedy_token_equal": bool(tok == R.argmax(want)), "ok": bool(err <= 2e-4)}
        small.close()
    dec.close()
    for h in mats.values():
        be.free_weight(h)
    return res


def trait_path(be, helpers, raw, shapes, x_h, h_h, copies: int, reps: int) -> dict:
    """What Backend::matmul really costs (backend/mod.rs:313, 362): host slices in, host slices out,
    through ogm_matmul / ogm_matmul_batch -- pinned staging, quantizer, GEMV, wait -- on weight copies
    that rotate like the headline's.  Wall clock per call, issued from compiled code
    (ogm_time_host_calls) as the reference's FFI would; and, for the record, from this interpreter,
    where a call costs about 5 us more."""
    from orangu_amd import MatmulOp, QuantMatrix
    mats = {k: [QuantMatrix(raw[k].copy(), Q4_K, *shapes[k]) for _ in range(copies)] for k in shapes}
    for k in mats:
        for m in mats[k]:
            be.upload(m)

    def stat(variants, groups):
        be.time_host_calls(variants, groups, 30)
        ts = np.sort(be.time_host_calls(variants, groups, reps))
        return {"min": round(float(ts[0]), 2), "median": round(float(ts[len(ts) // 2]), 2),
                "p90": round(float(ts[len(ts) * 9 // 10]), 2), "calls": reps}

    gate = [[MatmulOp(x_h, 1, mats["gate"][c])] for c in range(copies)]
    down = [[MatmulOp(h_h, 1, mats["down"][c])] for c in range(copies)]
    pair = [[MatmulOp(x_h, 1, mats["gate"][c]), MatmulOp(x_h, 1, mats["up"][c])] for c in range(copies)]
    ffn = [[MatmulOp(x_h, 1, mats["gate"][c]), MatmulOp(x_h, 1, mats["up"][c]), MatmulOp(h_h, 1, mats["down"][c])]
           for c in range(copies)]
    rows = {
        "matmul 4096->14336": stat(gate, [1]),
        "matmul 14336->4096": stat(down, [1]),
        "matmul_batch {gate, up}": stat(pair, [2]),
        "FFN block: matmul_batch {gate, up} + matmul down": stat(ffn, [2, 1]),
    }
    ts = []
    for i in range(reps + 20):
        a = time.perf_counter()
        be.matmul(x_h, 1, mats["gate"][i % copies])
        ts.append((time.perf_counter() - a) * 1e6)
    ts = sorted(ts[20:])
    rows["matmul 4096->14336 called from Python"] = {"min": round(ts[0], 2), "median": round(ts[len(ts) // 2], 2),
                                                     "calls": reps}
    for k in mats:
        for m in mats[k]:
            be.evict(m)
    return {"unit": "us per call, wall clock, host pointers in and out; calls issued by ogm_time_host_calls "
                    "(compiled code) unless the row says otherwise", "rows": rows}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--copies", type=int, default=12,
                    help="distinct copies of the three matrices (12 x 99 MB = 1.2 GB > 256 MB cache)")
    ap.add_argument("--roofline-launches", type=int, default=1200)
    ap.add_argument("--roofline-batch", type=int, default=100,
                    help="back-to-back launches between two HIP events (the event records leave a gap of their own)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU baseline budget; 0 skips it")
    ap.add_argument("--wg-waves", type=int, default=0, help="waves per workgroup override (0 = heuristic)")
    ap.add_argument("--separate", action="store_true",
                    help="issue gate and up as two calls instead of one grouped call")
    ap.add_argument("--gemm-tokens", type=int, default=512,
                    help="tokens of the prefill GEMM leg (Q4_K 4096 -> 14336 on MFMA); 0 skips it")
    ap.add_argument("--only-gemm", action="store_true", help="run only the prefill GEMM leg (for rocprofv3)")
    ap.add_argument("--gemm-one-pass", action="store_true",
                    help="with --only-gemm: the one-pass option of the large-grid kernel (tuning key gemm_one_pass)")
    ap.add_argument("--decode-steps", type=int, default=64,
                    help="tokens of the 8B-shaped decode leg (config 5); 0 skips it")
    ap.add_argument("--decode-ctx", type=int, default=2048, help="cached positions of the decode leg")
    ap.add_argument("--decode-model", choices=sorted(DECODE_MODELS), default="8b",
                    help="with --only-decode: the model whose layer shapes are decoded (405b: give --decode-layers too)")
    ap.add_argument("--decode-layers", type=int, default=0,
                    help="with --only-decode: run this many layers of the model instead of all of them")
    ap.add_argument("--only-decode", action="store_true", help="run only the decode leg (for rocprofv3)")
    ap.add_argument("--attn-timeline", action="store_true",
                    help="with --lib of a variant built with -DOGM_ATTN_STAMPS=1: the decode attention kernel's phases")
    ap.add_argument("--only-verify", type=int, default=0, metavar="N",
                    help="run only verify batches of N tokens at the decode context (for rocprofv3)")
    ap.add_argument("--only-prefill", type=int, default=0, metavar="N",
                    help="run only prefills of N tokens on the decode leg's model (for rocprofv3)")
    ap.add_argument("--tune", action="append", default=[], metavar="KEY=VALUE",
                    help="a kernel choice of ogm_set_tuning for this run (repeatable), e.g. gemm_small_max_tokens=1")
    ap.add_argument("--sweep", action="store_true",
                    help="time every benchmark configuration's kernels instead (one JSON object, not the "
                         "headline line)")
    ap.add_argument("--only-row", default="", metavar="TEXT",
                    help="with --sweep: only the rows whose label contains TEXT (for rocprofv3), e.g. 'C3 vocab batch 1'")
    ap.add_argument("--no-sweep", action="store_true", help="leave the sweep rows out of the headline line")
    ap.add_argument("--no-trait", action="store_true", help="leave the host-pointer rows out of the headline line")
    ap.add_argument("--only-roofline", action="store_true",
                    help="run only the dominant-kernel leg (for rocprofv3 --kernel-trace --stats)")
    ap.add_argument("--only-stream", action="store_true",
                    help="run only the read-only launch over gate+up's bytes (the measured peak; for rocprofv3)")
    ap.add_argument("--only-single", default="", choices=["", "gate", "down"],
                    help="run only the single-matrix GEMV launches of this shape (for rocprofv3)")
    ap.add_argument("--legs", default="", metavar="NAME[,NAME]",
                    help="run only these legs of the dominant-kernel section (for rocprofv3): gate+up, read probe, "
                         "gate alone, down, read probe one matrix, empty launch 1, empty launch 1792, quantize 4096")
    ap.add_argument("--trace-summary", default="", metavar="PATH",
                    help="no GPU work: condense a rocprofv3 kernel trace (csv file or the folder it is under) "
                         "into per-kernel durations and span per dispatch, as JSON")
    ap.add_argument("--trace-period", type=int, default=0, metavar="N",
                    help="with --trace-summary: also the mean duration by dispatch number modulo N (N = --copies "
                         "shows each weight copy of the rotation on its own)")
    ap.add_argument("--lib", default="", metavar="PATH",
                    help="load this build of the library instead of the in-tree one (a variant built by "
                         "`python3 orangu_amd/build.py --define ... --out PATH` with a kernel's timing switch set)")
    args = ap.parse_args()
    if args.lib:
        from orangu_amd import capi
        capi.LIB_PATH = os.path.abspath(args.lib)
    if args.trace_summary:
        print(json.dumps(trace_summary(args.trace_summary, args.trace_period), indent=1))
        return 0

    if args.gpus != 1:
        print("bench.py: this build measures one GPU only; --gpus N with N > 1 is not supported "
              "(the path has no collectives).", file=sys.stderr)
        return 2

    import helpers
    from orangu_amd import Mi355xBackend
    from orangu_amd import hiprt

    be = Mi355xBackend()  # raises without the HIP library or a gfx950 device
    for kv in args.tune:
        key, _, value = kv.partition("=")
        be.set_tuning(key, int(value))
    if args.sweep:
        print(json.dumps(sweep(be, helpers, hiprt, only=args.only_row)))
        be.close()
        return 0
    if args.only_prefill:
        print(json.dumps(decode_leg(be, helpers, hiprt, 1, 0, max(args.decode_ctx, args.only_prefill), False,
                                    only_prefill=args.only_prefill)))
        be.close()
        return 0
    if args.attn_timeline:
        chunks_per_wg = max([int(kv.partition("=")[2]) for kv in args.tune if kv.startswith("attn_decode_chunks=")] + [0])
        print(json.dumps(decode_leg(be, helpers, hiprt, 16, 4, args.decode_ctx, False, attn_timeline=True,
                                    attn_chunks_per_wg=chunks_per_wg)))
        be.close()
        return 0
    if args.only_verify:
        print(json.dumps(decode_leg(be, helpers, hiprt, 1, 0, args.decode_ctx, False, only_verify=args.only_verify)))
        be.close()
        return 0
    if args.only_decode:
        print(json.dumps(decode_leg(be, helpers, hiprt, max(1, args.decode_steps), 8, args.decode_ctx, False,
                                    with_prefill=False, model=args.decode_model, layers_run=args.decode_layers)))
        be.close()
        return 0
    if args.wg_waves:
        be.set_tuning("gemv_wg_waves", args.wg_waves)
    stream = hiprt.Stream()
    only_leg = args.only_roofline or args.only_gemm or args.only_stream or bool(args.only_single) or bool(args.legs)

    # ---- synthetic inputs -------------------------------------------------------------------
    seed = 20240607
    shapes = {"gate": (HIDDEN, FFN), "up": (HIDDEN, FFN), "down": (FFN, HIDDEN)}
    raw = {k: helpers.synth_weights(Q4_K, i, o, seed + n) for n, (k, (i, o)) in enumerate(shapes.items())}
    x_h = helpers.synth_x(1, HIDDEN, seed)[0]
    h_h = helpers.synth_x(1, FFN, seed + 1)[0]
    copies = max(1, args.copies)
    handles = {k: [be.upload_raw(raw[k], Q4_K, *shapes[k]) for _ in range(copies)] for k in shapes}
    x_d = hiprt.DeviceBuffer.from_numpy(x_h)
    h_d = hiprt.DeviceBuffer.from_numpy(h_h)
    y_gate, y_up, y_down = (hiprt.DeviceBuffer(4 * FFN), hiprt.DeviceBuffer(4 * FFN),
                            hiprt.DeviceBuffer(4 * HIDDEN))

    def step(i: int):
        # gate and up read the same input and go out as one call, as the forward pass batches
        # them (engine/arch/mod.rs:1082-1096); down follows on its own input.
        c = i % copies
        if args.separate:
            be.matmul_dev(handles["gate"][c], x_d.ptr, 1, y_gate.ptr, False, stream.ptr)
            be.matmul_dev(handles["up"][c], x_d.ptr, 1, y_up.ptr, False, stream.ptr)
        else:
            be.matmul_multi_dev([handles["gate"][c], handles["up"][c]], x_d.ptr, 1,
                                [y_gate.ptr, y_up.ptr], False, stream.ptr)
        be.matmul_dev(handles["down"][c], h_d.ptr, 1, y_down.ptr, False, stream.ptr)

    step_bytes = 2 * gemv_bytes(HIDDEN, FFN) + gemv_bytes(FFN, HIDDEN)
    result = {}
    step_stats = None

    if not only_leg:
        def timed_steps(k0: int, n: int) -> float:
            stream.synchronize()
            hiprt.device_synchronize()
            t0 = time.perf_counter()
            for i in range(n):
                step(k0 + i)
            stream.synchronize()
            hiprt.device_synchronize()
            return (time.perf_counter() - t0) * 1e3 / n

        for i in range(args.warmup):
            step(i)
        # the headline: exactly --steps steps between two synchronizations
        ms_per_step = timed_steps(args.warmup, args.steps)
        result["ms_per_step"] = ms_per_step
        result["value"] = step_bytes / (ms_per_step * 1e-3) / 1e9
        # the same region again, until at least 200 (and at least four times --steps) further steps have
        # run: how much one such region varies
        reps = [ms_per_step]
        extra = max(4, -(-200 // max(1, args.steps)))
        for r in range(extra):
            reps.append(timed_steps(args.warmup + (r + 1) * args.steps, args.steps))
        reps_sorted = sorted(reps)
        step_stats = {"regions": len(reps), "steps_each": args.steps,
                      "ms_per_step_min": round(reps_sorted[0], 5),
                      "ms_per_step_median": round(reps_sorted[len(reps) // 2], 5),
                      "ms_per_step_max": round(reps_sorted[-1], 5),
                      "GBps_median": round(step_bytes / (reps_sorted[len(reps) // 2] * 1e-3) / 1e9, 1)}

    # ---- dominant kernel: the Q4_K GEMV over gate+up (4096 -> 2 x 14336 in one launch), ---------
    # back-to-back over pre-quantized activations, HIP events on its stream, in batches
    n_launch = max(40, args.roofline_launches)
    per_batch = max(1, args.roofline_batch)
    batches = max(3, n_launch // per_batch)
    kbytes = 2 * gemv_bytes(HIDDEN, FFN) - 4 * HIDDEN  # both matrices read the same x
    weight_bytes2 = 2 * FFN * (HIDDEN // 256 * 144)
    roofline = None
    kernel_name = ""
    us_per_launch = 0.0
    achieved = 0.0
    if not args.only_gemm:
        be.act_quantize_dev(Q4_K, x_d.ptr, HIDDEN, 1, stream.ptr)
        legs = {}
        # which legs run: all of them in the headline run, a named subset under a profiler
        all_legs = ["gate+up", "read probe", "gate alone", "down", "read probe one matrix", "empty launch 1",
                    "empty launch 1792", "quantize 4096"]
        if args.legs:
            want = [l.strip() for l in args.legs.split(",") if l.strip()]
            bad = [l for l in want if l not in all_legs]
            if bad:
                raise SystemExit(f"--legs: unknown {bad}; known: {all_legs}")
        elif args.only_roofline:
            want = ["gate+up"]
        elif args.only_stream:
            want = ["read probe"]
        elif args.only_single:
            want = ["gate alone" if args.only_single == "gate" else "down"]
        else:
            want = all_legs
        mats = handles["gate"] + handles["up"]

        def timed(name, launch=None, many=None):
            if name in want:
                legs[name] = batched_us(hiprt, stream, launch, batches, per_batch, warm=50, many=many)

        # The launches of these legs are enqueued from compiled code (ogm_enqueue_repeated): the interpreter's
        # own time per call would otherwise show as idle gaps between kernels this short -- under rocprofv3,
        # whose hooks add to every call, gaps of 2 us between 12 us kernels.
        pair_sets = [[handles["gate"][c], handles["up"][c]] for c in range(copies)]
        single_sets = [[h] for h in mats]
        timed("gate+up", many=lambda i, n: be.enqueue_repeated(0, pair_sets, 1, [y_gate.ptr, y_up.ptr], i % copies, n,
                                                               False, stream.ptr))
        if "gate+up" in legs:
            kernel_name = be.last_kernel()
        # the yardstick: the same bytes through a launch that only reads them
        timed("read probe", many=lambda i, n: be.enqueue_repeated(1, pair_sets, 1, [], i % copies, n, False, stream.ptr))
        timed("gate alone", many=lambda i, n: be.enqueue_repeated(0, single_sets, 1, [y_gate.ptr], i % len(mats), n,
                                                                  False, stream.ptr))
        if "down" in want:
            be.act_quantize_dev(Q4_K, h_d.ptr, FFN, 1, stream.ptr)
            timed("down", many=lambda i, n: be.enqueue_repeated(0, [[h] for h in handles["down"]], 1, [y_down.ptr],
                                                                i % copies, n, False, stream.ptr))
        # one matrix's bytes through the read-only launch: what a launch of 33 MB can reach at all
        timed("read probe one matrix", many=lambda i, n: be.enqueue_repeated(1, single_sets, 1, [], i % len(mats), n,
                                                                             False, stream.ptr))
        # launches that do nothing, one workgroup wide and as wide as the gate+up GEMV (1792 workgroups of 256
        # threads): the kernel boundary, host and device side together, back to back on one stream
        timed("empty launch 1", many=lambda i, n: be.enqueue_repeated(2, [], 1, [], 0, n, False, stream.ptr))
        timed("empty launch 1792", many=lambda i, n: be.enqueue_repeated(2, [], 1792, [], 0, n, False, stream.ptr))
        timed("quantize 4096", lambda i: be.act_quantize_dev(Q4_K, x_d.ptr, HIDDEN, 1, stream.ptr))
        if args.only_roofline or args.only_stream or args.legs:
            # One plain device-to-device copy of known size: under `rocprofv3 --pmc FETCH_SIZE` /
            # `WRITE_SIZE` its counter reading calibrates the kernel's (bytes per counter unit).
            cal = 64 << 20
            src, dst = hiprt.DeviceBuffer(cal), hiprt.DeviceBuffer(cal)
            src.fill(1)
            hiprt.check(hiprt.hip().hipMemcpy(dst.ptr, src.ptr, cal, 3), "hipMemcpy D2D")
            hiprt.device_synchronize()
        main_leg = legs.get("gate+up") or legs.get("read probe") or next(iter(legs.values()))
        us_per_launch = main_leg["median"]
        achieved = kbytes / (us_per_launch * 1e-6) / 1e9
        one = gemv_bytes(HIDDEN, FFN)
        per_leg_bytes = {"gate+up": kbytes, "read probe": weight_bytes2, "gate alone": one,
                         "down": gemv_bytes(FFN, HIDDEN), "read probe one matrix": weight_bytes2 // 2,
                         "empty launch 1": 0, "empty launch 1792": 0, "quantize 4096": 4 * HIDDEN + HIDDEN + 64}
        roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": GEMV_Q4K_GATE_UP_TRAFFIC,
                    "traffic_source": "rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE on `bench.py --only-roofline`, "
                                      "each scaled by the same counter's reading for that run's 64 MiB copy "
                                      "(profiles/gemv_q4k_gate_up_4096x14336_hbm_counters.md)",
                    "rocprof_avg_us": GEMV_Q4K_GATE_UP_ROCPROF["avg_us"],
                    "rocprof_median_us": GEMV_Q4K_GATE_UP_ROCPROF["median_us"],
                    "rocprof_back_to_back_avg_us": GEMV_Q4K_GATE_UP_ROCPROF["back_to_back_avg_us"],
                    "rocprof_frac": round(kbytes / GEMV_Q4K_GATE_UP_ROCPROF["avg_us"] / 1e3 / HBM_PEAK_GBS, 4),
                    "rocprof_source": "rocprofv3 --kernel-trace --stats on `bench.py --only-roofline`, "
                                      f"{GEMV_Q4K_GATE_UP_ROCPROF['dispatches']} dispatches, condensed by `bench.py "
                                      "--trace-summary` (profiles/gemv_q4k_gate_up_4096x14336_kernel_trace.md); "
                                      "us_per_launch beside it is measured live in this run",
                    "kernel": (kernel_name or "(not run)") + " over gate+up", "us_per_launch": us_per_launch,
                    "us_per_launch_min": main_leg["min"], "bytes_per_launch": kbytes,
                    "launches": main_leg["launches"],
                    "timing": f"HIP events on the launch stream round {batches} batches of {per_batch} back-to-back "
                              "launches enqueued from compiled code; median batch (achieved, frac) and fastest batch",
                    "legs_us": {k: {**v, "GBps_median": round(per_leg_bytes[k] / v["median"] / 1e3, 1)}
                                for k, v in legs.items()}}
        if "read probe" in legs and "gate+up" in legs:
            peak_meas = weight_bytes2 / legs["read probe"]["median"] / 1e3
            roofline["measured_peak"] = {
                "GBps": round(peak_meas, 1), "us": legs["read probe"]["median"], "bytes": weight_bytes2,
                "what": "one launch that only reads gate+up's device bytes with the GEMV's non-temporal loads "
                        "(ogm_weights_read_probe), same rotation over weight copies",
                "frac_of_measured": round(achieved / peak_meas, 4)}

    # ---- prefill GEMM on MFMA: Q4_K 4096 -> 14336 at --gemm-tokens tokens (quantize + operand staging
    # + GEMM kernel per call), checked against the CPU path on a sample of rows
    gemm = None
    if args.gemm_tokens > 0 and (not only_leg or args.only_gemm):
        T = args.gemm_tokens
        xg_h = helpers.synth_x(T, HIDDEN, seed + 7)
        xg = hiprt.DeviceBuffer.from_numpy(xg_h)
        yg = hiprt.DeviceBuffer(4 * T * FFN)
        st_g = None
        if args.only_gemm:
            be.set_tuning("gemm_one_pass", 1 if args.gemm_one_pass else 0)
            for i in range(5):
                be.matmul_dev(handles["gate"][i % copies], xg.ptr, T, yg.ptr, False, stream.ptr)
            stream.synchronize()
        else:
            st_g = batched_us(hiprt, stream, lambda i: be.matmul_dev(handles["gate"][i % copies], xg.ptr, T, yg.ptr,
                                                                     False, stream.ptr), 10, 10, warm=GEMM_WARM)
        gemm_kernel = be.last_kernel()
        gemm = {"workload": f"Q4_K 4096->14336, {T} tokens (config a14 shape)", "kernel": gemm_kernel,
                "warm_up_calls": GEMM_WARM}
        if st_g is not None:
            flops = 2.0 * T * HIDDEN * FFN
            us_gemm = st_g["median"]
            # the kernel multiplies int8 operands (v_mfma_i32_32x32x32_i8): priced against the dense
            # int8 peak of 5.0 POP/s (against the 2.5 PFLOP/s f16 peak it would read twice as high)
            gemm.update({"us_per_matmul": round(us_gemm, 1), "us_per_matmul_min": round(st_g["min"], 1),
                         "calls": st_g["launches"], "tops": round(flops / us_gemm / 1e6, 1),
                         "mfma_type": "i8", "frac_of_int8_mfma_peak": round(flops / us_gemm / 1e6 / 5000.0, 4)})
            # the same call with the reference's separate min pass folded into the super-block step: an option,
            # off by default, whose f32 results are not the reference's bits (same integer sums)
            be.set_tuning("gemm_one_pass", 1)
            try:
                st_o = batched_us(hiprt, stream, lambda i: be.matmul_dev(handles["gate"][i % copies], xg.ptr, T,
                                                                         yg.ptr, False, stream.ptr), 10, 10, warm=GEMM_WARM)
                gemm["one_pass_option"] = {"kernel": be.last_kernel(), "us_per_matmul": round(st_o["median"], 1),
                                           "tops": round(flops / st_o["median"] / 1e6, 1),
                                           "parity": "integer sums exact; f32 within 1e-3 * sum|w x| of the "
                                                     "reference order, not its bits"}
            finally:
                be.set_tuning("gemm_one_pass", 0)
            be.matmul_dev(handles["gate"][0], xg.ptr, T, yg.ptr, False, stream.ptr)   # what the parity check reads
            stream.synchronize()
        if not args.only_gemm and args.cpu_seconds > 0:
            import oracle
            rows = np.r_[0:32, 7000:7032, FFN - 32:FFN]
            rb = HIDDEN // 256 * 144
            sub = np.concatenate([raw["gate"][r * rb:(r + 1) * rb] for r in rows])
            want = oracle.matmul(Q4_K, sub, HIDDEN, rows.size, xg_h, T).reshape(T, rows.size)
            got = yg.to_numpy(np.float32, T * FFN).reshape(T, FFN)[:, rows]
            gemm["parity_vs_cpu"] = "bit-exact" if np.array_equal(got.view(np.uint32), want.view(np.uint32)) \
                else ("within 1e-3/1e-5" if np.all(np.abs(got - want) <= 1e-3 * np.abs(want) + 1e-5) else "FAILED")
        xg.free()
        yg.free()

    # ---- parity of what was just timed + CPU baseline (the oracle, all host cores) -------------
    cpu = None
    parity = None
    if not only_leg and args.cpu_seconds > 0:
        import oracle
        step(0)
        stream.synchronize()
        got = {"gate": y_gate.to_numpy(np.float32, FFN), "up": y_up.to_numpy(np.float32, FFN),
               "down": y_down.to_numpy(np.float32, HIDDEN)}
        xin = {"gate": x_h, "up": x_h, "down": h_h}
        cores = oracle.host_threads()

        def cpu_step():
            return {k: oracle.matmul(Q4_K, raw[k], shapes[k][0], shapes[k][1], xin[k], 1, threads=0)[0]
                    for k in shapes}

        want = cpu_step()  # warm-up and the parity reference
        ok = all(np.all(np.abs(got[k].astype(np.float64) - want[k]) <= 1e-3 * np.abs(want[k]) + 1e-5)
                 for k in shapes)
        bits = all(np.array_equal(got[k].view(np.uint32), want[k].view(np.uint32)) for k in shapes)
        parity = "bit-exact" if bits else ("within 1e-3/1e-5" if ok else "FAILED")
        times = []
        t_end = time.perf_counter() + args.cpu_seconds
        while time.perf_counter() < t_end or len(times) < 5:
            a = time.perf_counter()
            cpu_step()
            times.append(time.perf_counter() - a)
        best, med = min(times), sorted(times)[len(times) // 2]
        # one thread, a few repetitions of one GEMV, scaled to the step
        t1s = []
        for _ in range(3):
            a = time.perf_counter()
            oracle.matmul(Q4_K, raw["gate"], HIDDEN, FFN, x_h, 1, threads=1)
            t1s.append(time.perf_counter() - a)
        cpu = {"value": round(step_bytes / med / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
               "sample": f"{len(times)} repetitions of the same 3-GEMV step ({step_bytes} B each), "
                         f"median; best {step_bytes / best / 1e9:.2f} GB/s; "
                         f"1 thread {gemv_bytes(HIDDEN, FFN) / min(t1s) / 1e9:.2f} GB/s; "
                         f"integer dots on {oracle.isa_name()}"}
        if parity == "FAILED":
            print("bench.py: GPU output differs from the CPU oracle beyond 1e-3/1e-5", file=sys.stderr)

    trait = None
    if not only_leg and not args.no_trait:
        trait = trait_path(be, helpers, raw, shapes, x_h, h_h, min(copies, 6), 200)

    for k in handles:          # make room: the legs below bring their own weights
        for h in handles[k]:
            be.free_weight(h)
    sweep_rows = None
    if not only_leg and not args.no_sweep:
        sweep_rows = sweep(be, helpers, hiprt, light=True)

    decode = None
    if args.decode_steps > 0 and not only_leg:
        decode = decode_leg(be, helpers, hiprt, args.decode_steps, 8, args.decode_ctx, args.cpu_seconds > 0)

    out = {
        "metric": "Q4_K GEMV HBM GB/s (batch-1 decode, Llama-3-8B FFN shapes)",
        "value": round(result.get("value", achieved), 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps if not only_leg else n_launch,
        "warmup": args.warmup,
        "ms_per_step": round(result.get("ms_per_step", us_per_launch * 1e-3), 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "i8 dot / i32 block sums / f32 combine",
        "data": "synthetic",
        "config": {"workload": "configs[1]: Q4_K decode GEMV batch 1, gate+up 4096->14336 and down "
                               "14336->4096; step = quantize(x) + GEMV over gate and up in one launch + "
                               "quantize(h) + GEMV down",
                   "algorithmic_bytes_per_step": step_bytes, "weight_copies": copies,
                   "frac_of_hbm_peak": round(result.get("value", achieved) / HBM_PEAK_GBS, 4),
                   "step_regions": step_stats,
                   "parity_vs_cpu": parity, "device": be.device_name()},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "prefill_gemm": gemm,
        "trait_path": trait,
        "sweep": sweep_rows,
        "decode": decode,
    }
    print(json.dumps(out))
    be.close()
    return 0 if parity != "FAILED" else 1


if __name__ == "__main__":
    sys.exit(main())
