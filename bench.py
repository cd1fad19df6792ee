#!/usr/bin/env python3
"""Benchmark of the batch-1 token-decode path on one MI355X.

Workload (default): Llama-2-7B shape (dim 4096, 32 layers, 32 heads, FFN 11008,
vocab 32000), weights seeded N(0, 0.02) quantized with the ggml reference
quantizers in a Q4_K_M-style mix (Q4_K; Q6_K for attn_v, output and the
ffn_down layers picked by use_more_bits), embedding f32, activations and KV
cache f32.  `--warmup` prompt tokens are pushed through the decoder one at a
time (untimed), then exactly `--steps` greedy decode steps are timed: one step =
one token = one pass over every weight.

Prints ONE JSON line: decode tok/s, the HBM roofline of the dominant kernel
(gemv_fused_kernel as launched for the gate/up projections: two Q4_K 11008x4096
matrices, RMSNorm folded into the staging of x, SiLU gating in the epilogue)
measured with HIP events on the library's own stream over the model's 32
layers, a GEMV sweep over the model's four matrix shapes for the three formats,
and the CPU baseline (the single-threaded C restatement of the reference's CPU
transformer) timed on this host on a bounded sample.

    python bench.py [--gpus 1] [--steps 256] [--warmup 128] [--model 7b|tiny]

Two further workloads print a JSON line of the same shape (no roofline / CPU
legs): `--model gpt2` (GPT-2 124M, every matrix Q8_0: a 32-token prompt, then
greedy tokens up to position 32 + steps) and `--model 8b-gqa` (Llama-3-8B shape
with grouped-query attention, every matrix Q6_K, KV caches filled with N(0,1)
up to position 8191: `--steps` decode steps from position 8192).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def gemv_bytes(qtype_bytes_per_matrix: int, nrows: int, ncols: int) -> int:
    """Algorithmic bytes of one GEMV: GGUF bytes of W + x (f32) + y (f32)."""
    return qtype_bytes_per_matrix + 4 * ncols + 4 * nrows


def time_gemv(W, gpu, mats, nrows, ncols, iters):
    """Average GPU duration (us) of out = M x over `iters` graph-recorded launches
    rotating through `mats` (distinct device copies, so nothing stays cached)."""
    from wgml_amd._lib import call

    out = W.GpuVector.uninit(gpu, nrows)
    x = W.GpuVector.init(gpu, W.rng_normal(99, ncols))
    arr = (C.c_void_p * len(mats))(*[m.handle for m in mats])
    ms = C.c_float()
    best = None
    for _ in range(3):
        call("wgml_bench_gemv_quant", gpu.handle, arr, len(mats), out.view(), x.view(), iters, 1,
             C.byref(ms))
        us = ms.value * 1e3 / iters
        best = us if best is None else min(best, us)
    return best


def time_gate_up(W, gpu, cfg, weights):
    """Average GPU duration (us) of the decoder's fused gate/up launch, back to back over
    every layer's own matrices (distinct memory, 1.6 GB in total), and its algorithmic bytes."""
    from wgml_amd._lib import View, call

    layers = weights.layers
    gate = [W.GpuQuantMatrix(gpu, l["ffn_gate"].qtype, cfg.hidden_dim, cfg.dim, l["ffn_gate"].data)
            for l in layers]
    up = [W.GpuQuantMatrix(gpu, l["ffn_up"].qtype, cfg.hidden_dim, cfg.dim, l["ffn_up"].data)
          for l in layers]
    n = len(layers)
    a = (C.c_void_p * n)(*[m.handle for m in gate])
    b = (C.c_void_p * n)(*[m.handle for m in up])
    modes = (C.c_int * 1)(2)
    out = W.GpuVector.uninit(gpu, cfg.hidden_dim)
    x = W.GpuVector.init(gpu, W.rng_normal(99, cfg.dim))
    nw = W.GpuVector.init(gpu, layers[0]["ffn_norm"])
    nwv = nw.view()
    ms = C.c_float()
    best = None
    iters = 4 * n
    for _ in range(3):
        call("wgml_bench_gemv_fused", gpu.handle, a, b, modes, 1, n, out.view(), cfg.hidden_dim,
             x.view(), C.byref(nwv), iters, C.byref(ms))
        us = ms.value * 1e3 / iters
        best = us if best is None else min(best, us)
    # W_gate + W_up (GGUF bytes) + x + norm weights (f32) in, hidden_dim f32 out
    nbytes = gate[0].gguf_bytes() + up[0].gguf_bytes() + 4 * cfg.dim * 2 + 4 * cfg.hidden_dim
    return best, nbytes


def gemv_sweep(W, gpu, nrows, ncols, min_total_bytes=640 << 20):
    """One matrix shape for Q8_0 / Q4_K / Q6_K: GB/s and fraction of HBM peak."""
    res = {}
    vals = W.rng_normal(4242, nrows * ncols, 0.0, 0.02)
    for qtype, name in ((W.Q8_0, "q8_0"), (W.Q4_K, "q4_k"), (W.Q6_K, "q6_k")):
        raw = W.quantize(qtype, vals)
        n_copies = max(2, -(-min_total_bytes // raw.nbytes))
        mats = [W.GpuQuantMatrix(gpu, qtype, nrows, ncols, raw) for _ in range(n_copies)]
        us = time_gemv(W, gpu, mats, nrows, ncols, iters=4 * n_copies)
        b = gemv_bytes(raw.nbytes, nrows, ncols)
        gbs = b / us * 1e-3
        res[name] = {"us": round(us, 3), "GB/s": round(gbs, 1), "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
                     "bytes": b, "copies": n_copies}
        log(f"  gemv {name} {nrows}x{ncols}: {us:.2f} us  {gbs:.0f} GB/s  "
            f"({100 * gbs / HBM_PEAK_GBS:.1f}% of HBM peak)")
        del mats
    return res


def cpu_baseline(weights, prompt, n_steps):
    """Times the CPU oracle (port of the reference's single-threaded CPU
    transformer, weights expanded to f32 at load as the reference does) on the
    first `n_steps` positions of the same model and prompt."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle as orc

    t0 = time.perf_counter()
    m = orc.Llama2(weights, predequantize=True)
    t_load = time.perf_counter() - t0
    t0 = time.perf_counter()
    for pos in range(n_steps):
        m.forward(int(prompt[pos]), pos)
    dt = time.perf_counter() - t0
    log(f"  cpu oracle: load (dequantize) {t_load:.1f}s, {n_steps} steps in {dt:.1f}s")
    return {"value": round(n_steps / dt, 4), "unit": "tok/s", "cores": 1, "kind": "port",
            "sample": f"{n_steps} decode steps (positions 0..{n_steps - 1}) of the same model, "
                      f"f32 weights dequantized at load, single thread"}


def bench_gpt2(args, W, gpu):
    """GPT-2 124M, Q8_0: tokens per second of the greedy loop (prompt positions included:
    the decoder takes one token per step either way)."""
    from wgml_amd.models import GPT2_124M, Gpt2, synth_gpt2

    p = GPT2_124M
    w = synth_gpt2(p, seed=3)
    m = Gpt2(gpu, p).load(w)
    prompt = W.prompt_tokens(3, 32, p.n_vocab)
    n = min(32 + args.steps, p.n_seq)
    m.generate_greedy(prompt, min(64, n))  # records the step
    gpu.synchronize()
    t0 = time.perf_counter()
    toks = m.generate_greedy(prompt, n)
    gpu.synchronize()
    dt = time.perf_counter() - t0
    launches = m.launches_per_token()
    m.set_fusion(0)  # one launch per reference op, a host read-back per token
    gpu.synchronize()
    t0 = time.perf_counter()
    m.generate_greedy(prompt, n)
    gpu.synchronize()
    dt0 = time.perf_counter() - t0
    log(f"gpt2-124m q8_0: {n} positions in {dt * 1e3:.1f} ms -> {n / dt:.0f} tok/s, {launches} "
        f"launches/token; launch per reference op: {n / dt0:.0f} tok/s, "
        f"{m.launches_per_token()} launches/token")
    return {"metric": "decode tok/s bs1 GPT-2 124M Q8_0", "value": round(n / dt, 1), "unit": "tok/s",
            "n_gpus": 1, "steps": n, "warmup": min(64, n), "ms_per_step": round(dt * 1e3 / n, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
            "data": "synthetic",
            "config": {"workload": f"gpt2-124m q8_0 bs1 greedy: 32-token prompt, positions 0..{n - 1}",
                       "launches_per_token": launches,
                       "tok_s_one_launch_per_reference_op": round(n / dt0, 1),
                       "last_token": int(toks[-1])},
            "roofline": None, "cpu_baseline": None}


def bench_8b_gqa(args, W, gpu):
    """Llama-3-8B shape (32 q heads / 8 kv heads, hidden 14336, vocab 128256), Q6_K, with the
    KV caches pre-filled to position 8191: decode steps at a long context."""
    from wgml_amd.models import LLAMA3_8B, Llama2, synth_llama

    cfg = LLAMA3_8B
    t0 = time.perf_counter()
    w = synth_llama(cfg, seed=5, scheme="q6_k")
    log(f"weights built in {time.perf_counter() - t0:.0f}s")
    m = Llama2(gpu, cfg).load(w)
    n_pre, n = 8192, min(args.steps, cfg.seq_len - 8192)
    for layer in range(cfg.n_layers):
        for which in (0, 1):
            kv = W.rng_normal(1000 + 2 * layer + which, n_pre * cfg.kv_dim).reshape(n_pre, cfg.kv_dim)
            m.kv_upload(layer, which, 0, kv)
    gpu.synchronize()
    m.decode_greedy(7, n_pre, 4)  # records the step
    gpu.synchronize()
    t0 = time.perf_counter()
    toks = m.decode_greedy(7, n_pre, n)
    gpu.synchronize()
    dt = time.perf_counter() - t0
    kvb = 2 * cfg.n_layers * cfg.kv_dim * 4 * (n_pre + n // 2)
    wb = w.weight_bytes_per_token()
    log(f"llama3-8b-shape q6_k at position {n_pre}: {n} steps in {dt * 1e3:.1f} ms -> {n / dt:.1f} "
        f"tok/s; {(wb + kvb) / (dt / n) / 1e12:.2f} TB/s over weights + KV")
    return {"metric": "decode tok/s bs1 Llama-3-8B-shape Q6_K at position 8192", "value": round(n / dt, 2),
            "unit": "tok/s", "n_gpus": 1, "steps": n, "warmup": 4, "ms_per_step": round(dt * 1e3 / n, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
            "data": "synthetic",
            "config": {"workload": f"llama3-8b-shape q6_k bs1 greedy decode, KV caches N(0,1) up to "
                                   f"position 8191, {n} timed steps from position 8192",
                       "weight_bytes_per_token": wb, "kv_bytes_per_token_mid_run": kvb,
                       "roofline_tok_s_at_8TBs": round(HBM_PEAK_GBS * 1e9 / (wb + kvb), 1),
                       "frac_of_roofline": round((n / dt) * (wb + kvb) / (HBM_PEAK_GBS * 1e9), 4),
                       "launches_per_token": m.launches_per_token(), "last_token": int(toks[-1])},
            "roofline": None, "cpu_baseline": None}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed decode steps (default 256; 128 for --model tiny)")
    ap.add_argument("--warmup", type=int, default=None,
                    help="prompt tokens before the timed steps (default 128; 16 for --model tiny)")
    ap.add_argument("--model", default="7b", choices=["7b", "tiny", "gpt2", "8b-gqa"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-sweep", action="store_true")
    ap.add_argument("--cpu-steps", type=int, default=0, help="CPU baseline steps (0 = auto)")
    ap.add_argument("--roofline-only", action="store_true",
                    help="only the dominant-kernel measurement (for profiler runs): the fused "
                         "gate/up launches, then three plain copies of 256 MiB (op_assign Copy) "
                         "as the known-size kernel that calibrates the HBM byte counters")
    ap.add_argument("--prefill-only", action="store_true",
                    help="only the batched prompt pass over a --warmup-token prompt, 1 untimed + "
                         "3 timed calls (for profiler runs)")
    ap.add_argument("--gemm-precision", type=int, default=1, choices=[0, 1],
                    help="with --prefill-only: 1 = split-f16 operands (default), 0 = plain f16")
    args = ap.parse_args()
    if args.steps is None:
        args.steps = 128 if args.model == "tiny" else 256
    if args.warmup is None:
        args.warmup = 16 if args.model == "tiny" else 128
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (every kernel uses a single device; "
                 "no collectives are built). Use --gpus 1.")

    import numpy as np

    import wgml_amd as W
    from wgml_amd.models import LLAMA2_7B, TINY_LLAMA, Llama2, synth_llama

    gpu = W.GpuInstance(0)
    name, n_cu = gpu.info()
    log(f"device: {name}, {n_cu} CUs")
    if args.model in ("gpt2", "8b-gqa"):
        line = bench_gpt2(args, W, gpu) if args.model == "gpt2" else bench_8b_gqa(args, W, gpu)
        print(json.dumps(line), flush=True)
        return

    if args.model == "7b":
        cfg, scheme, label = LLAMA2_7B, "q4_k_m", "llama2-7b-shape q4_k_m"
    else:
        cfg, scheme, label = TINY_LLAMA, "q8_0", "tiny-llama2 q8_0"
    assert args.warmup >= 1 and args.warmup + args.steps <= cfg.seq_len, "positions exceed seq_len"

    t0 = time.perf_counter()
    weights = synth_llama(cfg, seed=4, scheme=scheme,
                          progress=lambda l: log(f"  built layer {l + 1}/{cfg.n_layers} "
                                                 f"({time.perf_counter() - t0:.0f}s)")
                          if (l + 1) % 8 == 0 else None)
    log(f"weights built in {time.perf_counter() - t0:.0f}s "
        f"({weights.weight_bytes_per_token() / 1e9:.3f} GB per token)")
    if args.roofline_only:
        us, b = time_gate_up(W, gpu, cfg, weights)
        n = 64 << 20
        src = W.GpuVector.init(gpu, np.zeros(n, np.float32))
        dst = W.GpuVector.uninit(gpu, n)
        for _ in range(3):
            W.OpAssign(gpu, W.OpAssignVariant.Copy).dispatch(dst, src)
        gpu.synchronize()
        print(json.dumps({"kernel": "gemv_fused_kernel gate+up", "us_per_launch": round(us, 3),
                          "bytes_per_launch": b, "GB/s": round(b / us * 1e-3, 1),
                          "calibration": "op_assign Copy of 67108864 f32: 268435456 B read, "
                                         "268435456 B written per launch"}), flush=True)
        return
    model = Llama2(gpu, cfg).load(weights)
    prompt = W.prompt_tokens(4, args.warmup, cfg.vocab_size)
    if args.prefill_only:
        gpu.set_gemm_precision(args.gemm_precision)
        model.prefill(prompt)
        gpu.synchronize()
        t0 = time.perf_counter()
        for _ in range(3):
            model.prefill(prompt)
        gpu.synchronize()
        pdt = (time.perf_counter() - t0) / 3
        print(json.dumps({"prefill_tokens": args.warmup, "gemm_precision": args.gemm_precision,
                          "ms": round(pdt * 1e3, 3),
                          "tok_s": round(args.warmup / pdt, 1),
                          "launches": model.launches_per_token()}), flush=True)
        return

    # warm-up: the prompt, one token at a time (the reference has no batched prefill)
    out = model.generate_greedy(prompt, args.warmup)
    gpu.synchronize()
    first = int(out[-1])

    # the same steps with a blocking read-back of every sampled token, as the reference's
    # chat loop does (reported beside the headline figure, and it warms the recorded step)
    n_sync = min(args.steps, 64)
    gpu.synchronize()
    t0 = time.perf_counter()
    toks_sync = model.decode_greedy_sync(first, args.warmup, n_sync)
    gpu.synchronize()
    tok_s_sync = n_sync / (time.perf_counter() - t0)
    model.decode_greedy(first, args.warmup, 2)  # records the step (graph capture), untimed

    # timed region: exactly `steps` greedy decode steps.  Sampling (arg-max) and the loop
    # bookkeeping run on the device; the host enqueues one recorded step per token and
    # synchronises at the end, when the token ids are copied back.
    gpu.synchronize()
    t0 = time.perf_counter()
    toks = model.decode_greedy(first, args.warmup, args.steps)
    gpu.synchronize()
    dt = time.perf_counter() - t0
    tok_s = args.steps / dt
    assert np.array_equal(toks[:n_sync], toks_sync), "recorded and synchronous loops disagree"
    launches_per_token = model.launches_per_token()
    wbytes = weights.weight_bytes_per_token()
    kv_bytes_mid = 2 * cfg.n_layers * cfg.kv_dim * 4 * (args.warmup + args.steps // 2)
    roof_tok_s = HBM_PEAK_GBS * 1e9 / wbytes
    log(f"decode: {args.steps} steps in {dt * 1e3:.1f} ms -> {tok_s:.1f} tok/s "
        f"({100 * tok_s / roof_tok_s:.1f}% of the weight-bytes roofline {roof_tok_s:.0f} tok/s); "
        f"{launches_per_token} launches/token; with a host read-back per token: "
        f"{tok_s_sync:.1f} tok/s")

    # the batched prompt pass over the same prompt (f16 MFMA products, 128 tokens per run);
    # untimed first call allocates its buffers.  It rewrites KV rows 0..warmup-1 with values
    # that agree with the step-by-step ones to ~1e-3, which nothing after this point reads.
    prefill = None
    if args.warmup >= 2:
        layer_elems = cfg.n_layers * (2 * cfg.dim * cfg.dim + 2 * cfg.kv_dim * cfg.dim +
                                      3 * cfg.dim * cfg.hidden_dim)
        flops = 2.0 * layer_elems * args.warmup
        stepwise_logits = None
        prefill = {"tokens": args.warmup,
                   "ms_step_by_step_at_decode_rate": round(args.warmup / tok_s * 1e3, 1)}
        # level 1 (default): split-f16 operands, results to fp32 rounding; level 0: plain f16
        for level, key in ((1, "split_f16"), (0, "plain_f16")):
            gpu.set_gemm_precision(level)
            model.prefill(prompt)
            gpu.synchronize()
            reps = 3
            t0 = time.perf_counter()
            for _ in range(reps):
                model.prefill(prompt)
            gpu.synchronize()
            pdt = (time.perf_counter() - t0) / reps
            prefill[key] = {"ms": round(pdt * 1e3, 3), "tok_s": round(args.warmup / pdt, 1),
                            "model_TFLOP/s": round(flops / pdt * 1e-12, 1),
                            "first_token_matches_step_by_step": int(np.argmax(model.logits())) == first,
                            "launches": model.launches_per_token()}
            log(f"prefill ({key}): {args.warmup} tokens in {pdt * 1e3:.2f} ms -> {args.warmup / pdt:.0f} "
                f"tok/s, {flops / pdt * 1e-12:.1f} model TFLOP/s (step by step: "
                f"{args.warmup / tok_s * 1e3:.0f} ms); first token matches: "
                f"{prefill[key]['first_token_matches_step_by_step']}")
        gpu.set_gemm_precision(1)

    # dominant kernel: the fused gate/up launch (27% of a step), timed live over the model's
    # own per-layer matrices; the plain single-matrix Q4_K GEMV of the same shape beside it
    roofline = None
    if args.model == "7b":
        us, b = time_gate_up(W, gpu, cfg, weights)
        gbs = b / us * 1e-3
        traffic = None
        tpath = os.path.join(ROOT, "profiles", "traffic.json")
        if os.path.exists(tpath):
            traffic = json.load(open(tpath)).get("gemv_fused_gate_up_bytes_per_launch")
        gate = [W.GpuQuantMatrix(gpu, W.Q4_K, cfg.hidden_dim, cfg.dim, l["ffn_gate"].data)
                for l in weights.layers[:24]]
        us1 = time_gemv(W, gpu, gate, cfg.hidden_dim, cfg.dim, iters=4 * len(gate))
        b1 = gemv_bytes(gate[0].gguf_bytes(), cfg.hidden_dim, cfg.dim)
        del gate
        roofline = {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": traffic,
                    "kernel": "gemv_fused_kernel, gate+up launch: 2 x Q4_K 11008x4096, RMSNorm "
                              "folded into staging, SiLU epilogue",
                    "bytes_per_launch": b, "us_per_launch": round(us, 3),
                    "plain_gemv_q4_k_11008x4096": {"us_per_launch": round(us1, 3),
                                                   "bytes_per_launch": b1,
                                                   "GB/s": round(b1 / us1 * 1e-3, 1)}}
        log(f"dominant kernel gemv_fused_kernel gate+up: {us:.2f} us, {gbs:.0f} GB/s; "
            f"plain Q4_K gemv 11008x4096: {us1:.2f} us, {b1 / us1 * 1e-3:.0f} GB/s")

    sweep = None
    if not args.no_sweep and args.model == "7b":
        # the four GEMV shapes of the 7B model, three formats each; every timing rotates
        # through enough distinct copies (> 640 MB) that nothing is served from a cache
        sweep = {}
        for nrows, ncols in ((4096, 4096), (11008, 4096), (4096, 11008), (32000, 4096)):
            sweep[f"{nrows}x{ncols}"] = gemv_sweep(W, gpu, nrows, ncols)

    cpu = None
    if not args.no_cpu_baseline:
        n = args.cpu_steps or (2 if args.model == "7b" else 32)
        cpu = cpu_baseline(weights, prompt, min(n, args.warmup))

    line = {
        "metric": "decode tok/s bs1 Llama-2-7B-shape Q4_K" if args.model == "7b"
        else "decode tok/s bs1 tiny Llama-2 Q8_0",
        "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(dt * 1e3 / args.steps, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"{label} bs1 greedy decode: {args.warmup}-token prompt "
                               f"(one token per step), then {args.steps} timed steps",
                   "weights": "seeded N(0,0.02), ggml reference quantizers; embedding/activations/KV f32",
                   "weight_bytes_per_token": wbytes, "kv_bytes_per_token_mid_run": kv_bytes_mid,
                   "roofline_tok_s_at_8TBs": round(roof_tok_s, 1),
                   "frac_of_weight_roofline": round(tok_s / roof_tok_s, 4),
                   "launches_per_token": launches_per_token,
                   "tok_s_with_per_token_host_sync": round(tok_s_sync, 2),
                   "last_token": int(toks[-1])},
        "roofline": roofline, "cpu_baseline": cpu, "prefill": prefill, "gemv_sweep": sweep,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
