#!/usr/bin/env python3
"""Benchmark of the batch-1 token-decode path on one MI355X.

Workload (default): Llama-2-7B shape (dim 4096, 32 layers, 32 heads, FFN 11008,
vocab 32000), weights seeded N(0, 0.02) quantized with the ggml reference
quantizers in a Q4_K_M-style mix (Q4_K; Q6_K for attn_v, output and the
ffn_down layers picked by use_more_bits), embedding f32, KV cache f32.  The
128-token prompt always goes through the batched prompt pass (untimed here,
timed on its own below), then `--warmup` greedy decode steps run untimed from
position 128, then exactly `--steps` greedy decode steps are timed: one step =
one token = one pass over every weight.  The flags never change the workload's
shape, only how many steps of it are timed.

Prints ONE JSON line: decode tok/s; what arithmetic ran (`dtype`: the GEMVs
multiply the quantized weights with activations rounded to 16-bit block fixed
point on the integer dot-product units and accumulate in i32 / f32) with the
same decode on fp32 activations beside it; the logit error of the GPU step
against the CPU oracle on the positions the CPU baseline runs; the HBM roofline
of the dominant kernel (gemv_fused_kernel as launched for the gate/up
projections) measured with HIP events on the library's own stream, launch by
launch as rocprofv3 sees it, and inside a recorded graph as the decode loop
runs it; a GEMV sweep over the model's four matrix shapes for the three
formats, on the GPU (both activation modes) and on the host cores; and the CPU
baseline (the C restatement of the reference's CPU transformer) on a bounded
sample, single-threaded as the reference and on all host cores.

    python bench.py [--gpus 1] [--steps 256] [--warmup 8] [--model 7b|tiny]

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


DTYPE = ("quantized weights (q4_k/q6_k/q8_0 ints) x 16-bit block-fixed-point activations on "
         "v_dot4 i8, i32 sub-block sums, f32 scales and accumulation; norms/RoPE/attention f32")


class eager_launches:
    """Inside: recorded launch sequences are enqueued launch by launch instead of replayed as
    HIP graphs (what rocprofv3's kernel trace can see)."""

    def __enter__(self):
        self.old = os.environ.get("WGML_DISABLE_GRAPHS")
        os.environ["WGML_DISABLE_GRAPHS"] = "1"

    def __exit__(self, *a):
        if self.old is None:
            del os.environ["WGML_DISABLE_GRAPHS"]
        else:
            os.environ["WGML_DISABLE_GRAPHS"] = self.old


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


READ_CHAIN_ROWS = (4096, 11008, 22016, 46400)  # 9.4 / 25.4 / 50.7 / 106.9 MB per launch


def read_chain(gpu, use_graph=True):
    """The machine's own ceiling for a chain of launches: a kernel that only reads, with the
    Q4_K GEMV's access pattern (wgml_bench_read_chain), at four sizes.  A least-squares line
    through time per launch against bytes gives what a launch boundary costs (intercept) and
    what loads sustain (1 / slope)."""
    from wgml_amd._lib import call

    pts = []
    ms = C.c_float()
    for nrows in READ_CHAIN_ROWS:
        nbytes = nrows * 2304
        iters = max(64, min(600, (3 << 30) // nbytes))
        best = None
        for _ in range(3):
            call("wgml_bench_read_chain", gpu.handle, nrows, iters, 1 if use_graph else 0, C.byref(ms))
            us = ms.value * 1e3 / iters
            best = us if best is None else min(best, us)
        pts.append((nbytes, best))
    n = len(pts)
    sx = sum(b for b, _ in pts)
    sy = sum(t for _, t in pts)
    sxx = sum(b * b for b, _ in pts)
    sxy = sum(b * t for b, t in pts)
    slope = (n * sxy - sx * sy) / (n * sxx - sx * sx)  # us per byte
    icpt = (sy - slope * sx) / n
    return {"points": [{"bytes": b, "us_per_launch": round(t, 3), "GB/s": round(b / t * 1e-3, 1)}
                       for b, t in pts],
            "GB/s": round(1e-3 / slope, 1), "launch_overhead_us": round(icpt, 3),
            "how": "bare read kernel with the Q4_K GEMV's access pattern, one launch after the other "
                   + ("in a recorded graph" if use_graph else "launch by launch")
                   + ", rotating over a 1.5 GB pool; line through us per launch against bytes"}


def gemv_sweep(W, gpu, nrows, ncols, cpu_threads, min_total_bytes=640 << 20, formats=None):
    """One matrix shape for Q8_0 / Q4_K / Q6_K: GB/s and fraction of HBM peak on the GPU (the
    default integer-dot kernels and the fp32-activation kernels), and the CPU oracle's
    dequantize-and-dot over the same bytes on one core and on `cpu_threads` cores."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle as orc

    res = {}
    vals = W.rng_normal(4242, nrows * ncols, 0.0, 0.02)
    xcpu = W.rng_normal(99, ncols)
    for qtype, name in ((W.Q8_0, "q8_0"), (W.Q4_K, "q4_k"), (W.Q6_K, "q6_k")):
        if formats and name not in formats:
            continue
        raw = W.quantize(qtype, vals)
        n_copies = max(2, -(-min_total_bytes // raw.nbytes))
        mats = [W.GpuQuantMatrix(gpu, qtype, nrows, ncols, raw) for _ in range(n_copies)]
        us = time_gemv(W, gpu, mats, nrows, ncols, iters=4 * n_copies)
        gpu.set_tuning(gpu.TUNE_GEMV_F32_ACTIVATIONS, 1)
        us32 = time_gemv(W, gpu, mats, nrows, ncols, iters=4 * n_copies)
        gpu.set_tuning(gpu.TUNE_GEMV_F32_ACTIVATIONS, 0)
        b = gemv_bytes(raw.nbytes, nrows, ncols)
        gbs = b / us * 1e-3
        cpu = {}
        for threads in sorted({1, cpu_threads} if cpu_threads else ()):
            orc.set_threads(threads)
            t0 = time.perf_counter()
            orc.gemv_quant(qtype, raw, nrows, ncols, xcpu)
            cpu[f"GB/s_{threads}_cores"] = round(b / (time.perf_counter() - t0) * 1e-9, 3)
        orc.set_threads(1)
        res[name] = {"us": round(us, 3), "GB/s": round(gbs, 1), "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
                     "bytes": b, "copies": n_copies,
                     "fp32_activations": {"us": round(us32, 3), "GB/s": round(b / us32 * 1e-3, 1)},
                     "cpu_oracle": cpu}
        log(f"  gemv {name} {nrows}x{ncols}: {us:.2f} us  {gbs:.0f} GB/s  "
            f"({100 * gbs / HBM_PEAK_GBS:.1f}% of HBM peak); fp32 activations {us32:.2f} us; cpu {cpu}")
        del mats
    return res


def cpu_baseline(weights, prompt, n_steps, threads_all):
    """Times the CPU oracle (port of the reference's CPU transformer, weights expanded to f32
    at load as the reference does) on the first `n_steps` positions of the same model and
    prompt: single-threaded as the reference is, and once more with the rows of every
    matrix-vector product shared out over `threads_all` host cores.  Returns the JSON object
    and the oracle's logits per position."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle as orc

    t0 = time.perf_counter()
    m = orc.Llama2(weights, predequantize=True)
    t_load = time.perf_counter() - t0
    logits = []
    orc.set_threads(1)
    t0 = time.perf_counter()
    for pos in range(n_steps):
        logits.append(m.forward(int(prompt[pos]), pos))
    dt = time.perf_counter() - t0
    m2 = orc.Llama2(weights, predequantize=True) if threads_all > 1 else None
    dt_all = None
    if m2 is not None:
        orc.set_threads(threads_all)
        t0 = time.perf_counter()
        for pos in range(n_steps):
            m2.forward(int(prompt[pos]), pos)
        dt_all = time.perf_counter() - t0
        orc.set_threads(1)
    log(f"  cpu oracle: load (dequantize) {t_load:.1f}s, {n_steps} steps in {dt:.1f}s on 1 core"
        + (f", {dt_all:.1f}s on {threads_all} cores" if dt_all else ""))
    out = {"value": round(n_steps / dt, 4), "unit": "tok/s", "cores": 1, "kind": "port",
           "sample": f"{n_steps} decode steps (positions 0..{n_steps - 1}) of the same model and "
                     f"prompt, f32 weights dequantized at load, single thread as the reference",
           "all_cores": None}
    if dt_all:
        out["all_cores"] = {"value": round(n_steps / dt_all, 4), "unit": "tok/s", "cores": threads_all,
                            "sample": "the same steps, rows of every matrix-vector product shared "
                                      "out over the host cores (OpenMP); identical results"}
    return out, logits


def parity_at_timed_positions(W, gpu, model, weights, prompt, generated, first, p0, warmup, steps, cores):
    """The GPU step against the CPU oracle at positions the timed region covers.  The oracle
    (all host cores; same sums for any thread count) is fed the prompt and then the tokens the
    GPU chose, so both sides see the same context; its logits at up to four timed positions
    (the first two, one a little later, and the last one within a budget of 40 decode
    positions) are compared with the GPU's step at those positions, for the default
    integer-dot step and for the step with fp32 activations in every GEMV."""
    import numpy as np

    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle as orc

    seq = np.concatenate([np.asarray(prompt, dtype=np.int64), [first], np.asarray(generated, dtype=np.int64)])
    # seq[pos] = the token fed at position pos
    t_first = p0 + warmup
    t_last = min(t_first + steps - 1, p0 + 39)
    cand = sorted({t_first, min(t_first + 1, t_last), min(t_first + 7, t_last), t_last})
    cand = [c for c in cand if c >= t_first]
    orc.set_threads(cores)
    t0 = time.perf_counter()
    ref = orc.Llama2(weights, predequantize=True)
    want = {}
    for pos in range(cand[-1] + 1):
        lg = ref.forward(int(seq[pos]), pos)
        if pos in cand:
            want[pos] = lg.astype(np.float64).copy()
    orc.set_threads(1)
    dt = time.perf_counter() - t0

    def worst_error():
        # the state the timed steps ran on: the prompt through the batched pass at its default
        # precision, then one step per position (every step rewrites its own KV row)
        gpu.set_gemm_precision(1)
        model.prefill(prompt)
        worst = 0.0
        for pos in range(p0, cand[-1] + 1):
            got = model.forward_logits(pos, int(seq[pos]))
            if pos in want:
                worst = max(worst, float(np.abs(got.astype(np.float64) - want[pos]).max() /
                                         np.abs(want[pos]).max()))
        return worst

    e_default = worst_error()
    gpu.set_tuning(gpu.TUNE_GEMV_F32_ACTIVATIONS, 1)
    e_f32 = worst_error()
    gpu.set_tuning(gpu.TUNE_GEMV_F32_ACTIVATIONS, 0)
    log(f"  GPU step vs oracle logits at positions {cand} (oracle through {cand[-1] + 1} positions on "
        f"{cores} cores: {dt:.0f}s): {e_default:.2e} of max|logit| (integer-dot step), {e_f32:.2e} "
        f"(fp32 activations); budget 1e-3")
    return {"max_logit_err_over_max_logit": float(f"{e_default:.3e}"),
            "fp32_activations_max_logit_err_over_max_logit": float(f"{e_f32:.3e}"),
            "positions": cand, "timed_positions": [t_first, t_first + steps - 1], "budget": 1e-3,
            "against": "CPU oracle fed the prompt and the tokens the GPU generated (same weights), "
                       "logits at positions inside the timed region"}


def host_cores():
    """Cores this process may use (the box's CPU share, not the machine's core count)."""
    n = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    env = os.environ.get("OMP_NUM_THREADS")
    if env and env.isdigit() and int(env) > 0:
        n = min(n, int(env))
    return max(1, n)


def bench_gpt2(args, W, gpu):
    """GPT-2 124M, Q8_0: tokens per second of the greedy loop (prompt positions included:
    the decoder takes one token per step either way)."""
    from wgml_amd.models import GPT2_124M, Gpt2, synth_gpt2

    p = GPT2_124M
    w = synth_gpt2(p, seed=3)
    m = Gpt2(gpu, p).load(w)
    prompt = W.prompt_tokens(3, 32, p.n_vocab)
    n = min(32 + args.steps, p.n_seq)
    m.generate_greedy(prompt, min(64, n))  # warm-up
    m.record_steps(n)  # the recorded steps of every range of positions the timed run passes
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
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": DTYPE,
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
    m.record_steps(n_pre, n)
    m.decode_greedy(7, n_pre, 4)  # warm-up
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
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": DTYPE,
            "data": "synthetic",
            "config": {"workload": f"llama3-8b-shape q6_k bs1 greedy decode, KV caches N(0,1) up to "
                                   f"position 8191, {n} timed steps from position 8192",
                       "weight_bytes_per_token": wb, "kv_bytes_per_token_mid_run": kvb,
                       "roofline_tok_s_at_8TBs": round(HBM_PEAK_GBS * 1e9 / (wb + kvb), 1),
                       "frac_of_roofline": round((n / dt) * (wb + kvb) / (HBM_PEAK_GBS * 1e9), 4),
                       "launches_per_token": m.launches_per_token(), "last_token": int(toks[-1])},
            "roofline": None, "cpu_baseline": None}


def attention_leg(W, gpu):
    """Decode attention on its own at the Llama-3-8B head layout (32 query / 8 KV heads of 128),
    position 8192: GB/s of the K and V rows read, launches rotating over eight cache sets
    (553 MB, nothing stays cached), position read from device memory as in a recorded step."""
    import numpy as np
    from wgml_amd._lib import AttnParams, View, call

    seq_len, n_heads, kv_mul, hs, pos = 8448, 32, 4, 128, 8192
    kv_dim = n_heads // kv_mul * hs
    n_sets = 8
    q = W.GpuVector.init(gpu, W.rng_normal(71, n_heads * hs))
    sets = [(W.GpuVector.init(gpu, W.rng_normal(72 + 2 * i, seq_len * kv_dim)),
             W.GpuVector.init(gpu, W.rng_normal(73 + 2 * i, seq_len * kv_dim))) for i in range(n_sets)]
    xb = W.GpuVector.uninit(gpu, n_heads * hs)
    kv = (View * n_sets)(*[k.view() for k, _ in sets])
    vv = (View * n_sets)(*[v.view() for _, v in sets])
    p = AttnParams(seq_len, kv_dim, kv_mul, n_heads, hs, pos)
    ms, iters, best = C.c_float(), 64, None
    for _ in range(3):
        call("wgml_bench_attention", gpu.handle, C.byref(p), seq_len, q.view(), kv, vv, n_sets, xb.view(),
             iters, C.byref(ms))
        us = ms.value * 1e3 / iters
        best = us if best is None else min(best, us)
    nbytes = 2 * kv_dim * 4 * (pos + 1)
    return {"workload": "decode attention, 32 query / 8 KV heads of 128, position 8192 (attention + "
                        "merge of the partial results), f32 caches",
            "us_per_layer": round(best, 3), "kv_bytes": nbytes, "GB/s": round(nbytes / best * 1e-3, 1),
            "frac_hbm_peak": round(nbytes / best * 1e-3 / HBM_PEAK_GBS, 4)}


def gpt2_leg(W, gpu, steps=288):
    from wgml_amd.models import GPT2_124M, Gpt2, synth_gpt2

    p = GPT2_124M
    m = Gpt2(gpu, p).load(synth_gpt2(p, seed=3))
    prompt = W.prompt_tokens(3, 32, p.n_vocab)
    n = min(32 + steps, p.n_seq)
    m.generate_greedy(prompt, min(64, n))  # warm-up
    m.record_steps(n)  # the recorded steps of every range of positions the timed run passes
    gpu.synchronize()
    t0 = time.perf_counter()
    m.generate_greedy(prompt, n)
    gpu.synchronize()
    dt = time.perf_counter() - t0
    return {"workload": f"gpt2-124m q8_0 bs1 greedy: 32-token prompt, positions 0..{n - 1}",
            "tok_s": round(n / dt, 1), "launches_per_token": m.launches_per_token()}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed decode steps (default 256; 112 for --model tiny)")
    ap.add_argument("--warmup", type=int, default=8,
                    help="untimed decode steps between the prompt and the timed steps (default 8)")
    ap.add_argument("--model", default="7b", choices=["7b", "tiny", "gpt2", "8b-gqa"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-sweep", action="store_true")
    ap.add_argument("--cpu-steps", type=int, default=0, help="CPU baseline steps (0 = auto)")
    ap.add_argument("--roofline-only", action="store_true",
                    help="only the dominant-kernel measurement, launch by launch (for profiler "
                         "runs): the fused gate/up launches, then three plain copies of 256 MiB "
                         "(op_assign Copy) as the known-size kernel that calibrates the HBM byte "
                         "counters")
    ap.add_argument("--sweep-only", action="store_true",
                    help="only the GEMV sweep, launch by launch (for profiler runs)")
    ap.add_argument("--sweep-shape", default=None,
                    help="with --sweep-only: one shape, ROWSxCOLS (e.g. 4096x11008), default all four")
    ap.add_argument("--sweep-format", default=None,
                    help="with --sweep-only: one of q8_0, q4_k, q6_k (default all three)")
    ap.add_argument("--decode-only", action="store_true",
                    help="only the prompt pass, the warm-up and the timed decode steps (for profiler "
                         "runs: the kernel trace then holds the decode step and little else)")
    ap.add_argument("--prefill-only", action="store_true",
                    help="only the batched prompt pass over the prompt, 1 untimed + 3 timed calls "
                         "(for profiler runs)")
    ap.add_argument("--ceiling", action="store_true",
                    help="only the machine's own read ceiling: a bare read kernel with the Q4_K "
                         "GEMV's access pattern at 9.4 / 25.4 / 50.7 / 106.9 MB per launch, in a "
                         "recorded graph and launch by launch (for profiler runs: set "
                         "WGML_DISABLE_GRAPHS=1)")
    ap.add_argument("--gemm-precision", type=int, default=1, choices=[0, 1],
                    help="with --prefill-only: 1 = split-f16 operands (default), 0 = plain f16")
    ap.add_argument("--tune", action="append", default=[], metavar="KEY=VALUE",
                    help="launch-shape override, e.g. GEMM_K_SPLIT=4 (a TUNE_* key of GpuInstance); "
                         "may be given several times (for sweeps)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (every kernel uses a single device; "
                 "no collectives are built). Use --gpus 1.")

    import numpy as np

    import wgml_amd as W
    from wgml_amd.models import LLAMA2_7B, TINY_LLAMA, Llama2, synth_llama

    gpu = W.GpuInstance(0)
    name, n_cu = gpu.info()
    cores = host_cores()
    log(f"device: {name}, {n_cu} CUs; host cores for the CPU legs: {cores}")
    for kv in args.tune:
        key, value = kv.split("=")
        gpu.set_tuning(getattr(gpu, "TUNE_" + key.upper()), int(value))
    if args.ceiling:
        print(json.dumps({"read_chain_in_graph": read_chain(gpu, True),
                          "read_chain_launch_by_launch": read_chain(gpu, False)}), flush=True)
        return
    if args.model in ("gpt2", "8b-gqa"):
        if args.steps is None:
            args.steps = 256
        line = bench_gpt2(args, W, gpu) if args.model == "gpt2" else bench_8b_gqa(args, W, gpu)
        print(json.dumps(line), flush=True)
        return

    # The workload's shape is fixed: the flags only say how many of its decode steps are
    # warm-up and how many are timed.
    if args.model == "7b":
        cfg, scheme, label, n_prompt = LLAMA2_7B, "q4_k_m", "llama2-7b-shape q4_k_m", 128
    else:
        cfg, scheme, label, n_prompt = TINY_LLAMA, "q8_0", "tiny-llama2 q8_0", 16
    if args.steps is None:
        args.steps = 256 if args.model == "7b" else 112
    if args.warmup < 1 or n_prompt + args.warmup + args.steps > cfg.seq_len:
        sys.exit(f"bench.py: {n_prompt} prompt positions + {args.warmup} warm-up + {args.steps} timed "
                 f"steps must fit the model's {cfg.seq_len} positions (and --warmup >= 1)")

    if args.sweep_only:
        shapes = ((4096, 4096), (11008, 4096), (4096, 11008), (32000, 4096))
        if args.sweep_shape:
            shapes = (tuple(int(v) for v in args.sweep_shape.split("x")),)
        with eager_launches():
            for nrows, ncols in shapes:
                gemv_sweep(W, gpu, nrows, ncols, 0,
                           formats=(args.sweep_format,) if args.sweep_format else None)
        return

    t0 = time.perf_counter()
    weights = synth_llama(cfg, seed=4, scheme=scheme,
                          progress=lambda l: log(f"  built layer {l + 1}/{cfg.n_layers} "
                                                 f"({time.perf_counter() - t0:.0f}s)")
                          if (l + 1) % 8 == 0 else None)
    log(f"weights built in {time.perf_counter() - t0:.0f}s "
        f"({weights.weight_bytes_per_token() / 1e9:.3f} GB per token)")
    if args.roofline_only:
        with eager_launches():
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
    prompt = W.prompt_tokens(4, n_prompt, cfg.vocab_size)
    if args.prefill_only:
        gpu.set_gemm_precision(args.gemm_precision)
        model.prefill(prompt)
        gpu.synchronize()
        t0 = time.perf_counter()
        for _ in range(3):
            model.prefill(prompt)
        gpu.synchronize()
        pdt = (time.perf_counter() - t0) / 3
        print(json.dumps({"prefill_tokens": n_prompt, "gemm_precision": args.gemm_precision,
                          "ms": round(pdt * 1e3, 3),
                          "tok_s": round(n_prompt / pdt, 1),
                          "launches": model.launches_per_token()}), flush=True)
        return

    # the prompt: one batched pass (timed on its own further down); its last logits give the
    # first generated token
    model.prefill(prompt)
    first = int(np.argmax(model.logits()))
    p0 = n_prompt  # position of the first decode step

    # the steps are recorded (captured as graphs, one per range of positions) before anything
    # is timed: a run that crosses position 256 would otherwise record the next range inside
    # the timed region
    model.record_steps(p0, args.warmup + args.steps)

    if args.decode_only:
        wtoks = model.decode_greedy(first, p0, args.warmup)
        gpu.synchronize()
        t0 = time.perf_counter()
        model.decode_greedy(int(wtoks[-1]), p0 + args.warmup, args.steps)
        gpu.synchronize()
        dt = time.perf_counter() - t0
        print(json.dumps({"decode_steps": args.steps, "from_position": p0 + args.warmup,
                          "tok_s": round(args.steps / dt, 2),
                          "launches_per_token": model.launches_per_token()}), flush=True)
        return

    # the same steps with a blocking read-back of every sampled token, as the reference's
    # chat loop does (reported beside the headline figure; part of the warm-up)
    n_sync = min(args.steps, 64)
    gpu.synchronize()
    t0 = time.perf_counter()
    toks_sync = model.decode_greedy_sync(first, p0, args.warmup + n_sync)
    gpu.synchronize()
    tok_s_sync = (args.warmup + n_sync) / (time.perf_counter() - t0)

    # warm-up: `--warmup` recorded steps (the first call captures the step as a graph)
    wtoks = model.decode_greedy(first, p0, args.warmup)
    gpu.synchronize()

    # timed region: exactly `steps` greedy decode steps.  Sampling (arg-max) and the loop
    # bookkeeping run on the device; the host enqueues one recorded step per token and
    # synchronises at the end, when the token ids are copied back.
    t0 = time.perf_counter()
    toks = model.decode_greedy(int(wtoks[-1]), p0 + args.warmup, args.steps)
    gpu.synchronize()
    dt = time.perf_counter() - t0
    tok_s = args.steps / dt
    # the two loops plan their attention launches differently (per range of positions / per
    # position), so their sums are ordered differently: equal tokens are expected, and reported
    # rather than assumed (a near-tie of two logits may fall either way)
    same_as_sync = bool(np.array_equal(np.concatenate([wtoks, toks])[:args.warmup + n_sync], toks_sync))
    if not same_as_sync:
        log("note: the recorded loop and the loop with a host read-back per token chose different tokens")
    launches_per_token = model.launches_per_token()  # of the last timed step
    # the recorded step differs between ranges of positions (attention without partial results
    # below position 256, with a merge launch from there on): say which range the figure is for
    launches_note = (f"{launches_per_token} at position {p0 + args.warmup + args.steps - 1} (the last "
                     f"timed step); the step is recorded per range of positions (limits 256, 512, "
                     f"1024, ...): attention below position 256 is one launch per layer, two from there on")
    wbytes = weights.weight_bytes_per_token()
    kv_bytes_mid = 2 * cfg.n_layers * cfg.kv_dim * 4 * (p0 + args.warmup + args.steps // 2)
    roof_tok_s = HBM_PEAK_GBS * 1e9 / wbytes
    log(f"decode: {args.steps} steps in {dt * 1e3:.1f} ms -> {tok_s:.1f} tok/s "
        f"({100 * tok_s / roof_tok_s:.1f}% of the weight-bytes roofline {roof_tok_s:.0f} tok/s); "
        f"{launches_per_token} launches/token; with a host read-back per token: "
        f"{tok_s_sync:.1f} tok/s")

    # the same decode with fp32 activations in every GEMV (no 16-bit rounding of x; the
    # arithmetic of the reference's shaders), same fused launches
    gpu.set_tuning(gpu.TUNE_GEMV_F32_ACTIVATIONS, 1)
    n32 = min(args.steps, 64)
    model.record_steps(p0, n32)  # (a changed override drops the recorded steps)
    model.decode_greedy(first, p0, 2)
    gpu.synchronize()
    t0 = time.perf_counter()
    toks32 = model.decode_greedy(first, p0, n32)
    gpu.synchronize()
    dt32 = time.perf_counter() - t0
    fp32_act = {"tok_s": round(n32 / dt32, 2), "steps": n32, "launches_per_token": model.launches_per_token(),
                "same_tokens_as_default": bool(np.array_equal(toks32, np.concatenate([wtoks, toks])[:n32])),
                "note": "fp32 activations staged in LDS, the same fused launches as the default step"}
    gpu.set_tuning(gpu.TUNE_GEMV_F32_ACTIVATIONS, 0)
    log(f"decode with fp32 activations: {n32 / dt32:.1f} tok/s ({fp32_act['launches_per_token']} launches/token), "
        f"same tokens: {fp32_act['same_tokens_as_default']}")

    # the batched prompt pass over the prompt (MFMA products, 128 tokens per run).  It
    # rewrites KV rows 0..n_prompt-1 with the values they already hold.
    layer_elems = cfg.n_layers * (2 * cfg.dim * cfg.dim + 2 * cfg.kv_dim * cfg.dim +
                                  3 * cfg.dim * cfg.hidden_dim)
    flops = 2.0 * layer_elems * n_prompt
    prefill = {"tokens": n_prompt, "ms_step_by_step_at_decode_rate": round(n_prompt / tok_s * 1e3, 1)}
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
        prefill[key] = {"ms": round(pdt * 1e3, 3), "tok_s": round(n_prompt / pdt, 1),
                        "model_TFLOP/s": round(flops / pdt * 1e-12, 1),
                        "first_token_matches_default": int(np.argmax(model.logits())) == first,
                        "launches": model.launches_per_token()}
        log(f"prefill ({key}): {n_prompt} tokens in {pdt * 1e3:.2f} ms -> {n_prompt / pdt:.0f} "
            f"tok/s, {flops / pdt * 1e-12:.1f} model TFLOP/s (step by step: "
            f"{n_prompt / tok_s * 1e3:.0f} ms); first token matches: "
            f"{prefill[key]['first_token_matches_default']}")
    gpu.set_gemm_precision(1)

    # dominant kernel: the fused gate/up launch (27% of a step), timed live over the model's
    # own per-layer matrices.  `achieved` / `frac` come from launch-by-launch timing, the way
    # rocprofv3's kernel trace sees the same command (profiles/); the figure inside a recorded
    # graph, as the decode loop runs it, is carried beside it.
    roofline = None
    if args.model == "7b":
        with eager_launches():
            us_eager, b = time_gate_up(W, gpu, cfg, weights)
        us_graph, _ = time_gate_up(W, gpu, cfg, weights)
        gbs = b / us_eager * 1e-3
        traffic, traffic_src = None, None
        tpath = os.path.join(ROOT, "profiles", "traffic.json")
        if os.path.exists(tpath):
            tj = json.load(open(tpath))
            traffic = tj.get("gemv_fused_gate_up_bytes_per_launch")
            traffic_src = tj.get("source")
            # the counters were read for the kernel as it was then: say so when it has changed
            ksrc = os.path.join(ROOT, "wgml_amd", "csrc", "gemv.hip")
            if os.path.exists(ksrc) and os.path.getmtime(ksrc) > os.path.getmtime(tpath) + 1:
                log("WARNING: wgml_amd/csrc/gemv.hip is newer than profiles/traffic.json: "
                    "roofline.traffic was measured for an earlier build of the kernel")
                traffic_src = (traffic_src or "") + " (measured before the kernel source last changed)"
        gate = [W.GpuQuantMatrix(gpu, W.Q4_K, cfg.hidden_dim, cfg.dim, l["ffn_gate"].data)
                for l in weights.layers[:24]]
        us1 = time_gemv(W, gpu, gate, cfg.hidden_dim, cfg.dim, iters=4 * len(gate))
        b1 = gemv_bytes(gate[0].gguf_bytes(), cfg.hidden_dim, cfg.dim)
        del gate
        chain = read_chain(gpu, True)
        log(f"machine read ceiling (bare read chain in a graph): {chain['GB/s']:.0f} GB/s sustained, "
            f"{chain['launch_overhead_us']:.2f} us per launch boundary")
        roofline = {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": traffic,
                    "achievable": chain,
                    "traffic_source": traffic_src,
                    "kernel": "gemv_fused_kernel, gate+up launch: 2 x Q4_K 11008x4096, RMSNorm "
                              "folded into staging, SiLU epilogue",
                    "bytes_per_launch": b, "us_per_launch": round(us_eager, 3),
                    "timing": "HIP events around back-to-back launches on the library's stream, "
                              "launch by launch (no graph)",
                    "in_recorded_graph": {"us_per_launch": round(us_graph, 3),
                                          "GB/s": round(b / us_graph * 1e-3, 1),
                                          "frac": round(b / us_graph * 1e-3 / HBM_PEAK_GBS, 4)},
                    "plain_gemv_q4_k_11008x4096_in_graph": {"us_per_launch": round(us1, 3),
                                                            "bytes_per_launch": b1,
                                                            "GB/s": round(b1 / us1 * 1e-3, 1)}}
        log(f"dominant kernel gemv_fused_kernel gate+up: {us_eager:.2f} us launch by launch "
            f"({gbs:.0f} GB/s), {us_graph:.2f} us in a graph; plain Q4_K gemv 11008x4096: "
            f"{us1:.2f} us, {b1 / us1 * 1e-3:.0f} GB/s")

    sweep = None
    if not args.no_sweep and args.model == "7b":
        # the four GEMV shapes of the 7B model, three formats each; every GPU timing rotates
        # through enough distinct copies (> 640 MB) that nothing is served from a cache
        sweep = {}
        for nrows, ncols in ((4096, 4096), (11008, 4096), (4096, 11008), (32000, 4096)):
            sweep[f"{nrows}x{ncols}"] = gemv_sweep(W, gpu, nrows, ncols, cores)

    cpu, parity = None, None
    if not args.no_cpu_baseline:
        n = args.cpu_steps or (2 if args.model == "7b" else 16)
        n = min(n, n_prompt)
        cpu, _ = cpu_baseline(weights, prompt, n, cores)
        parity = parity_at_timed_positions(W, gpu, model, weights, prompt, np.concatenate([wtoks, toks]),
                                           first, p0, args.warmup, args.steps, cores)

    other = None
    if args.model == "7b" and not args.no_sweep:
        # cheap legs of the two other large workloads, so that the one line carries them
        other = {"attention_8b_gqa_pos8192": attention_leg(W, gpu), "gpt2_124m_q8_0": gpt2_leg(W, gpu)}
        log(f"other workloads: attention at the 8B-GQA layout, position 8192: "
            f"{other['attention_8b_gqa_pos8192']['us_per_layer']:.2f} us per layer, "
            f"{other['attention_8b_gqa_pos8192']['GB/s']:.0f} GB/s; GPT-2 124M: "
            f"{other['gpt2_124m_q8_0']['tok_s']:.0f} tok/s")

    line = {
        "metric": "decode tok/s bs1 Llama-2-7B-shape Q4_K" if args.model == "7b"
        else "decode tok/s bs1 tiny Llama-2 Q8_0",
        "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(dt * 1e3 / args.steps, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": DTYPE,
        "data": "synthetic",
        "config": {"workload": f"{label} bs1 greedy decode: {n_prompt}-token prompt (batched prompt "
                               f"pass), {args.warmup} untimed steps from position {p0}, then "
                               f"{args.steps} timed steps from position {p0 + args.warmup}",
                   "weights": "seeded N(0,0.02), ggml reference quantizers; embedding/KV f32",
                   "weight_bytes_per_token": wbytes, "kv_bytes_per_token_mid_run": kv_bytes_mid,
                   "roofline_tok_s_at_8TBs": round(roof_tok_s, 1),
                   "frac_of_weight_roofline": round(tok_s / roof_tok_s, 4),
                   "launches_per_token": launches_per_token,
                   "launches_per_token_note": launches_note,
                   "tok_s_with_per_token_host_sync": round(tok_s_sync, 2),
                   "same_tokens_with_per_token_host_sync": same_as_sync,
                   "fp32_activations": fp32_act,
                   "last_token": int(toks[-1])},
        "roofline": roofline, "cpu_baseline": cpu, "parity": parity, "prefill": prefill,
        "gemv_sweep": sweep, "other_workloads": other,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
