#!/usr/bin/env python3
"""Benchmark of the per-token forward path: LLaMA-7B-shape f16 batch-1 greedy decode on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c1] [--no-cpu-baseline]

A "step" is one decoded token: the full token step (5 kernels per layer + output head) plus the greedy
pick, fed on the device with the previous step's token.  The workload is config 1 of the benchmark
definition: 128 synthetic prompt ids, then K (default 256) greedy tokens; random-init weights N(0, 0.02)
from the repo's counter-based generator, seed 0.  Prints ONE JSON line.

Nothing here reads the reference checkout; the CPU oracle is used only for the `cpu_baseline` leg.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published
# HBM bytes per launch of the dominant kernel (c1: w13 GEMV; c3: w1-shape GEMM; 7B shapes).  These are RECORDED values, not
# something a bench run measures: they come from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this same script, each scaled
# by the same counter on a 1 GiB copy kernel; the summaries named here hold the commands and the raw counter readings.
MEASURED_TRAFFIC = {"c1": 180_986_026, "c3": 284_149_621}
TRAFFIC_SOURCE = {"c1": "profiles/decode_c1_hbm_traffic_pmc.md", "c3": "profiles/prefill_c3_hbm_traffic_pmc.md"}

CONFIGS = {
    # name: (dim, n_layers, n_heads, ffn_hidden, vocab, n_prompt, default decode steps)
    "c0": (1024, 8, 16, 2816, 32000, 16, 64),
    "c1": (4096, 32, 32, 11008, 32000, 128, 256),
    "c2": (5120, 40, 40, 13824, 32000, 2048, 128),
    "c3": (4096, 32, 32, 11008, 32000, 1024, 1),          # prompt prefill: one forward over 1024 tokens
    "c4": (8192, 80, 64, 22016, 32000, 256, 128),
}


def cpu_baseline(model, dim, n_layers, n_heads, ffn, vocab, n_prompt=8, n_decode=16):
    """The CPU oracle (restatement of rllama's AVX2 path) on this host's cores, on the same weights.

    Times `n_decode` single-token forwards after an `n_prompt`-token prompt, ms/token defined like
    rllama_main.rs:890-894 (prefill call excluded), threads = the cores this process may use.
    """
    import oracle
    import rllama_amd as ra

    cores = len(os.sched_getaffinity(0))
    try:
        cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    except ValueError:
        pass
    oracle.set_threads(cores)
    oracle.set_reference_threading(True)
    om = oracle.Model(dim, n_layers, n_heads, ffn, vocab, n_prompt + n_decode + 1, 1e-6, True)
    shapes = {ra.WQ: (dim, dim), ra.WK: (dim, dim), ra.WV: (dim, dim), ra.WO: (dim, dim), ra.W1: (ffn, dim), ra.W3: (ffn, dim), ra.W2: (dim, ffn)}
    for kind in (ra.TOK_EMB, ra.OUTPUT):
        om.set_tensor(kind, 0, model.get_tensor(kind, 0, vocab, dim, as_f16_bits=True))
    om.set_tensor(ra.NORM, 0, model.get_tensor(ra.NORM, 0, 1, dim))
    for l in range(n_layers):
        for kind, (r, c) in shapes.items():
            om.set_tensor(kind, l, model.get_tensor(kind, l, r, c, as_f16_bits=True))
        for kind in (ra.ATTN_NORM, ra.FFN_NORM):
            om.set_tensor(kind, l, model.get_tensor(kind, l, 1, dim))
    prompt = ra.synth_tokens(0, n_prompt, 3, vocab)
    oc = om.make_caches()
    toks = list(prompt)
    t0 = time.perf_counter()
    logits = om.forward(toks, 0, oc)
    t_first = time.perf_counter() - t0
    per, o_logits, o_ids = [], [logits], []
    for _ in range(n_decode):
        tok, _, _ = oracle.sample_greedy(logits)
        toks.append(tok)
        o_ids.append(tok)
        t0 = time.perf_counter()
        logits = om.forward(toks[-1:], len(toks) - 1, oc)
        per.append(time.perf_counter() - t0)
        o_logits.append(logits)
    ms = 1e3 * float(np.mean(per))
    baseline = {
        "value": round(ms, 2), "unit": "ms/token", "cores": cores, "kind": "port",
        "sample": f"same shape and weights, f16 mode, {n_prompt} prompt + {n_decode} greedy decode tokens "
                  f"(first call {1e3 * t_first:.0f} ms excluded)",
        "tokens_per_s": round(1e3 / ms, 3),
    }
    # The same calls on the device (the oracle here is the checker, as in the tests): logits of every call against the
    # oracle's, max |a - b| / max |b|, and the device's own greedy loop against the oracle's ids.
    def rel(a, b):
        return float(np.max(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64))) / max(float(np.max(np.abs(b))), 1e-30))
    gc = model.make_caches()
    errs = [rel(model.forward(prompt, 0, gc), o_logits[0])]
    for i, tok in enumerate(o_ids):
        errs.append(rel(model.forward([tok], n_prompt + i, gc), o_logits[i + 1]))
    gc.free()
    gc = model.make_caches()
    g_ids, _, _ = model.generate_greedy(prompt, n_decode, gc)
    gc.free()
    same = 0
    for a, b in zip(g_ids.tolist(), o_ids):
        if a != b:
            break
        same += 1
    parity = {"against": "CPU oracle (restatement of the reference's AVX2 path), full depth, same weights and token ids",
              "max_rel_err": float(f"{max(errs):.3e}"), "tolerance": 1e-2, "measure": "max|a-b| / max|b| over the logits of each call",
              "calls": len(errs), "greedy_ids_identical": same, "greedy_ids_compared": len(o_ids)}
    return baseline, parity


def measure_prefill(ra, ctx, model, prompt, reps, dim, n_layers, ffn, vocab):
    """One forward over the whole prompt (+ the greedy pick): wall and HIP-event time to the first token, and the dominant
    kernel -- w1 and w3 of one block (n x 2 ffn x dim) -- timed alone with HIP events on the library's stream."""
    n = len(prompt)
    model.generate_greedy(prompt, 1, model.make_caches())            # warm-up (also sizes the work buffers)
    times = []
    for _ in range(reps):
        cc = model.make_caches()
        ctx.sync()
        t0 = time.perf_counter()
        _, ms_first, _ = model.generate_greedy(prompt, 1, cc)
        ctx.sync()
        times.append((1e3 * (time.perf_counter() - t0), ms_first))
        cc.free()
    wall_ms = float(np.mean([t[0] for t in times]))
    ev_ms = float(np.mean([t[1] for t in times]))
    flops_linear = 2.0 * n * n_layers * (4 * dim * dim + 3 * dim * ffn)
    flops_attn = 2.0 * n * n * dim * n_layers          # causal: half of the dense 4 n^2 d
    flops_head = 2.0 * vocab * dim
    flops_total = flops_linear + flops_attn + flops_head
    tflops = flops_total / (ev_ms * 1e-3) / 1e12
    # the dominant kernel alone: w1 and w3 of one block as the forward runs them at this prompt length -- one pass over the
    # normalised rows with two accumulator sets (rlh_ffn_gate) -- on operands of the same shapes
    ga = ra.Tensor.from_numpy(ctx, ra.synth_normal_f16(1, 5, 0, n * dim, std=0.5).reshape(n, dim))
    gb = ra.Tensor.from_numpy(ctx, ra.synth_normal_f16(2, 5, 0, ffn * dim, std=0.02).reshape(ffn, dim))
    gb3 = ra.Tensor.from_numpy(ctx, ra.synth_normal_f16(3, 5, 0, ffn * dim, std=0.02).reshape(ffn, dim))
    gc = ra.Tensor.zeros(ctx, n, ffn, ra.TensorDType.Float16)
    for _ in range(3):
        ra.check(ctx._lib.rlh_ffn_gate(gc._h, ga._h, gb._h, gb3._h))
    ctx.sync()
    iters = 20
    e0 = ctx.event()
    for _ in range(iters):
        ra.check(ctx._lib.rlh_ffn_gate(gc._h, ga._h, gb._h, gb3._h))
    e1 = ctx.event()
    gemm_us = e0.elapsed_ms(e1) / iters * 1e3
    gemm_flops = 4.0 * n * ffn * dim
    gemm_tflops = gemm_flops / (gemm_us * 1e-6) / 1e12
    for t in (ga, gb, gb3, gc):
        t.free()
    return wall_ms, ev_ms, tflops, gemm_us, gemm_tflops, gemm_flops, flops_total


def other_config_block(ra, ctx, name, warmup=8, kernel_iters=160):
    """One of the other decode configurations of the benchmark definition, measured like the headline one: its own model
    (random-init, seed 0), its prompt through the matrix-core path, then its K greedy decode steps timed between two syncs;
    the token-step kernels timed one by one at the mean sequence length of those steps."""
    dim, n_layers, n_heads, ffn, vocab, n_prompt, K = CONFIGS[name]
    max_seq = n_prompt + max(K, warmup) + 1
    model = ra.Transformer(ctx, dim, n_layers, n_heads, ffn, vocab, max_seq, 1e-6, ra.DataSettings(ctx).force_f16())
    model.fill_synthetic(seed=0, std=0.02)
    prompt = ra.synth_tokens(0, n_prompt, 3, vocab)
    cw = model.make_caches()
    model.generate_greedy(prompt, 1, cw)                     # sizes the work buffers
    model.decode_greedy(warmup, cw)
    cw.free()
    caches = model.make_caches()
    ctx.sync()
    t0 = time.perf_counter()
    _, ms_prompt, _ = model.generate_greedy(prompt, 1, caches)
    ctx.sync()
    prompt_wall = 1e3 * (time.perf_counter() - t0)
    t0 = time.perf_counter()
    _, ms_events = model.decode_greedy(K, caches)
    ctx.sync()
    ms = 1e3 * (time.perf_counter() - t0) / K
    mean_bytes = float(np.mean([model.decode_bytes(n_prompt + i + 1) for i in range(K)]))
    T_mid = n_prompt + K // 2
    kernels = {}
    for which, kname in enumerate(ra.Transformer.STEP_KERNELS):
        us, nbytes = model.time_kernel(which, T_mid, kernel_iters if which != 5 else max(20, kernel_iters // 8), caches)
        kernels[kname] = {"us": round(us, 2), "bytes": nbytes, "GBps": round(nbytes / us / 1e3, 1), "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 3)}
    caches.free()
    model.free()
    return {
        "workload": f"{name}: dim {dim}, {n_layers} layers, {n_heads} heads, ffn {ffn}, vocab {vocab}; {n_prompt} prompt ids then {K} greedy decode tokens, batch 1",
        "ms_per_token": round(ms, 4), "ms_per_token_hip_events": round(ms_events / K, 4), "tokens_per_s": round(1e3 / ms, 2),
        "algorithmic_bytes_per_token": int(mean_bytes), "hbm_GBps_end_to_end": round(mean_bytes / (ms * 1e-3) / 1e9, 1),
        "hbm_frac_end_to_end": round(mean_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
        "ms_prompt_pass": round(ms_prompt, 2), "ms_prompt_pass_wall": round(prompt_wall, 2), "prompt_tokens": n_prompt,
        "kernels_at_T": T_mid, "kernels": kernels,
    }


def vendor_calibration(ra, ctx) -> int:
    """Same-box calibration against the vendor library (torch.mm / torch.mv -> hipBLASLt / rocBLAS, f16 in, f16 out): the
    prompt-path products of the 7B shape at 1024 rows and of the 13B shape at 2048 rows, and the single-row products of the
    7B shape.  Both sides cycle through enough distinct weight matrices that nothing stays in the 256 MB memory-side cache.
    torch is used for the vendor side only; nothing of the library depends on it."""
    import torch
    rng = np.random.default_rng(0)
    dev = torch.device("cuda:0")

    def n_copies(n, k):
        return max(2, int(6e8 // (n * k * 2)) + 1)

    def gemm_pair(m, n, k, iters=24):
        nb = n_copies(n, k)
        a = (torch.randn(m, k, device=dev) * 0.1).half()
        bs = [(torch.randn(n, k, device=dev) * 0.02).half() for _ in range(nb)]
        for i in range(3 * iters):        # the clocks of an idle part take a few milliseconds of load to come up
            c = a @ bs[i % nb].t()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(iters):
            c = a @ bs[i % nb].t()
        e1.record()
        torch.cuda.synchronize()
        vendor = e0.elapsed_time(e1) / iters * 1e3
        del bs, c
        A = ra.Tensor.from_numpy(ctx, (rng.standard_normal((m, k)) * 0.1).astype(np.float16))
        Bs = [ra.Tensor.from_numpy(ctx, ra.synth_normal_f16(7, 5, i, n * k, std=0.02).reshape(n, k)) for i in range(nb)]
        out = ra.Tensor.zeros(ctx, m, n, ra.TensorDType.Float16)
        for i in range(3 * iters):
            ra.check(ctx._lib.rlh_matrix_mul_inplace_transposed(out._h, A._h, Bs[i % nb]._h))
        ctx.sync()
        e0 = ctx.event()
        for i in range(iters):
            ra.check(ctx._lib.rlh_matrix_mul_inplace_transposed(out._h, A._h, Bs[i % nb]._h))
        e1 = ctx.event()
        here = e0.elapsed_ms(e1) / iters * 1e3
        res = {"vendor_us": round(vendor, 1), "here_us": round(here, 1), "distinct_weight_matrices": nb}
        if nb >= 2 and n % 8 == 0 and m > 1:
            for i in range(iters):
                ra.check(ctx._lib.rlh_ffn_gate(out._h, A._h, Bs[i % nb]._h, Bs[(i + 1) % nb]._h))
            ctx.sync()
            e0 = ctx.event()
            for i in range(iters):
                ra.check(ctx._lib.rlh_ffn_gate(out._h, A._h, Bs[i % nb]._h, Bs[(i + 1) % nb]._h))
            e1 = ctx.event()
            res["two_products_in_one_pass_us"] = round(e0.elapsed_ms(e1) / iters * 1e3, 1)
        for t in [A, out] + Bs:
            t.free()
        return res

    def gemv_pair(n, k, iters=120):
        nb = n_copies(n, k)
        ws = [(torch.randn(n, k, device=dev) * 0.02).half() for _ in range(nb)]
        x = torch.randn(k, device=dev).half()
        for i in range(2 * iters):
            y = torch.mv(ws[i % nb], x)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(iters):
            y = torch.mv(ws[i % nb], x)
        e1.record()
        torch.cuda.synchronize()
        vendor = e0.elapsed_time(e1) / iters * 1e3
        del ws, y
        here = ctx.time_gemv(n, k, ra.TensorDType.Float16, False, False, n_buffers=nb, iters=iters)
        return {"vendor_us": round(vendor, 2), "here_us": round(here, 2), "distinct_weight_matrices": nb}

    out = {"calibration": "vendor library (torch 2.x -> hipBLASLt / rocBLAS) against this library, same box, f16", "gemm": {}, "gemv": {}}
    for label, (m, d, F) in (("7B shape, 1024 rows", (1024, 4096, 11008)), ("13B shape, 2048 rows", (2048, 5120, 13824))):
        out["gemm"][label] = {"wq|wk|wv (plain product, no RoPE epilogue)": gemm_pair(m, 3 * d, d), "wo": gemm_pair(m, d, d),
                              "w1 (one of the pair)": gemm_pair(m, F, d), "w2": gemm_pair(m, d, F)}
    for n, k in ((4096, 4096), (12288, 4096), (11008, 4096), (22016, 4096), (4096, 11008), (32000, 4096)):
        out["gemv"][f"{n}x{k}"] = gemv_pair(n, k)
    print(json.dumps(out))
    return 0


def bench_layer_split(args, ra, ctx, info) -> int:
    """The device's share of a model split by percentage_to_gpu: one prompt call, then K single-token calls of
    rlh_forward_layers, each taking the stream from host memory and returning it there (the hand-off the reference makes at
    the layer boundary).  The host-side blocks are the caller's and are not part of this figure."""
    dim, n_layers, n_heads, ffn, vocab, n_prompt, dflt_steps = CONFIGS[args.config]
    K = args.steps if args.steps is not None else dflt_steps
    W = max(0, args.warmup)
    max_seq = n_prompt + K + W + 1
    ds = ra.DataSettings(ctx).force_f16().percentage_to_gpu(args.percentage_to_gpu)
    model = ra.Transformer(ctx, dim, n_layers, n_heads, ffn, vocab, max_seq, 1e-6, ds)
    model.fill_synthetic(seed=0, std=0.02)
    last = model.last_layer_on_gpu()
    cc = model.make_caches()
    rng = np.random.default_rng(0)
    x = rng.standard_normal((n_prompt, dim)).astype(np.float32)
    model.forward_layers(x, 0, cc, 0, last)                                  # sizes the work buffers
    t0 = time.perf_counter()
    y = model.forward_layers(x, 0, cc, 0, last)
    prompt_ms = 1e3 * (time.perf_counter() - t0)
    row = y[-1:].copy()
    pos = n_prompt
    for _ in range(W):
        row = model.forward_layers(row, pos, cc, 0, last)
        pos += 1
    t0 = time.perf_counter()
    for _ in range(K):
        row = model.forward_layers(row, pos, cc, 0, last)
        pos += 1
    ms = 1e3 * (time.perf_counter() - t0) / K
    n_res = last + 1
    t_mean = n_prompt + W + (K + 1) / 2.0
    bytes_call = n_res * ((4 * dim * dim + 3 * dim * ffn) * 2 + 2 * t_mean * dim * 2 + 2 * dim * 2)
    out = {
        "metric": "ms per token, device share of a layer-split LLaMA-7B-shape f16 model (stream handed over per call), 1 MI355X",
        "value": round(ms, 4), "unit": "ms/token", "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": round(ms, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f16 weights, fp32 accumulate",
        "data": "synthetic (random-init N(0,0.02) weights seed 0, random stream rows)",
        "config": {"workload": f"{args.config}: dim {dim}, layers 0..{last} of {n_layers} on the device (percentage_to_gpu {args.percentage_to_gpu}), "
                               f"{n_prompt}-row prompt call then {K} single-row calls"},
        "prompt_call_ms": round(prompt_ms, 3), "us_per_resident_layer": round(1e3 * ms / n_res, 2),
        "handoff_bytes_per_call": 2 * dim * 4,
        "roofline": {"bound": "hbm", "achieved": round(bytes_call / (ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(bytes_call / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4), "traffic": None,
                     "algorithmic_bytes_per_call": int(bytes_call)},
        "cpu_baseline": None, "device": info["name"],
    }
    print(json.dumps(out))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--config", default="c1", choices=sorted(CONFIGS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-prefill-block", action="store_true", help="c1: skip the 1024-token prefill measurement (prefill_c3)")
    ap.add_argument("--no-other-configs", action="store_true", help="c1: skip the 13B (c2) and 65B (c4) decode measurements (other_configs)")
    ap.add_argument("--kernel-iters", type=int, default=320)
    ap.add_argument("--kernels-only", action="store_true",
                    help="skip the token loop and the CPU baseline: only the per-kernel timing loops (short runs for "
                         "rocprofv3 --pmc passes)")
    ap.add_argument("--kernel", default=None, help="with --kernels-only: time only this token-step kernel (a name from the output's \"kernels\")")
    ap.add_argument("--kernel-T", type=int, default=None, help="with --kernels-only: the sequence length the attention kernel sees")
    ap.add_argument("--percentage-to-gpu", type=float, default=1.0,
                    help="below 1: time the device's share of a layer-split model (rlh_forward_layers over layers "
                         "0..=round(p * (n_layers - 1)), stream handed over from and to host memory on every call)")
    ap.add_argument("--probe-gemv-phases", action="store_true",
                    help="run only the wall-clock decomposition of the isolated GEMV launch (rlh_probe_gemv_phases) on the shapes of the 7B model")
    ap.add_argument("--vendor-calibration", action="store_true",
                    help="run only the same-box comparison with the vendor library's GEMM / GEMV (needs torch; for profiles/prefill_vendor_calibration.md)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run only a plain copy kernel over 1 GiB of f32 (reads 1 GiB, writes 1 GiB per launch): "
                         "the known-size reference for scaling rocprofv3's FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (batch-1 decode of one model resident in one device's HBM); "
              f"--gpus {args.gpus} is not supported.", file=sys.stderr)
        return 2

    import rllama_amd as ra

    if args.probe_gemv_phases:
        ctx = ra.Context(0)
        out = {"probe": "100 MHz wall clock read by every wavefront at entry, x staged, first burst consumed, last burst consumed, exit; "
                        "means over 63 back-to-back launches on distinct weight matrices, microseconds", "shapes": {}}
        for rows, k in ((8, 4096), (2048, 4096), (4096, 4096), (12288, 4096), (11008, 4096), (4096, 11008), (32000, 4096)):
            nb = min(24, max(2, int(1.2e9 // (rows * k * 2)) + 1))
            r = ctx.probe_gemv_phases(rows, k, n_buffers=nb, launches=64)
            r["hip_event_us_per_launch"] = round(ctx.time_gemv(rows, k, ra.TensorDType.Float16, False, False, n_buffers=nb, iters=200), 2)
            r["weight_bytes"] = rows * k * 2
            out["shapes"][f"{rows}x{k}"] = r
        ctx.close()
        print(json.dumps(out))
        return 0
    if args.vendor_calibration:
        import torch  # before the library's own context: torch brings its own copy of the HIP runtime and wants to be first
        torch.zeros(1, device="cuda:0")
        ctx = ra.Context(0)
        rc = vendor_calibration(ra, ctx)
        ctx.close()
        return rc
    if args.calibrate_copy:
        ctx = ra.Context(0)
        rows, cols = 16384, 16384  # 2^28 f32 = 1 GiB
        src = ra.Tensor.zeros(ctx, rows, cols, ra.TensorDType.Float32)
        for _ in range(4):
            dst = src.clone()     # one convert_kernel<float, float> launch: 1 GiB read + 1 GiB written
            dst.free()
        ctx.sync()
        print(json.dumps({"calibration": "convert_kernel<float,float> copy", "launches": 4, "bytes_read_per_launch": rows * cols * 4,
                          "bytes_written_per_launch": rows * cols * 4}))
        return 0

    dim, n_layers, n_heads, ffn, vocab, n_prompt, dflt_steps = CONFIGS[args.config]
    K = args.steps if args.steps is not None else dflt_steps
    W = max(0, args.warmup)
    max_seq = max(n_prompt + max(K, W) + 1, (args.kernel_T or 0) + 1)
    with_prefill_block = args.config == "c1" and not args.kernels_only and not args.no_prefill_block
    if with_prefill_block:
        max_seq = max(max_seq, 1025)   # room for the 1024-token prompt of the prefill block (config c3 on the same model)
    if args.config == "c1" and not args.kernels_only:
        max_seq = max(max_seq, 128 + 256 + 1)   # and for the full 128 + 256 workload when --steps asks for fewer

    ctx = ra.Context(0, verbose=False)
    info = ctx.device_info()
    if args.percentage_to_gpu < 1.0:
        return bench_layer_split(args, ra, ctx, info)
    ds = ra.DataSettings(ctx).force_f16()
    model = ra.Transformer(ctx, dim, n_layers, n_heads, ffn, vocab, max_seq, 1e-6, ds)
    model.fill_synthetic(seed=0, std=0.02)
    prompt = ra.synth_tokens(0, n_prompt, 3, vocab)

    if args.config == "c3":
        # prefill: time-to-first-token of one n_prompt-token forward (+ greedy pick), TFLOP/s against the dense f16 MFMA peak
        reps = max(1, K)
        n = n_prompt
        wall_ms, ev_ms, tflops, gemm_us, gemm_tflops, gemm_flops, flops_total = measure_prefill(ra, ctx, model, prompt, reps, dim, n_layers, ffn, vocab)
        flops_linear = 2.0 * n * n_layers * (4 * dim * dim + 3 * dim * ffn)
        flops_attn = 2.0 * n * n * dim * n_layers
        flops_head = 2.0 * vocab * dim
        out = {
            "metric": "time to first token, LLaMA-7B-shape f16 prompt prefill (1024 tokens), 1 MI355X",
            "value": round(wall_ms, 3), "unit": "ms", "n_gpus": 1, "steps": reps, "warmup": 1, "ms_per_step": round(wall_ms, 3),
            "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f16 operands, fp32 accumulate (MFMA)",
            "data": "synthetic (random-init N(0,0.02) weights seed 0, synthetic token ids)",
            "config": {"workload": f"c3: dim {dim}, {n_layers} layers, {n_heads} heads, ffn {ffn}; one forward over {n} prompt tokens"},
            "ms_hip_events": round(ev_ms, 3), "tokens_per_s": round(n / (wall_ms * 1e-3), 1),
            "tflops_end_to_end": round(tflops, 1), "algorithmic_flops_end_to_end": flops_linear + flops_attn + flops_head,
            "roofline": {"bound": "mfma", "kernel": f"gemm_f16_dma_kernel, w1 and w3 in one pass (256x192 tile of each, v_mfma_f32_32x32x16_f16, SiLU-gate epilogue): {n} x 2*{ffn} x {dim}",
                         "achieved": round(gemm_tflops, 1), "peak": 2500.0, "unit": "TFLOP/s", "frac": round(gemm_tflops / 2500.0, 4), "traffic": MEASURED_TRAFFIC.get("c3"),
                         "traffic_source": TRAFFIC_SOURCE["c3"] + " (recorded rocprofv3 --pmc run, not measured by this run)",
                         "us_per_launch": round(gemm_us, 2), "algorithmic_flops": gemm_flops,
                         "algorithmic_bytes_per_launch": 2 * (n * dim + 2 * ffn * dim + n * ffn)},
            "cpu_baseline": None, "device": info["name"],
        }
        print(json.dumps(out))
        return 0

    if args.kernels_only:
        caches = model.make_caches()
        T_mid = args.kernel_T if args.kernel_T else n_prompt + K // 2
        out = {"kernels_only": True, "T": T_mid, "kernels": {}}
        for which, name in enumerate(ra.Transformer.STEP_KERNELS):
            if args.kernel and name != args.kernel:
                continue
            us, nbytes = model.time_kernel(which, T_mid, args.kernel_iters, caches)
            out["kernels"][name] = {"us": round(us, 2), "bytes": nbytes}
        print(json.dumps(out))
        return 0

    # ---- warmup: W untimed decode steps (own caches, same prompt) ----
    cw = model.make_caches()
    model.generate_greedy(prompt, 1, cw)
    if W > 0:
        model.decode_greedy(W, cw)
    cw.free()

    # ---- timed region: exactly K decode steps after the prompt ----
    caches = model.make_caches()
    first_ids, ms_prompt, _ = model.generate_greedy(prompt, 1, caches)   # prompt pass + first token (untimed)
    ctx.sync()
    t0 = time.perf_counter()
    ids, ms_events = model.decode_greedy(K, caches)                      # K token steps, no host round trip
    ctx.sync()
    wall_ms = 1e3 * (time.perf_counter() - t0)
    ms_per_step = wall_ms / K

    # algorithmic HBM bytes of the K steps: weights once per token + KV rows read + written
    T_values = [n_prompt + i + 1 for i in range(K)]                      # sequence length seen by step i
    step_bytes = [model.decode_bytes(T) for T in T_values]
    mean_bytes = float(np.mean(step_bytes))
    e2e_gbps = mean_bytes / (ms_per_step * 1e-3) / 1e9

    # ---- per-kernel timing (HIP events on the launch stream, weights cycled over all layers) ----
    T_mid = n_prompt + K // 2
    kernels = {}
    for which, name in enumerate(ra.Transformer.STEP_KERNELS):
        us, nbytes = model.time_kernel(which, T_mid, args.kernel_iters if which != 5 else max(20, args.kernel_iters // 8), caches)
        kernels[name] = {"us": round(us, 2), "bytes": nbytes, "GBps": round(nbytes / us / 1e3, 1), "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 3)}
    dom = "w13_silu"  # ffn_norm + w1|w3 + SiLU*gate: the largest share of the bytes of a token step
    roofline = {
        "bound": "hbm", "kernel": "gemv_kernel<f16 weights, f16 x, SiLU epilogue> (" + dom + ")",
        "achieved": kernels[dom]["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
        "frac": round(kernels[dom]["GBps"] / HBM_PEAK_GBPS, 4), "traffic": MEASURED_TRAFFIC.get(args.config),
        "traffic_source": (TRAFFIC_SOURCE[args.config] + " (recorded rocprofv3 --pmc run, not measured by this run)") if args.config in TRAFFIC_SOURCE else None,
        "algorithmic_bytes_per_launch": kernels[dom]["bytes"], "us_per_launch": kernels[dom]["us"],
    }

    # ---- isolated GEMV microbench: [11008 x 4096] and [4096 x 11008] f16 against fp32 x, >1 GB of weights cycled ----
    micro = {}
    if args.config == "c1":
        for rows, k in ((11008, 4096), (4096, 11008)):
            us = ctx.time_gemv(rows, k, ra.TensorDType.Float16, False, False, n_buffers=12, iters=240)
            nb = rows * k * 2 + k * 4 + rows * 4
            micro[f"{rows}x{k}"] = {"us": round(us, 2), "bytes": nb, "GBps": round(nb / us / 1e3, 1), "frac": round(nb / us / 1e3 / HBM_PEAK_GBPS, 3)}

    out = {
        "metric": f"ms/token, LLaMA-{ {'c0': 'tiny', 'c1': '7B', 'c2': '13B', 'c4': '65B'}[args.config] }-shape f16 batch-1 greedy decode, 1 MI355X",
        "value": round(ms_per_step, 4), "unit": "ms/token", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 weights/KV, fp32 accumulate", "data": "synthetic (random-init N(0,0.02) weights seed 0, synthetic token ids)",
        "config": {"workload": f"{args.config}: dim {dim}, {n_layers} layers, {n_heads} heads, ffn {ffn}, vocab {vocab}; "
                               f"{n_prompt} prompt ids then {K} greedy decode tokens, batch 1", "max_seq_len": max_seq},
        "tokens_per_s": round(1e3 / ms_per_step, 2),
        "ms_per_token_hip_events": round(ms_events / K, 4),
        "ms_prompt_pass": round(ms_prompt, 2),
        "hbm_GBps_end_to_end": round(e2e_gbps, 1),
        "hbm_frac_end_to_end": round(e2e_gbps / HBM_PEAK_GBPS, 4),
        "algorithmic_bytes_per_token": int(mean_bytes),
        "roofline": roofline,
        "kernels": kernels,
        "gemv_microbench": micro,
        "device": info["name"],
        "first_tokens": [int(first_ids[0])] + [int(t) for t in ids[:7]],
    }
    if args.config == "c1" and K != dflt_steps:
        # the benchmark definition's workload is 128 prompt + 256 decode tokens; with another --steps the line above is quoted on
        # a shorter (or longer) sequence, so the full workload is measured too
        c2 = model.make_caches()
        model.generate_greedy(prompt, 1, c2)
        ctx.sync()
        t0 = time.perf_counter()
        model.decode_greedy(dflt_steps, c2)
        ctx.sync()
        ms256 = 1e3 * (time.perf_counter() - t0) / dflt_steps
        b256 = float(np.mean([model.decode_bytes(n_prompt + i + 1) for i in range(dflt_steps)]))
        out["workload_128_plus_256"] = {"ms_per_token": round(ms256, 4), "hbm_frac_end_to_end": round(b256 / (ms256 * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                                        "note": f"--steps {K} changes the mean sequence length; this is the defined workload (256 decode steps)"}
        c2.free()
    if with_prefill_block:
        # config c3 on the same weights: one forward over a 1024-token prompt, MFMA roofline of its dominant GEMM
        p1024 = ra.synth_tokens(0, 1024, 3, vocab)
        wall_p, ev_p, tflops_p, gemm_us, gemm_tflops, gemm_flops, flops_total = measure_prefill(ra, ctx, model, p1024, 3, dim, n_layers, ffn, vocab)
        out["prefill_c3"] = {
            "workload": "c3: one forward over a 1024-token prompt on the same model", "ttft_ms": round(wall_p, 3), "ttft_ms_hip_events": round(ev_p, 3),
            "prompt_tokens_per_s": round(1024 / (wall_p * 1e-3), 1), "tflops_end_to_end": round(tflops_p, 1), "algorithmic_flops_end_to_end": flops_total,
            "roofline": {"bound": "mfma", "kernel": f"gemm_f16_dma_kernel, w1 and w3 in one pass (256x192 tile of each, v_mfma_f32_32x32x16_f16, SiLU-gate epilogue): 1024 x 2*{ffn} x {dim}",
                         "achieved": round(gemm_tflops, 1), "peak": 2500.0, "unit": "TFLOP/s", "frac": round(gemm_tflops / 2500.0, 4),
                         "us_per_launch": round(gemm_us, 2), "algorithmic_flops": gemm_flops, "traffic": MEASURED_TRAFFIC["c3"],
                         "traffic_source": TRAFFIC_SOURCE["c3"] + " (recorded rocprofv3 --pmc run, not measured by this run)"},
        }
    if not args.no_cpu_baseline:
        out["cpu_baseline"], out["parity"] = cpu_baseline(model, dim, n_layers, n_heads, ffn, vocab)
    else:
        out["cpu_baseline"] = None
    caches.free()
    model.free()
    if args.config == "c1" and not args.no_other_configs:
        # the other two decode configurations of the benchmark definition, each on its own model (the 7B one is freed first:
        # the 65B weights alone are 130 GB)
        out["other_configs"] = {}
        for name in ("c2", "c4"):
            try:
                out["other_configs"][name] = other_config_block(ra, ctx, name)
            except ra.RllamaHipError as e:   # e.g. a smaller part without room for the 65B shape: say so, keep the headline line
                out["other_configs"][name] = {"error": str(e)}
    ctx.close()
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
