"""Writes tests/golden/config0_oracle.json and tests/golden/tiny_oracle.json: what the CPU oracle (oracle/) produces on
seeded synthetic inputs, frozen so that a change of the oracle, of the generator or of the device path shows up as a diff
against committed data.

Run from the repository root:  python tests/golden/make_oracle_fixtures.py       (about a minute of CPU)

config 0 (the benchmark definition's CPU-runnable case: dim 1024, 8 layers, 16 heads, ffn 2816, vocab 32000, eps 1e-6, f16
weights N(0, 0.02) seed 0, norm weights 1.0; 16 prompt ids, then 64 greedy steps): SHA-256 of every generated weight tensor,
the prompt ids, the 64 greedy ids, per step the gap between the two largest logits (after the sampler's token-0 rule) and 32
sampled logits as fp32 bit patterns.  Tiny shapes: the full logits of an f16-mode and an f32-mode forward.  Data only.
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(HERE))
import oracle  # noqa: E402
import rllama_amd  # noqa: E402
from common import CONFIG0, TINY, make_oracle, random_f32_weights, synth_weights  # noqa: E402

KIND_NAMES = {rllama_amd.TOK_EMB: "tok_embeddings", rllama_amd.OUTPUT: "output", rllama_amd.WQ: "wq", rllama_amd.WK: "wk", rllama_amd.WV: "wv",
              rllama_amd.WO: "wo", rllama_amd.W1: "w1", rllama_amd.W2: "w2", rllama_amd.W3: "w3"}
SAMPLE_IDS = [int(v) for v in np.linspace(0, 31999, 32).astype(np.int64)]


def config0():
    shape = CONFIG0
    W = synth_weights(shape, seed=0, std=0.02)
    sha = {f"{KIND_NAMES[k]}.{l}": hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest() for (k, l), a in sorted(W.items()) if k in KIND_NAMES}
    prompt = rllama_amd.synth_tokens(0, 16, 3, 32000)
    om = make_oracle(shape, W, True)
    oc = om.make_caches()
    toks, prev = [int(t) for t in prompt], 0
    ids, gaps, samples = [], [], []
    for _ in range(64):
        logits = om.forward(toks[prev:], prev, oc)
        tok, _, ties = oracle.sample_greedy(logits)
        assert ties == 1
        l2 = logits.copy()
        l2[0] = 0.0
        top2 = np.sort(l2)[-2:]
        gaps.append(float(top2[1] - top2[0]))
        samples.append([int(v) for v in logits[SAMPLE_IDS].astype(np.float32).view(np.uint32)])
        ids.append(int(tok))
        toks.append(int(tok))
        prev = len(toks) - 1
    return {"shape": {"dim": shape.dim, "n_layers": shape.n_layers, "n_heads": shape.n_heads, "ffn_hidden": shape.ffn_hidden,
                      "vocab_size": shape.vocab_size, "norm_eps": shape.norm_eps}, "seed": 0, "std": 0.02, "weight_sha256": sha,
            "prompt_ids": [int(t) for t in prompt], "greedy_ids": ids, "top2_logit_gap": gaps, "sample_token_ids": SAMPLE_IDS,
            "sample_logits_f32_bits": samples}


def tiny():
    out = {}
    toks = [int(t) for t in np.random.default_rng(22).integers(0, TINY.vocab_size, 12)]
    for mode, W, f16 in (("f16", synth_weights(TINY, seed=21, std=0.08, norm_ones=False), True), ("f32", random_f32_weights(TINY, seed=23, std=0.08), False)):
        om = make_oracle(TINY, W, f16)
        oc = om.make_caches()
        prefill = om.forward(toks[:7], 0, oc)
        step = om.forward(toks[7:8], 7, oc)
        out[mode] = {"tokens": toks[:8], "logits_after_7_f32_bits": [int(v) for v in prefill.astype(np.float32).view(np.uint32)],
                     "logits_after_8_f32_bits": [int(v) for v in step.astype(np.float32).view(np.uint32)]}
    return out


if __name__ == "__main__":
    json.dump(config0(), open(os.path.join(HERE, "config0_oracle.json"), "w"), indent=1)
    json.dump(tiny(), open(os.path.join(HERE, "tiny_oracle.json"), "w"), indent=1)
    print("wrote config0_oracle.json, tiny_oracle.json")
