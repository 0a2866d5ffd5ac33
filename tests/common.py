"""Shared helpers of the test-suite: seeded synthetic models fed identically to the oracle and to the library,
and an independent float64 LLaMA forward (library matmuls, textbook formulas) that pins the oracle."""
from __future__ import annotations

import contextlib

import numpy as np

import oracle
import rllama_amd
from rllama_amd import (ATTN_NORM, FFN_NORM, NORM, OUTPUT, TOK_EMB, W1, W2, W3, WK, WO, WQ, WV)

PER_LAYER = (WQ, WK, WV, WO, W1, W2, W3)


class Shape:
    def __init__(self, dim, n_layers, n_heads, ffn_hidden, vocab_size, max_seq_len, norm_eps=1e-6):
        self.dim, self.n_layers, self.n_heads = dim, n_layers, n_heads
        self.ffn_hidden, self.vocab_size, self.max_seq_len, self.norm_eps = ffn_hidden, vocab_size, max_seq_len, norm_eps
        self.head_dim = dim // n_heads

    def tensor_shape(self, kind):
        d, F, V = self.dim, self.ffn_hidden, self.vocab_size
        return {TOK_EMB: (V, d), OUTPUT: (V, d), WQ: (d, d), WK: (d, d), WV: (d, d), WO: (d, d), W1: (F, d), W3: (F, d),
                W2: (d, F), ATTN_NORM: (1, d), FFN_NORM: (1, d), NORM: (1, d)}[kind]


TINY = Shape(dim=64, n_layers=2, n_heads=2, ffn_hidden=192, vocab_size=96, max_seq_len=24)       # head_dim 32
SMALL = Shape(dim=256, n_layers=3, n_heads=4, ffn_hidden=704, vocab_size=512, max_seq_len=48)    # head_dim 64
# config 0 of the benchmark definition: the reference's own CPU-runnable case
CONFIG0 = Shape(dim=1024, n_layers=8, n_heads=16, ffn_hidden=2816, vocab_size=32000, max_seq_len=80, norm_eps=1e-6)


def synth_weights(shape: Shape, seed: int = 0, std: float = 0.02, norm_ones: bool = True):
    """dict[(kind, layer)] -> uint16 f16 bits (matrices) or float32 (norm vectors), from the counter-based generator."""
    W = {}
    for kind in (TOK_EMB, OUTPUT):
        r, c = shape.tensor_shape(kind)
        W[(kind, 0)] = rllama_amd.synth_normal_f16(seed, kind, 0, r * c, std=std).reshape(r, c)
    for l in range(shape.n_layers):
        for kind in PER_LAYER:
            r, c = shape.tensor_shape(kind)
            W[(kind, l)] = rllama_amd.synth_normal_f16(seed, kind, l, r * c, std=std).reshape(r, c)
    rng = np.random.default_rng(seed + 12345)
    for l in range(shape.n_layers):
        for kind in (ATTN_NORM, FFN_NORM):
            W[(kind, l)] = np.ones((1, shape.dim), np.float32) if norm_ones else rng.uniform(0.5, 1.5, (1, shape.dim)).astype(np.float32)
    W[(NORM, 0)] = np.ones((1, shape.dim), np.float32) if norm_ones else rng.uniform(0.5, 1.5, (1, shape.dim)).astype(np.float32)
    return W


def random_f32_weights(shape: Shape, seed: int, std: float = 0.05):
    """Weights that are NOT f16-representable (f32 mode with genuinely f32 data)."""
    rng = np.random.default_rng(seed)
    W = {}
    for kind in (TOK_EMB, OUTPUT):
        W[(kind, 0)] = (rng.standard_normal(shape.tensor_shape(kind)) * std).astype(np.float32)
    for l in range(shape.n_layers):
        for kind in PER_LAYER:
            W[(kind, l)] = (rng.standard_normal(shape.tensor_shape(kind)) * std).astype(np.float32)
        for kind in (ATTN_NORM, FFN_NORM):
            W[(kind, l)] = rng.uniform(0.5, 1.5, (1, shape.dim)).astype(np.float32)
    W[(NORM, 0)] = rng.uniform(0.5, 1.5, (1, shape.dim)).astype(np.float32)
    return W


def make_oracle(shape: Shape, W, force_f16: bool) -> oracle.Model:
    m = oracle.Model(shape.dim, shape.n_layers, shape.n_heads, shape.ffn_hidden, shape.vocab_size, shape.max_seq_len,
                     shape.norm_eps, force_f16)
    for (kind, layer), arr in W.items():
        m.set_tensor(kind, layer, arr)
    return m


def make_gpu(ctx, shape: Shape, W, force_f16: bool) -> rllama_amd.Transformer:
    ds = rllama_amd.DataSettings(ctx)
    if force_f16:
        ds = ds.force_f16()
    m = rllama_amd.Transformer(ctx, shape.dim, shape.n_layers, shape.n_heads, shape.ffn_hidden, shape.vocab_size,
                               shape.max_seq_len, shape.norm_eps, ds)
    for (kind, layer), arr in W.items():
        m.set_tensor(kind, layer, arr)
    return m


@contextlib.contextmanager
def options(ctx, **switches):
    """Sets switches of the library on the context (rlh_set_option: NAME of the RLLAMA_HIP_<NAME> variables) for the
    duration of a with block, then puts the defaults back."""
    try:
        for name, value in switches.items():
            ctx.set_option(name, value)
        yield
    finally:
        for name in switches:
            ctx.set_option(name, None)


def to_f64(arr: np.ndarray) -> np.ndarray:
    if arr.dtype == np.uint16:
        return arr.view(np.float16).astype(np.float64)
    return arr.astype(np.float64)


def max_rel_err(a: np.ndarray, b: np.ndarray) -> float:
    """max |a - b| / max |b|: the error measure used for logits (relative to the logit scale)."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.max(np.abs(a - b)) / max(np.max(np.abs(b)), 1e-30))


# ---------------------------------------------------------------------------------------------------------
# Independent float64 LLaMA forward.  Written from the architecture's definition (RMSNorm, rotary embedding
# as a complex multiplication on interleaved pairs, causal softmax attention with a KV cache, SwiGLU),
# with numpy's matmul and float16 casts -- none of the oracle's loops or lane orders.
# ---------------------------------------------------------------------------------------------------------
class RefF64:
    def __init__(self, shape: Shape, W, f16_points: bool, via_f32: bool = False):
        self.s = shape
        self.via_f32 = via_f32   # round to f32 first, then to f16: the reference's values are f32 before every cast
        self.W = {k: to_f64(v) for k, v in W.items()}
        self.f16_points = f16_points
        L, H, hd, T = shape.n_layers, shape.n_heads, shape.head_dim, shape.max_seq_len
        self.k = np.zeros((L, H, T, hd))
        self.v = np.zeros((L, H, T, hd))

    def r(self, x):
        if not self.f16_points:
            return x
        if self.via_f32:
            return x.astype(np.float32).astype(np.float16).astype(np.float64)
        return x.astype(np.float16).astype(np.float64)

    def norm(self, x, w):
        return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + self.s.norm_eps) * w

    def forward(self, tokens, start_pos):
        s, W = self.s, self.W
        n, H, hd = len(tokens), s.n_heads, s.head_dim
        x = W[(TOK_EMB, 0)][np.asarray(tokens)]
        pos = np.arange(start_pos, start_pos + n)
        inv_freq = 1.0 / (10000.0 ** (np.arange(0, hd, 2) / hd))
        rot = np.exp(1j * np.outer(pos, inv_freq))  # [n, hd/2]
        T = start_pos + n
        for l in range(s.n_layers):
            xn = self.r(self.norm(x, W[(ATTN_NORM, l)]))
            q = self.r(xn @ W[(WQ, l)].T).reshape(n, H, hd // 2, 2)
            k = self.r(xn @ W[(WK, l)].T).reshape(n, H, hd // 2, 2)
            v = self.r(xn @ W[(WV, l)].T).reshape(n, H, hd)
            qc = (q[..., 0] + 1j * q[..., 1]) * rot[:, None, :]
            kc = (k[..., 0] + 1j * k[..., 1]) * rot[:, None, :]
            q = np.stack([qc.real, qc.imag], axis=-1).reshape(n, H, hd)
            k = np.stack([kc.real, kc.imag], axis=-1).reshape(n, H, hd)
            self.k[l, :, start_pos:T] = self.r(k).transpose(1, 0, 2)
            self.v[l, :, start_pos:T] = self.r(v).transpose(1, 0, 2)
            att = np.zeros((n, H, hd))
            for h in range(H):
                sc = q[:, h] @ self.k[l, h, :T].T / np.sqrt(hd)  # [n, T]
                if n > 1:
                    mask = np.triu(np.full((n, T), -np.inf), k=start_pos + 1)
                    sc = sc + mask
                sc = sc - sc.max(axis=-1, keepdims=True)
                p = np.exp(sc)
                p /= p.sum(axis=-1, keepdims=True)
                att[:, h] = p @ self.v[l, h, :T]
            a = self.r(self.r(att.reshape(n, H * hd)) @ W[(WO, l)].T)
            h_ = x + a
            hn = self.r(self.norm(h_, W[(FFN_NORM, l)]))
            g = self.r(hn @ W[(W1, l)].T)
            u = self.r(hn @ W[(W3, l)].T)
            mm = self.r(g / (1.0 + np.exp(-g)) * u)
            x = h_ + self.r(mm @ W[(W2, l)].T)
        xf = self.norm(x, W[(NORM, 0)])
        return xf[-1] @ W[(OUTPUT, 0)].T


def oracle_from_device(gm: "rllama_amd.Transformer", max_seq_len: int, force_f16: bool = True) -> oracle.Model:
    """An oracle model holding exactly the values the device model holds: every tensor is read back from HBM and handed to
    the oracle (f16 bits in f16 mode, fp32 values in f32 mode), so both sides start from the same weights whatever filled them."""
    d, L, H, F, V = gm.dim, gm.n_layers, gm.n_heads, gm.ffn_hidden, gm.vocab_size
    om = oracle.Model(d, L, H, F, V, max_seq_len, gm.params.norm_eps, force_f16)
    shapes = {WQ: (d, d), WK: (d, d), WV: (d, d), WO: (d, d), W1: (F, d), W3: (F, d), W2: (d, F)}
    for kind in (TOK_EMB, OUTPUT):
        om.set_tensor(kind, 0, gm.get_tensor(kind, 0, V, d, as_f16_bits=True))   # held as f16 on the device in both modes (exact)
    om.set_tensor(NORM, 0, gm.get_tensor(NORM, 0, 1, d))
    for l in range(L):
        for kind, (r, c) in shapes.items():
            om.set_tensor(kind, l, gm.get_tensor(kind, l, r, c, as_f16_bits=force_f16))
        for kind in (ATTN_NORM, FFN_NORM):
            om.set_tensor(kind, l, gm.get_tensor(kind, l, 1, d))
    return om


def elementwise_rel_err(a: np.ndarray, b: np.ndarray, floor_frac: float = 0.01) -> float:
    """max |a - b| / |b| over the entries with |b| above floor_frac of the largest |b| (an element-wise relative error that
    leaves out the entries small through cancellation)."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    keep = np.abs(b) >= floor_frac * np.max(np.abs(b))
    return float(np.max(np.abs(a - b)[keep] / np.abs(b)[keep]))
