"""ctypes binding of the CPU oracle (oracle/rllama_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke`` and by the
``cpu_baseline`` leg of ``bench.py``.  The shipped package never imports this module.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "librllama_oracle.so")

TOK_EMB, WQ, WK, WV, WO, W1, W2, W3, ATTN_NORM, FFN_NORM, NORM, OUTPUT = range(12)
F16, F32 = 0, 1


class Params(C.Structure):
    _fields_ = [
        ("dim", C.c_int32),
        ("n_layers", C.c_int32),
        ("n_heads", C.c_int32),
        ("ffn_hidden", C.c_int32),
        ("vocab_size", C.c_int32),
        ("max_seq_len", C.c_int32),
        ("norm_eps", C.c_double),
        ("force_f16", C.c_int32),
    ]


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (oracle/Makefile)."""
    src = os.path.join(_HERE, "rllama_oracle.c")
    hdr = os.path.join(_HERE, "rllama_oracle.h")
    stale = (not os.path.exists(_SO)) or any(
        os.path.getmtime(f) > os.path.getmtime(_SO) for f in (src, hdr)
    )
    if force or stale:
        if force:
            subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
        subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_SO):
        build()
    L = C.CDLL(_SO)
    fp = C.POINTER(C.c_float)
    u16p = C.POINTER(C.c_uint16)
    dp = C.POINTER(C.c_double)
    i32p = C.POINTER(C.c_int32)
    vp = C.c_void_p
    sig = {
        "orc_f32_to_f16_bits": (C.c_uint16, [C.c_float]),
        "orc_f16_bits_to_f32": (C.c_float, [C.c_uint16]),
        "orc_f32_to_f16_hw": (C.c_uint16, [C.c_float]),
        "orc_f16_to_f32_hw": (C.c_float, [C.c_uint16]),
        "orc_f32_to_f16_array": (None, [fp, u16p, C.c_size_t]),
        "orc_f16_to_f32_array": (None, [u16p, fp, C.c_size_t]),
        "orc_hsum8": (C.c_float, [fp]),
        "orc_dot8_f32": (C.c_float, [fp, fp, C.c_int]),
        "orc_dot8_f16": (C.c_float, [u16p, u16p, C.c_int]),
        "orc_dot8_f32_scalar": (C.c_float, [fp, fp, C.c_int]),
        "orc_matmul_transposed_f32": (None, [fp, C.c_int, fp, C.c_int, C.c_int, fp]),
        "orc_matmul_transposed_f16": (None, [u16p, C.c_int, u16p, C.c_int, C.c_int, u16p]),
        "orc_matmul_f32_seqk": (None, [fp, C.c_int, fp, C.c_int, C.c_int, fp]),
        "orc_vector_matrix_mul_f32": (None, [fp, fp, C.c_int, C.c_int, fp]),
        "orc_rmsnorm_row": (None, [fp, fp, C.c_int, C.c_double, fp]),
        "orc_softmax_row": (None, [fp, C.c_int, fp]),
        "orc_silu": (C.c_float, [C.c_float]),
        "orc_freqs_cis": (None, [C.c_int, C.c_int, C.c_double, dp]),
        "orc_rope_row": (None, [fp, C.c_int, C.c_int, dp]),
        "orc_sample_greedy": (C.c_int32, [fp, C.c_int, C.c_float, fp, i32p]),
        "orc_sample_candidates": (C.c_int32, [fp, C.c_int, C.c_float, C.c_float, C.c_int32, C.c_float, i32p, C.c_int32, i32p, fp, fp]),
        "orc_sample_pick": (C.c_int32, [i32p, fp, C.c_int32, C.c_float, C.c_float, fp]),
        "orc_set_threads": (None, [C.c_int]),
        "orc_get_threads": (C.c_int, []),
        "orc_set_reference_threading": (None, [C.c_int]),
        "orc_set_alt_order": (None, [C.c_int]),
        "orc_set_exact_sums": (None, [C.c_int]),
        "orc_model_create": (vp, [C.POINTER(Params)]),
        "orc_model_free": (None, [vp]),
        "orc_model_set_tensor": (C.c_int, [vp, C.c_int, C.c_int, vp, C.c_int, C.c_int, C.c_int]),
        "orc_caches_create": (vp, [vp]),
        "orc_caches_true_clone": (vp, [vp]),
        "orc_caches_shift_left": (None, [vp, C.c_int]),
        "orc_caches_free": (None, [vp]),
        "orc_caches_read": (None, [vp, C.c_int, C.c_int, C.c_int, fp]),
        "orc_forward": (C.c_int, [vp, vp, i32p, C.c_int, C.c_int, fp]),
        "orc_embed": (C.c_int, [vp, i32p, C.c_int, fp]),
        "orc_forward_layers": (C.c_int, [vp, vp, fp, C.c_int, C.c_int, C.c_int, C.c_int, fp]),
        "orc_head": (C.c_int, [vp, fp, C.c_int, fp]),
        "orc_set_layer_tap": (None, [fp]),
    }
    for name, (res, args) in sig.items():
        f = getattr(L, name)
        f.restype = res
        f.argtypes = args
    _lib = L
    return L


def _fp(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _u16p(a):
    return a.ctypes.data_as(C.POINTER(C.c_uint16))


# ---- thin numpy wrappers over the building blocks ---------------------------------------------

def f32_to_f16_bits(a: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float32)
    out = np.empty(a.shape, dtype=np.uint16)
    lib().orc_f32_to_f16_array(_fp(a), _u16p(out), a.size)
    return out


def f16_bits_to_f32(a: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.uint16)
    out = np.empty(a.shape, dtype=np.float32)
    lib().orc_f16_to_f32_array(_u16p(a), _fp(out), a.size)
    return out


def f16r(a: np.ndarray) -> np.ndarray:
    return f16_bits_to_f32(f32_to_f16_bits(a))


def dot8_f32(a, b) -> float:
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    assert a.size == b.size
    return float(lib().orc_dot8_f32(_fp(a), _fp(b), a.size))


def dot8_f32_scalar(a, b) -> float:
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    return float(lib().orc_dot8_f32_scalar(_fp(a), _fp(b), a.size))


def dot8_f16(a_bits, b_bits) -> float:
    a = np.ascontiguousarray(a_bits, dtype=np.uint16)
    b = np.ascontiguousarray(b_bits, dtype=np.uint16)
    return float(lib().orc_dot8_f16(_u16p(a), _u16p(b), a.size))


def matmul_transposed_f32(x, w) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    n, k = x.shape
    nw, k2 = w.shape
    assert k == k2
    out = np.empty((n, nw), dtype=np.float32)
    lib().orc_matmul_transposed_f32(_fp(x), n, _fp(w), nw, k, _fp(out))
    return out


def matmul_transposed_f16(x_bits, w_bits) -> np.ndarray:
    x = np.ascontiguousarray(x_bits, dtype=np.uint16)
    w = np.ascontiguousarray(w_bits, dtype=np.uint16)
    n, k = x.shape
    nw, k2 = w.shape
    assert k == k2
    out = np.empty((n, nw), dtype=np.uint16)
    lib().orc_matmul_transposed_f16(_u16p(x), n, _u16p(w), nw, k, _u16p(out))
    return out


def matmul_f32_seqk(a, b) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    m, k = a.shape
    k2, n = b.shape
    assert k == k2
    out = np.empty((m, n), dtype=np.float32)
    lib().orc_matmul_f32_seqk(_fp(a), m, _fp(b), n, k, _fp(out))
    return out


def vector_matrix_mul_f32(a, b) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    k, n = b.shape
    assert a.size == k
    out = np.empty(n, dtype=np.float32)
    lib().orc_vector_matrix_mul_f32(_fp(a), _fp(b), k, n, _fp(out))
    return out


def rmsnorm_row(x, w, eps: float) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    out = np.empty_like(x)
    lib().orc_rmsnorm_row(_fp(x), _fp(w), x.size, eps, _fp(out))
    return out


def softmax_row(s) -> np.ndarray:
    s = np.ascontiguousarray(s, dtype=np.float32)
    out = np.empty_like(s)
    lib().orc_softmax_row(_fp(s), s.size, _fp(out))
    return out


def silu(v: float) -> float:
    return float(lib().orc_silu(float(v)))


def freqs_cis(head_dim: int, max_seq_len: int, theta: float = 10000.0) -> np.ndarray:
    out = np.empty((max_seq_len, head_dim // 2, 2), dtype=np.float64)
    lib().orc_freqs_cis(head_dim, max_seq_len, theta, out.ctypes.data_as(C.POINTER(C.c_double)))
    return out


def rope_row(x, n_heads: int, head_dim: int, fc_at_pos) -> np.ndarray:
    x = np.array(x, dtype=np.float32).reshape(n_heads * head_dim).copy()
    fc = np.ascontiguousarray(fc_at_pos, dtype=np.float64)
    lib().orc_rope_row(_fp(x), n_heads, head_dim, fc.ctypes.data_as(C.POINTER(C.c_double)))
    return x


def sample_greedy(logits, temperature: float = 1.0):
    """Returns (token id, probability, number of ids tied at the top probability)."""
    l = np.ascontiguousarray(logits, dtype=np.float32).reshape(-1)
    prob = C.c_float(0)
    ties = C.c_int32(0)
    tok = lib().orc_sample_greedy(_fp(l), l.size, temperature, C.byref(prob), C.byref(ties))
    return int(tok), float(prob.value), int(ties.value)


def sample_candidates(logits, temperature: float, top_p: float, top_k: int, repetition_penalty: float, existing_tokens=()):
    """token_sampler.rs:83-159: (ids, probabilities, total_p) of the candidates the draw chooses from, in draw order."""
    l = np.ascontiguousarray(logits, dtype=np.float32).reshape(-1)
    ex = np.ascontiguousarray(existing_tokens, dtype=np.int32).reshape(-1)
    cap = max(1, min(int(top_k), l.size))
    ids = np.zeros(cap, np.int32)
    probs = np.zeros(cap, np.float32)
    tot = C.c_float(0)
    n = lib().orc_sample_candidates(_fp(l), l.size, temperature, top_p, int(min(top_k, 2**31 - 1)), repetition_penalty,
                                    ex.ctypes.data_as(C.POINTER(C.c_int32)), ex.size, ids.ctypes.data_as(C.POINTER(C.c_int32)), _fp(probs), C.byref(tot))
    return ids[:n].copy(), probs[:n].copy(), float(tot.value)


def sample_pick(ids, probs, total_p: float, u: float):
    """token_sampler.rs:160-173 with the uniform variate u in [0, 1] passed in. Returns (token id, probability / total_p)."""
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    probs = np.ascontiguousarray(probs, dtype=np.float32)
    prob = C.c_float(0)
    tok = lib().orc_sample_pick(ids.ctypes.data_as(C.POINTER(C.c_int32)), _fp(probs), ids.size, total_p, u, C.byref(prob))
    return int(tok), float(prob.value)


def set_threads(n: int) -> None:
    lib().orc_set_threads(n)


def set_alt_order(on: bool) -> None:
    """Sensitivity probe: f16 projections summed in another valid fp32 order (NOT the reference's values)."""
    lib().orc_set_alt_order(1 if on else 0)


def set_exact_sums(on: bool) -> None:
    """Second probe: every sum accumulated in float64 and rounded once (NOT the reference's values; same rounding points)."""
    lib().orc_set_exact_sums(1 if on else 0)


def set_reference_threading(on: bool) -> None:
    lib().orc_set_reference_threading(1 if on else 0)


# ---- model level ---------------------------------------------------------------------------------

class Caches:
    def __init__(self, handle, model):
        self._h = handle
        self._model = model

    def true_clone(self) -> "Caches":
        return Caches(lib().orc_caches_true_clone(self._h), self._model)

    def shift_left(self, shifts: int) -> None:
        lib().orc_caches_shift_left(self._h, shifts)

    def read(self, layer: int, head: int, which: int) -> np.ndarray:
        """[head_dim x max_seq_len] f32; which: 0 = K, 1 = V."""
        m = self._model
        out = np.empty((m.head_dim, m.params.max_seq_len), dtype=np.float32)
        lib().orc_caches_read(self._h, layer, head, which, _fp(out))
        return out

    def __del__(self):
        if getattr(self, "_h", None):
            lib().orc_caches_free(self._h)
            self._h = None


class Model:
    """Oracle twin of rllama's Transformer (transformer.rs:17-34)."""

    def __init__(self, dim, n_layers, n_heads, ffn_hidden, vocab_size, max_seq_len, norm_eps, force_f16):
        self.params = Params(dim, n_layers, n_heads, ffn_hidden, vocab_size, max_seq_len, norm_eps, 1 if force_f16 else 0)
        self.head_dim = dim // n_heads
        self._h = lib().orc_model_create(C.byref(self.params))
        if not self._h:
            raise ValueError("orc_model_create failed (dim % n_heads != 0?)")

    def set_tensor(self, kind: int, layer: int, arr: np.ndarray) -> None:
        """arr: uint16 (f16 bits) or float32, shape [rows, cols] (1-D norms as [dim])."""
        if arr.dtype == np.uint16:
            dt = F16
        elif arr.dtype == np.float32:
            dt = F32
        else:
            raise TypeError(arr.dtype)
        a = np.ascontiguousarray(arr)
        if a.ndim == 1:
            a = a.reshape(1, -1)
        rc = lib().orc_model_set_tensor(self._h, kind, layer, a.ctypes.data_as(C.c_void_p), a.shape[0], a.shape[1], dt)
        if rc != 0:
            raise ValueError(f"orc_model_set_tensor(kind={kind}, layer={layer}, shape={a.shape}) -> {rc}")

    def make_caches(self) -> Caches:
        return Caches(lib().orc_caches_create(self._h), self)

    def forward(self, tokens, start_pos: int, caches: Caches, layer_tap: bool = False):
        toks = np.ascontiguousarray(tokens, dtype=np.int32)
        logits = np.empty(self.params.vocab_size, dtype=np.float32)
        tap = None
        if layer_tap:
            tap = np.zeros((self.params.n_layers, toks.size, self.params.dim), dtype=np.float32)
            lib().orc_set_layer_tap(_fp(tap))
        try:
            rc = lib().orc_forward(self._h, caches._h, toks.ctypes.data_as(C.POINTER(C.c_int32)), toks.size, start_pos, _fp(logits))
        finally:
            if layer_tap:
                lib().orc_set_layer_tap(None)
        if rc != 0:
            raise RuntimeError(f"orc_forward -> {rc} (the reference panics here)")
        return (logits, tap) if layer_tap else logits

    # the forward cut at the reference's layer split (transformer.rs:262-279): embed -> forward_layers(...) -> head
    def embed(self, tokens) -> np.ndarray:
        toks = np.ascontiguousarray(tokens, dtype=np.int32)
        x = np.empty((toks.size, self.params.dim), dtype=np.float32)
        rc = lib().orc_embed(self._h, toks.ctypes.data_as(C.POINTER(C.c_int32)), toks.size, _fp(x))
        if rc != 0:
            raise RuntimeError(f"orc_embed -> {rc}")
        return x

    def forward_layers(self, x: np.ndarray, start_pos: int, caches: Caches, first_layer: int, last_layer: int) -> np.ndarray:
        xin = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, self.params.dim)
        out = np.empty_like(xin)
        rc = lib().orc_forward_layers(self._h, caches._h, _fp(xin), xin.shape[0], start_pos, first_layer, last_layer, _fp(out))
        if rc != 0:
            raise RuntimeError(f"orc_forward_layers -> {rc}")
        return out

    def head(self, x: np.ndarray) -> np.ndarray:
        xin = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, self.params.dim)
        logits = np.empty(self.params.vocab_size, dtype=np.float32)
        rc = lib().orc_head(self._h, _fp(xin), xin.shape[0], _fp(logits))
        if rc != 0:
            raise RuntimeError(f"orc_head -> {rc}")
        return logits

    def __del__(self):
        if getattr(self, "_h", None):
            lib().orc_model_free(self._h)
            self._h = None
