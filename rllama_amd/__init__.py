"""rllama_amd -- rllama's per-token transformer forward path on one MI355X (gfx950).

The product is ``librllama_hip.so`` (C ABI in ``include/rllama_hip.h``; HIP kernels in ``rllama_amd/csrc``).
This package is a thin ctypes binding that keeps the reference's names -- ``Transformer``,
``TransformerCaches``, ``Tensor``, ``DataSettings`` (Noeda/rllama ``src/transformer.rs``, ``src/tensor.rs``) --
so that tests and the benchmark read like the reference's call sites.  It holds no arithmetic and no CPU
fallback: every method is one call into the library, and a missing library or device raises.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence, Tuple

import numpy as np

from . import _lib
from ._lib import ModelParams, RllamaHipError, check

__all__ = [
    "DataSettings", "Transformer", "TransformerCaches", "Tensor", "TensorDType", "Context",
    "RllamaHipError", "synth_normal_f16", "synth_tokens", "llama_ffn_hidden",
]

TOK_EMB, WQ, WK, WV, WO, W1, W2, W3, ATTN_NORM, FFN_NORM, NORM, OUTPUT = range(12)


class TensorDType:
    """TensorDType of src/tensor.rs:50-54 (the 4-bit variant is unimplemented in the reference too)."""
    Float16 = 0
    Float32 = 1


def llama_ffn_hidden(dim: int, multiple_of: int = 256) -> int:
    """LLaMA's FFN width rule: 2/3 * 4 * dim rounded up to multiple_of (the reference reads it off w1's shape)."""
    hidden = int(2 * (4 * dim) / 3)
    return multiple_of * ((hidden + multiple_of - 1) // multiple_of)


class Context:
    """The device context: OpenCL::new(verbose, nth_device) of src/tensor_opencl_support.rs:86."""

    def __init__(self, nth_device: int = 0, verbose: bool = False):
        self._lib = _lib.load()
        h = C.c_void_p()
        check(self._lib.rlh_init(nth_device, 1 if verbose else 0, C.byref(h)))
        self._h = h

    def flush(self) -> None:
        check(self._lib.rlh_sync(self._h))

    sync = flush

    def set_option(self, name: str, value=None) -> None:
        """One of the library's switches (NAME of the RLLAMA_HIP_<NAME> variables rlh_init reads once); None = its default."""
        check(self._lib.rlh_set_option(self._h, name.encode(), None if value is None else str(value).encode()))

    def device_info(self):
        name = C.create_string_buffer(256)
        cus = C.c_int()
        hbm = C.c_uint64()
        check(self._lib.rlh_device_info(self._h, name, 256, C.byref(cus), C.byref(hbm)))
        return {"name": name.value.decode(), "compute_units": cus.value, "hbm_bytes": hbm.value}

    def event(self) -> "Event":
        h = C.c_void_p()
        check(self._lib.rlh_event_record(self._h, C.byref(h)))
        return Event(self._lib, h)

    def time_gemv(self, rows: int, k: int, dtype: int = 0, round_x: bool = False, round_y: bool = False,
                  n_buffers: int = 12, iters: int = 200) -> float:
        """Microseconds per launch of the isolated GEMV, cycling through n_buffers distinct weight matrices."""
        us = C.c_float()
        check(self._lib.rlh_time_gemv(self._h, rows, k, dtype, 1 if round_x else 0, 1 if round_y else 0, n_buffers, iters, C.byref(us)))
        return us.value

    GEMV_PHASES = ("gap_after_previous_launch", "dispatch_ramp", "prologue", "first_byte_latency", "streaming", "epilogue", "tail_skew", "first_entry_to_last_exit")

    def probe_gemv_phases(self, rows: int, k: int, n_buffers: int = 12, launches: int = 64):
        """Microseconds of each phase of the isolated f16 GEMV launch, from wall-clock readings inside the kernel."""
        out = (C.c_float * 8)()
        check(self._lib.rlh_probe_gemv_phases(self._h, rows, k, n_buffers, launches, out))
        return dict(zip(self.GEMV_PHASES, (round(float(v), 3) for v in out)))

    def close(self) -> None:
        """Ends the context.  Handles made from it are dead afterwards (their free() becomes a no-op)."""
        if getattr(self, "_h", None):
            self._lib.rlh_shutdown(self._h)
            self._h = None


class Event:
    def __init__(self, lib, h):
        self._lib, self._h = lib, h

    def elapsed_ms(self, stop: "Event") -> float:
        ms = C.c_float()
        check(self._lib.rlh_event_elapsed_ms(self._h, stop._h, C.byref(ms)))
        return ms.value

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.rlh_event_free(self._h)
            self._h = None


class DataSettings:
    """DataSettings of src/transformer.rs:38-109: builder-style switches for where and how weights live."""

    def __init__(self, ctx: Optional[Context] = None):
        self.ctx = ctx
        self._force_f16 = False
        self._percentage_to_gpu = 1.0

    def force_f16(self) -> "DataSettings":
        self._force_f16 = True
        return self

    def percentage_to_gpu(self, percentage: float) -> "DataSettings":
        self._percentage_to_gpu = float(percentage)  # clamped by the library like transformer.rs:91-103
        return self


class TransformerCaches:
    """TransformerCaches of src/transformer.rs:111-113, 200-214; resident in HBM."""

    def __init__(self, model: "Transformer", handle):
        self._model = model
        self._lib = model._lib
        self._h = handle

    def true_clone(self) -> "TransformerCaches":
        h = C.c_void_p()
        check(self._lib.rlh_caches_true_clone(self._h, C.byref(h)))
        return TransformerCaches(self._model, h)

    def shift_left(self, shifts: int) -> None:
        check(self._lib.rlh_caches_shift_left(self._h, shifts))

    def read(self, layer: int, head: int, which: int) -> np.ndarray:
        """Test hook: [head_dim x max_seq_len] f32 in the reference's orientation; which: 0 = K, 1 = V."""
        m = self._model
        out = np.empty((m.head_dim, m.max_seq_len), dtype=np.float32)
        check(self._lib.rlh_caches_read(self._h, layer, head, which, out.ctypes.data_as(C.POINTER(C.c_float))))
        return out

    def free(self) -> None:
        if getattr(self, "_h", None):
            if self._model.ctx._h:
                self._lib.rlh_caches_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Transformer:
    """Transformer of src/transformer.rs:17-34, 240-383."""

    def __init__(self, ctx: Context, dim: int, n_layers: int, n_heads: int, ffn_hidden: int, vocab_size: int,
                 max_seq_len: int, norm_eps: float, data_settings: Optional[DataSettings] = None):
        ds = data_settings or DataSettings(ctx)
        self.ctx = ctx
        self._lib = ctx._lib
        self.dim, self.n_layers, self.n_heads = dim, n_layers, n_heads
        self.ffn_hidden, self.vocab_size, self.max_seq_len = ffn_hidden, vocab_size, max_seq_len
        self.head_dim = dim // n_heads
        self.force_f16 = ds._force_f16
        self.params = ModelParams(dim, n_layers, n_heads, ffn_hidden, vocab_size, max_seq_len, norm_eps,
                                  1 if ds._force_f16 else 0, ds._percentage_to_gpu)
        h = C.c_void_p()
        check(self._lib.rlh_model_create(ctx._h, C.byref(self.params), C.byref(h)))
        self._h = h

    # -- weights ---------------------------------------------------------------------------------
    def set_tensor(self, kind: int, layer: int, arr: np.ndarray) -> None:
        """arr: uint16 (IEEE f16 bits, as stored in consolidated.NN/data/*) or float32; 1-D norms allowed."""
        if arr.dtype == np.uint16:
            dt = TensorDType.Float16
        elif arr.dtype == np.float32:
            dt = TensorDType.Float32
        else:
            raise TypeError(f"unsupported dtype {arr.dtype}")
        a = np.ascontiguousarray(arr)
        if a.ndim == 1:
            a = a.reshape(1, -1)
        check(self._lib.rlh_model_set_tensor(self._h, kind, layer, a.ctypes.data_as(C.c_void_p), a.shape[0], a.shape[1], dt))

    def get_tensor(self, kind: int, layer: int, rows: int, cols: int, as_f16_bits: bool = False) -> np.ndarray:
        """The stored weight as float32, or as uint16 IEEE f16 bits."""
        out = np.empty((rows, cols), dtype=np.uint16 if as_f16_bits else np.float32)
        check(self._lib.rlh_model_get_tensor(self._h, kind, layer, out.ctypes.data_as(C.c_void_p), rows, cols,
                                             TensorDType.Float16 if as_f16_bits else TensorDType.Float32))
        return out

    def fill_synthetic(self, seed: int = 0, std: float = 0.02) -> None:
        check(self._lib.rlh_model_fill_synthetic(self._h, seed, std))

    def set_prefill_mode(self, token_by_token: bool) -> None:
        """False (default): matrix-core prefill for n > 1 in f16 mode.  True: the decode kernels for every prompt token."""
        check(self._lib.rlh_model_set_prefill_mode(self._h, 1 if token_by_token else 0))

    def last_layer_on_gpu(self) -> int:
        v = C.c_int()
        check(self._lib.rlh_model_layers_on_gpu(self._h, C.byref(v)))
        return v.value

    def decode_bytes(self, T: int) -> int:
        v = C.c_uint64()
        check(self._lib.rlh_model_decode_bytes(self._h, T, C.byref(v)))
        return v.value

    # -- the reference's API ---------------------------------------------------------------------
    def make_caches(self) -> TransformerCaches:
        h = C.c_void_p()
        check(self._lib.rlh_caches_create(self._h, C.byref(h)))
        return TransformerCaches(self, h)

    def forward(self, tokens: Sequence[int], start_pos: int, caches: TransformerCaches) -> np.ndarray:
        """Returns the logits [vocab] (the reference returns a vocab x 1 f32 Tensor, transformer.rs:381)."""
        toks = np.ascontiguousarray(tokens, dtype=np.int32)
        logits = np.empty(self.vocab_size, dtype=np.float32)
        check(self._lib.rlh_forward(self._h, caches._h, toks.ctypes.data_as(C.POINTER(C.c_int32)), toks.size, start_pos,
                                    logits.ctypes.data_as(C.POINTER(C.c_float))))
        return logits

    def forward_layers(self, x: np.ndarray, start_pos: int, caches: TransformerCaches, first_layer: int, last_layer: int) -> np.ndarray:
        """Blocks first_layer..=last_layer on the n rows of the residual stream x [n x dim] f32 (the loop body of
        transformer.rs:361-376 for the layers percentage_to_gpu keeps on the device, :262-279). Returns the stream after them."""
        xin = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, self.dim)
        out = np.empty_like(xin)
        check(self._lib.rlh_forward_layers(self._h, caches._h, xin.ctypes.data_as(C.POINTER(C.c_float)), xin.shape[0], start_pos,
                                           first_layer, last_layer, out.ctypes.data_as(C.POINTER(C.c_float))))
        return out

    def forward_greedy(self, tokens: Sequence[int], start_pos: int, caches: TransformerCaches) -> int:
        toks = np.ascontiguousarray(tokens, dtype=np.int32)
        nxt = C.c_int32()
        check(self._lib.rlh_forward_greedy(self._h, caches._h, toks.ctypes.data_as(C.POINTER(C.c_int32)), toks.size, start_pos, C.byref(nxt)))
        return nxt.value

    def generate_greedy(self, prompt: Sequence[int], n_new: int, caches: TransformerCaches):
        """The token loop of src/rllama_main.rs:821-897 at top_k = 1. Returns (ids, ms_first, ms_per_token)."""
        toks = np.ascontiguousarray(prompt, dtype=np.int32)
        out = np.empty(n_new, dtype=np.int32)
        a, b = C.c_float(), C.c_float()
        check(self._lib.rlh_generate_greedy(self._h, caches._h, toks.ctypes.data_as(C.POINTER(C.c_int32)), toks.size, n_new,
                                            out.ctypes.data_as(C.POINTER(C.c_int32)), C.byref(a), C.byref(b)))
        return out, a.value, b.value

    def forward_sample(self, tokens: Sequence[int], start_pos: int, caches: TransformerCaches, sampler: "TokenSampler",
                       existing_tokens: Sequence[int], rng: np.random.Generator):
        """forward + TokenSampler::sample, the body of the token loop (src/rllama_main.rs:846-860). Returns (id, probability)."""
        toks = np.ascontiguousarray(tokens, dtype=np.int32)
        ex = np.ascontiguousarray(existing_tokens, dtype=np.int32).reshape(-1)
        tok, prob = C.c_int32(0), C.c_float(0)
        check(self._lib.rlh_forward_sample(self._h, caches._h, toks.ctypes.data_as(C.POINTER(C.c_int32)), toks.size, start_pos, C.byref(sampler._p),
                                           ex.ctypes.data_as(C.POINTER(C.c_int32)), ex.size, float(rng.random(dtype=np.float32)), C.byref(tok), C.byref(prob)))
        return int(tok.value), float(prob.value)

    def decode_greedy(self, n_steps: int, caches: TransformerCaches):
        """Continues the greedy loop on the device for n_steps tokens. Returns (ids, HIP-event ms for the n_steps)."""
        out = np.empty(n_steps, dtype=np.int32)
        ms = C.c_float()
        check(self._lib.rlh_decode_greedy(self._h, caches._h, n_steps, out.ctypes.data_as(C.POINTER(C.c_int32)), C.byref(ms)))
        return out, ms.value

    STEP_KERNELS = ("qkv_rope_kvwrite", "attn_decode", "wo_residual", "w13_silu", "w2_residual", "head")

    def time_kernel(self, which: int, T: int, iters: int, caches: TransformerCaches):
        """(microseconds per launch, algorithmic bytes per launch) of one token-step kernel, HIP-event timed."""
        us = C.c_float()
        nbytes = C.c_uint64()
        check(self._lib.rlh_model_time_kernel(self._h, caches._h, which, T, iters, C.byref(us), C.byref(nbytes)))
        return us.value, nbytes.value

    def free(self) -> None:
        if getattr(self, "_h", None):
            if self.ctx._h:
                self._lib.rlh_model_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Tensor:
    """A device tensor: the subset of src/tensor.rs's Tensor that the reference can hold on its GPU
    (OpenCLTensor, src/tensor_opencl_support.rs:23-38), dense row-major f16 or f32."""

    def __init__(self, ctx: Context, handle, rows: int, cols: int, dtype: int):
        self.ctx, self._lib, self._h = ctx, ctx._lib, handle
        self._rows, self._cols, self._dtype = rows, cols, dtype

    # constructors
    @staticmethod
    def from_numpy(ctx: Context, arr: np.ndarray) -> "Tensor":
        """to_gpu_inplace (src/tensor.rs:2127-2147): uint16 arrays are f16 bits, float32 arrays are f32."""
        if arr.dtype == np.uint16:
            dt = TensorDType.Float16
        elif arr.dtype == np.float32:
            dt = TensorDType.Float32
        elif arr.dtype == np.float16:
            arr, dt = arr.view(np.uint16), TensorDType.Float16
        else:
            raise TypeError(arr.dtype)
        a = np.ascontiguousarray(arr)
        if a.ndim == 1:
            a = a.reshape(1, -1)
        h = C.c_void_p()
        check(ctx._lib.rlh_tensor_upload(ctx._h, a.ctypes.data_as(C.c_void_p), a.shape[0], a.shape[1], a.shape[1], dt, C.byref(h)))
        return Tensor(ctx, h, a.shape[0], a.shape[1], dt)

    @staticmethod
    def zeros(ctx: Context, rows: int, cols: int, dtype: int) -> "Tensor":
        h = C.c_void_p()
        check(ctx._lib.rlh_tensor_alloc(ctx._h, rows, cols, dtype, C.byref(h)))
        return Tensor(ctx, h, rows, cols, dtype)

    def rows(self) -> int:
        return self._rows

    def cols(self) -> int:
        return self._cols

    def dtype(self) -> int:
        return self._dtype

    def to_numpy(self) -> np.ndarray:
        """to_cpu_inplace (src/tensor.rs:2150-2166): f16 tensors come back as float16 arrays."""
        out = np.empty((self._rows, self._cols), dtype=np.uint16 if self._dtype == TensorDType.Float16 else np.float32)
        check(self._lib.rlh_tensor_download(self._h, out.ctypes.data_as(C.c_void_p), self._cols, None))
        return out.view(np.float16) if self._dtype == TensorDType.Float16 else out

    # ops (src/tensor_opencl_support.rs:215-405 via src/tensor.rs wrappers)
    def _like(self, rows=None, cols=None) -> "Tensor":
        return Tensor.zeros(self.ctx, rows or self._rows, cols or self._cols, self._dtype)

    def clone(self) -> "Tensor":
        out = self._like()
        check(self._lib.rlh_copy_inplace(out._h, self._h))
        return out

    def transpose(self) -> "Tensor":
        out = Tensor.zeros(self.ctx, self._cols, self._rows, self._dtype)
        check(self._lib.rlh_transpose_from(out._h, self._h))
        return out

    def hadamard_product(self, other: "Tensor") -> "Tensor":
        out = self.clone()
        check(self._lib.rlh_hadamard_product_inplace(out._h, other._h))
        return out

    def silu(self) -> "Tensor":
        out = self.clone()
        check(self._lib.rlh_silu_inplace(out._h))
        return out

    def matrix_mul_transposed(self, other: "Tensor") -> "Tensor":
        """self [n x k] times other[m x k]^T -> [n x m] (src/tensor.rs:999-1025)."""
        out = Tensor.zeros(self.ctx, self._rows, other._rows, self._dtype)
        check(self._lib.rlh_matrix_mul_inplace_transposed(out._h, self._h, other._h))
        return out

    def gemv(self, x: "Tensor", round_x: bool, round_y: bool) -> "Tensor":
        """Decode product with the fused path's rounding switches: self = W [m x k], x f32 [1 x k] -> f32 [1 x m]."""
        out = Tensor.zeros(self.ctx, 1, self._rows, TensorDType.Float32)
        check(self._lib.rlh_gemv(out._h, self._h, x._h, 1 if round_x else 0, 1 if round_y else 0))
        return out

    def rmsnorm(self, weight: "Tensor", eps: float, round_y: bool = False) -> "Tensor":
        out = self._like()
        check(self._lib.rlh_rmsnorm(out._h, self._h, weight._h, eps, 1 if round_y else 0))
        return out

    def rope_inplace(self, n_heads: int, head_dim: int, pos: int) -> None:
        check(self._lib.rlh_rope_inplace(self._h, n_heads, head_dim, pos))

    # the host-side steps of the reference's attention block and token loop, as device ops
    def add(self, other: "Tensor") -> "Tensor":
        """Tensor::add (src/tensor.rs:573-593), f32."""
        out = self._like()
        check(self._lib.rlh_add(out._h, self._h, other._h))
        return out

    def silu_mul(self, up: "Tensor") -> "Tensor":
        """silu(self) * up with one rounding for f16 tensors (src/transformer.rs:557-565)."""
        out = self._like()
        check(self._lib.rlh_silu_mul(out._h, self._h, up._h))
        return out

    def ffn_gate(self, w1: "Tensor", w3: "Tensor") -> "Tensor":
        """self = x [n x k] f16: f16(silu(f16(x w1^T)) * f16(x w3^T)) for all rows at once (src/transformer.rs:551-565)."""
        out = Tensor.zeros(self.ctx, self._rows, w1._rows, TensorDType.Float16)
        check(self._lib.rlh_ffn_gate(out._h, self._h, w1._h, w3._h))
        return out

    def rope_kvwrite(self, k: "Tensor", v: "Tensor", cache_k: "Tensor", cache_v: "Tensor", n_heads: int, max_seq_len: int, pos: int) -> None:
        """self = q: RoPE on q (in place) and k at pos; k and v into the cache planes at pos (src/transformer.rs:704-761)."""
        check(self._lib.rlh_rope_kvwrite(self._h, k._h, v._h, cache_k._h, cache_v._h, n_heads, max_seq_len, pos))

    def attn_decode(self, cache_k: "Tensor", cache_v: "Tensor", n_heads: int, max_seq_len: int, T: int, n_splits: int = 0,
                    round_out: bool = False) -> "Tensor":
        """self = q after RoPE: single-query attention over positions 0..T-1 of the cache planes (src/transformer.rs:762-781)."""
        out = Tensor.zeros(self.ctx, 1, self._rows * self._cols, TensorDType.Float32)
        check(self._lib.rlh_attn_decode(out._h, self._h, cache_k._h, cache_v._h, n_heads, max_seq_len, T, n_splits, 1 if round_out else 0))
        return out

    def attn_decode_noalloc(self, out: "Tensor", cache_k: "Tensor", cache_v: "Tensor", n_heads: int, max_seq_len: int, T: int,
                            n_splits: int = 0, round_out: bool = False) -> None:
        """attn_decode into a tensor the caller made, on the library's static work memory: the call allocates nothing."""
        check(self._lib.rlh_attn_decode_noalloc(out._h, self._h, cache_k._h, cache_v._h, n_heads, max_seq_len, T, n_splits, 1 if round_out else 0))

    def attn_prefill(self, cache_k: "Tensor", cache_v: "Tensor", n_heads: int, max_seq_len: int) -> "Tensor":
        """self = qkv f16 [n x 3 dim]: RoPE, cache write and causal attention of a prompt (src/transformer.rs:704-796) -> f16 [n x dim]."""
        out = Tensor.zeros(self.ctx, self._rows, self._cols // 3, TensorDType.Float16)
        check(self._lib.rlh_attn_prefill(out._h, self._h, cache_k._h, cache_v._h, n_heads, max_seq_len))
        return out

    def argmax_greedy(self, temperature: float = 1.0) -> int:
        """TokenSampler::sample at top_k = 1 on device logits (src/token_sampler.rs:83-174)."""
        tok = C.c_int32()
        check(self._lib.rlh_argmax_greedy(self._h, float(temperature), C.byref(tok)))
        return int(tok.value)

    def free(self) -> None:
        if getattr(self, "_h", None):
            if self.ctx._h:
                self._lib.rlh_tensor_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class TokenSampler:
    """TokenSampler (src/token_sampler.rs:6-174): builder-style settings, sampling done by the library's host arithmetic.
    The uniform variate comes from the caller's generator (the reference draws from rand::thread_rng)."""

    def __init__(self):
        self._p = _lib.SamplerParams()
        _lib.load().rlh_sampler_default(C.byref(self._p))  # TokenSampler::new(), :20-29

    def _with(self, **kw) -> "TokenSampler":
        t = TokenSampler()
        t._p = _lib.SamplerParams(self._p.temperature, self._p.top_p, self._p.top_k, self._p.repetition_penalty)
        for k, v in kw.items():
            setattr(t._p, k, v)
        return t

    def temperature(self, v: float) -> "TokenSampler":
        return self._with(temperature=v)

    def top_p(self, v: float) -> "TokenSampler":
        return self._with(top_p=v)

    def top_k(self, v: int) -> "TokenSampler":
        return self._with(top_k=int(min(v, 2**31 - 1)))

    def repetition_penalty(self, v: float) -> "TokenSampler":
        return self._with(repetition_penalty=v)

    def get_temperature(self) -> float:
        return self._p.temperature

    def get_top_p(self) -> float:
        return self._p.top_p

    def get_top_k(self) -> int:
        return self._p.top_k

    def get_repetition_penalty(self) -> float:
        return self._p.repetition_penalty

    @staticmethod
    def _existing(existing_tokens):
        ex = np.ascontiguousarray(existing_tokens, dtype=np.int32).reshape(-1)
        return ex, ex.ctypes.data_as(C.POINTER(C.c_int32))

    def candidates(self, logits: np.ndarray, existing_tokens: Sequence[int] = ()):
        """(ids, probabilities, total_p) of what the draw chooses from, in draw order (:83-159)."""
        l = np.ascontiguousarray(logits, dtype=np.float32).reshape(-1)
        ex, exp_ = self._existing(existing_tokens)
        cap = max(1, min(self._p.top_k, l.size))
        ids, probs = np.zeros(cap, np.int32), np.zeros(cap, np.float32)
        n, tot = C.c_int(0), C.c_float(0)
        check(_lib.load().rlh_sample_candidates(l.ctypes.data_as(C.POINTER(C.c_float)), l.size, C.byref(self._p), exp_, ex.size,
                                                ids.ctypes.data_as(C.POINTER(C.c_int32)), probs.ctypes.data_as(C.POINTER(C.c_float)), cap,
                                                C.byref(n), C.byref(tot)))
        return ids[:n.value].copy(), probs[:n.value].copy(), float(tot.value)

    def sample(self, logits: np.ndarray, existing_tokens: Sequence[int], rng: np.random.Generator) -> Tuple[int, float]:
        """sample(logits, tokenizer, existing_tokens) -> (token id, probability) (:83-174)."""
        l = np.ascontiguousarray(logits, dtype=np.float32).reshape(-1)
        ex, exp_ = self._existing(existing_tokens)
        tok, prob = C.c_int32(0), C.c_float(0)
        check(_lib.load().rlh_sample(l.ctypes.data_as(C.POINTER(C.c_float)), l.size, C.byref(self._p), exp_, ex.size, float(rng.random(dtype=np.float32)),
                                     C.byref(tok), C.byref(prob)))
        return int(tok.value), float(prob.value)


# -- synthetic inputs (host side of csrc/synth.h; needs no device) --------------------------------------

def synth_normal_f16(seed: int, kind: int, layer: int, count: int, first_index: int = 0, std: float = 0.02) -> np.ndarray:
    """f16 bits of `count` i.i.d. N(0, std^2) values of tensor (kind, layer) starting at element first_index."""
    out = np.empty(count, dtype=np.uint16)
    _lib.load().rlh_synth_normal_f16(seed, kind, layer, first_index, count, std, out.ctypes.data_as(C.POINTER(C.c_uint16)))
    return out


def synth_tokens(seed: int, count: int, lo: int = 3, hi: int = 32000, first_index: int = 0) -> np.ndarray:
    out = np.empty(count, dtype=np.int32)
    _lib.load().rlh_synth_tokens(seed, first_index, count, lo, hi, out.ctypes.data_as(C.POINTER(C.c_int32)))
    return out
