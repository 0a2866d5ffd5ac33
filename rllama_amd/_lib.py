"""Loader of librllama_hip.so.  There is no fallback: if the library is missing or a call fails, it raises."""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# RLLAMA_HIP_LIB names another build of the same library (e.g. a variant under test)
LIB_PATH = os.environ.get("RLLAMA_HIP_LIB") or os.path.join(HERE, "librllama_hip.so")
HEADER_PATH = os.path.join(os.path.dirname(HERE), "include", "rllama_hip.h")


class RllamaHipError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"[rlh status {code}] {message}")
        self.code = code


class ModelParams(C.Structure):
    _fields_ = [
        ("dim", C.c_int32),
        ("n_layers", C.c_int32),
        ("n_heads", C.c_int32),
        ("ffn_hidden", C.c_int32),
        ("vocab_size", C.c_int32),
        ("max_seq_len", C.c_int32),
        ("norm_eps", C.c_double),
        ("force_f16", C.c_int32),
        ("percentage_to_gpu", C.c_float),
    ]


class SamplerParams(C.Structure):
    _fields_ = [("temperature", C.c_float), ("top_p", C.c_float), ("top_k", C.c_int32), ("repetition_penalty", C.c_float)]


_vp = C.c_void_p
_vpp = C.POINTER(C.c_void_p)
_i32p = C.POINTER(C.c_int32)
_fp = C.POINTER(C.c_float)
_ip = C.POINTER(C.c_int)

# name -> (restype, argtypes); one entry per declaration in include/rllama_hip.h
SIGNATURES = {
    "rlh_init": (C.c_int, [C.c_int, C.c_int, _vpp]),
    "rlh_shutdown": (None, [_vp]),
    "rlh_sync": (C.c_int, [_vp]),
    "rlh_last_error": (C.c_char_p, []),
    "rlh_set_option": (C.c_int, [_vp, C.c_char_p, C.c_char_p]),
    "rlh_device_info": (C.c_int, [_vp, C.c_char_p, C.c_int, _ip, C.POINTER(C.c_uint64)]),
    "rlh_model_create": (C.c_int, [_vp, C.POINTER(ModelParams), _vpp]),
    "rlh_model_free": (None, [_vp]),
    "rlh_model_set_tensor": (C.c_int, [_vp, C.c_int, C.c_int, _vp, C.c_int, C.c_int, C.c_int]),
    "rlh_model_get_tensor": (C.c_int, [_vp, C.c_int, C.c_int, _vp, C.c_int, C.c_int, C.c_int]),
    "rlh_model_fill_synthetic": (C.c_int, [_vp, C.c_uint64, C.c_double]),
    "rlh_model_set_prefill_mode": (C.c_int, [_vp, C.c_int]),
    "rlh_model_layers_on_gpu": (C.c_int, [_vp, _ip]),
    "rlh_model_decode_bytes": (C.c_int, [_vp, C.c_int, C.POINTER(C.c_uint64)]),
    "rlh_caches_create": (C.c_int, [_vp, _vpp]),
    "rlh_caches_true_clone": (C.c_int, [_vp, _vpp]),
    "rlh_caches_shift_left": (C.c_int, [_vp, C.c_int]),
    "rlh_caches_free": (None, [_vp]),
    "rlh_caches_read": (C.c_int, [_vp, C.c_int, C.c_int, C.c_int, _fp]),
    "rlh_forward": (C.c_int, [_vp, _vp, _i32p, C.c_int, C.c_int, _fp]),
    "rlh_forward_greedy": (C.c_int, [_vp, _vp, _i32p, C.c_int, C.c_int, _i32p]),
    "rlh_forward_layers": (C.c_int, [_vp, _vp, _fp, C.c_int, C.c_int, C.c_int, C.c_int, _fp]),
    "rlh_generate_greedy": (C.c_int, [_vp, _vp, _i32p, C.c_int, C.c_int, _i32p, _fp, _fp]),
    "rlh_decode_greedy": (C.c_int, [_vp, _vp, C.c_int, _i32p, _fp]),
    "rlh_sampler_default": (None, [C.POINTER(SamplerParams)]),
    "rlh_sample_candidates": (C.c_int, [_fp, C.c_int, C.POINTER(SamplerParams), _i32p, C.c_int, _i32p, _fp, C.c_int, _ip, _fp]),
    "rlh_sample": (C.c_int, [_fp, C.c_int, C.POINTER(SamplerParams), _i32p, C.c_int, C.c_float, _i32p, _fp]),
    "rlh_forward_sample": (C.c_int, [_vp, _vp, _i32p, C.c_int, C.c_int, C.POINTER(SamplerParams), _i32p, C.c_int, C.c_float, _i32p, _fp]),
    "rlh_tensor_upload": (C.c_int, [_vp, _vp, C.c_int, C.c_int, C.c_int, C.c_int, _vpp]),
    "rlh_tensor_alloc": (C.c_int, [_vp, C.c_int, C.c_int, C.c_int, _vpp]),
    "rlh_tensor_download": (C.c_int, [_vp, _vp, C.c_int, _vpp]),
    "rlh_tensor_free": (None, [_vp]),
    "rlh_tensor_shape": (C.c_int, [_vp, _ip, _ip, _ip]),
    "rlh_event_wait": (C.c_int, [_vp]),
    "rlh_event_record": (C.c_int, [_vp, _vpp]),
    "rlh_event_elapsed_ms": (C.c_int, [_vp, _vp, _fp]),
    "rlh_event_free": (None, [_vp]),
    "rlh_copy_inplace": (C.c_int, [_vp, _vp]),
    "rlh_transpose_from": (C.c_int, [_vp, _vp]),
    "rlh_hadamard_product_inplace": (C.c_int, [_vp, _vp]),
    "rlh_silu_inplace": (C.c_int, [_vp]),
    "rlh_matrix_mul_inplace_transposed": (C.c_int, [_vp, _vp, _vp]),
    "rlh_gemv": (C.c_int, [_vp, _vp, _vp, C.c_int, C.c_int]),
    "rlh_rmsnorm": (C.c_int, [_vp, _vp, _vp, C.c_double, C.c_int]),
    "rlh_rope_inplace": (C.c_int, [_vp, C.c_int, C.c_int, C.c_int]),
    "rlh_add": (C.c_int, [_vp, _vp, _vp]),
    "rlh_silu_mul": (C.c_int, [_vp, _vp, _vp]),
    "rlh_ffn_gate": (C.c_int, [_vp, _vp, _vp, _vp]),
    "rlh_rope_kvwrite": (C.c_int, [_vp, _vp, _vp, _vp, _vp, C.c_int, C.c_int, C.c_int]),
    "rlh_attn_decode": (C.c_int, [_vp, _vp, _vp, _vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]),
    "rlh_attn_decode_noalloc": (C.c_int, [_vp, _vp, _vp, _vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]),
    "rlh_attn_prefill": (C.c_int, [_vp, _vp, _vp, _vp, C.c_int, C.c_int]),
    "rlh_argmax_greedy": (C.c_int, [_vp, C.c_float, _i32p]),
    "rlh_model_time_kernel": (C.c_int, [_vp, _vp, C.c_int, C.c_int, C.c_int, _fp, C.POINTER(C.c_uint64)]),
    "rlh_time_gemv": (C.c_int, [_vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _fp]),
    "rlh_probe_gemv_phases": (C.c_int, [_vp, C.c_int, C.c_int, C.c_int, C.c_int, _fp]),
    "rlh_synth_normal_f16": (None, [C.c_uint64, C.c_int, C.c_int, C.c_uint64, C.c_uint64, C.c_double, C.POINTER(C.c_uint16)]),
    "rlh_synth_tokens": (None, [C.c_uint64, C.c_uint64, C.c_uint64, C.c_int32, C.c_int32, _i32p]),
    "rlh_abi_version": (C.c_int, []),
}

_lib = None


def load() -> C.CDLL:
    """Loads the in-tree library; raises if it has not been built (python -m rllama_amd.build)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FileNotFoundError(
            f"{LIB_PATH} is missing: build it with `python -m rllama_amd.build` (hipcc, gfx950). There is no CPU fallback."
        )
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here = header/library mismatch
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int) -> None:
    if rc != 0:
        msg = load().rlh_last_error()
        raise RllamaHipError(rc, msg.decode("utf-8", "replace") if msg else "")
