"""CPU-side checks of the product library: it loads, exports exactly what include/rllama_hip.h declares,
fails cleanly without a device, and its synthetic-input generator is what the fixtures say."""
import hashlib
import json
import os
import re

import numpy as np
import pytest
import scipy.stats

import rllama_amd
from rllama_amd import _lib

HERE = os.path.dirname(os.path.abspath(__file__))


def _declared_symbols():
    text = open(_lib.HEADER_PATH).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rlh_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    declared = _declared_symbols()
    assert len(declared) >= 35
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in rllama_hip.h but not exported"
    assert sorted(_lib.SIGNATURES) == declared, "ctypes signature table and header disagree"
    assert lib.rlh_abi_version() == 1


def test_rust_ffi_crate_matches_the_header():
    """rust/rllama-hip-sys/src/lib.rs (the extern "C" seam a Rust host links against) is what the generator makes of the
    header today, and declares every function with the argument count of the ctypes table."""
    import importlib.util
    root = os.path.dirname(HERE)
    gen_path = os.path.join(root, "rust", "rllama-hip-sys", "gen_bindings.py")
    spec = importlib.util.spec_from_file_location("gen_bindings", gen_path)
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)
    lib_rs = open(os.path.join(root, "rust", "rllama-hip-sys", "src", "lib.rs")).read()
    assert lib_rs == gen.generate(), "run `python rust/rllama-hip-sys/gen_bindings.py` after changing include/rllama_hip.h"
    decls = dict((m.group(1), m.group(2)) for m in re.finditer(r"pub fn (rlh_[a-z0-9_]+)\((.*?)\)(?: -> [^;]+)?;", lib_rs))
    assert sorted(decls) == _declared_symbols()
    for name, (res, args) in _lib.SIGNATURES.items():
        n_rust = 0 if not decls[name].strip() else decls[name].count(":")
        assert n_rust == len(args), (name, decls[name])
    for const in ("RLH_OK", "RLH_ERR_UNSUPPORTED", "RLH_F16", "RLH_F32", "RLH_TOK_EMB", "RLH_OUTPUT"):
        assert f"pub const {const}: c_int" in lib_rs
    for field in [f[0] for f in _lib.ModelParams._fields_] + [f[0] for f in _lib.SamplerParams._fields_]:
        assert f"pub {field}:" in lib_rs
    # every entry point that the integration guide at the repository root shows must exist in the crate
    doc = open(os.path.join(root, "INTEGRATION.md")).read()
    for name in set(re.findall(r"\b(rlh_[a-z0-9_]+)\b", doc)):
        assert name in decls or name in ("rlh_model_params", "rlh_sampler_params", "rlh_ctx", "rlh_model", "rlh_caches", "rlh_tensor", "rlh_event",
                                         "rlh_tensor_kind", "rlh_status", "rlh_dtype"), f"the integration guide names {name}, which the header does not declare"


def _ctypes_of_rust(t: str):
    """The ctypes type a Rust FFI type corresponds to (what the C ABI passes for it)."""
    import ctypes as C
    scalars = {"c_int": C.c_int, "c_float": C.c_float, "c_double": C.c_double, "i32": C.c_int32, "u16": C.c_uint16, "u64": C.c_uint64, "usize": C.c_size_t,
               "f32": C.c_float, "f64": C.c_double}
    t = t.strip()
    if t in scalars:
        return scalars[t]
    m = re.match(r"^\*(const|mut) (.*)$", t)
    assert m, t
    inner = m.group(2).strip()
    if inner == "c_char":
        return C.c_char_p
    if inner == "c_void" or inner in ("rlh_ctx", "rlh_model", "rlh_caches", "rlh_tensor", "rlh_event"):
        return C.c_void_p                                   # opaque handles and untyped buffers
    if inner == "rlh_model_params":
        return C.POINTER(_lib.ModelParams)
    if inner == "rlh_sampler_params":
        return C.POINTER(_lib.SamplerParams)
    return C.POINTER(_ctypes_of_rust(inner))


def test_rust_ffi_types_match_the_ctypes_tables():
    """Neither cargo nor rustc exists where this suite runs, so the generated crate is never compiled here.  What can be
    checked without a compiler: every argument and return type of every function, and every field (type and order) of the two
    #[repr(C)] structs, denote the same C type as the ctypes tables that the whole GPU suite calls through; and the struct
    layouts ctypes computes are the C compiler's (sizes and offsets of include/rllama_hip.h compiled with gcc)."""
    import ctypes as C
    import subprocess
    import tempfile
    root = os.path.dirname(HERE)
    lib_rs = open(os.path.join(root, "rust", "rllama-hip-sys", "src", "lib.rs")).read()
    decls = {m.group(1): (m.group(2), m.group(3)) for m in re.finditer(r"pub fn (rlh_[a-z0-9_]+)\((.*?)\)(?: -> ([^;]+))?;", lib_rs)}
    assert sorted(decls) == sorted(_lib.SIGNATURES)
    same = lambda a, b: a is b or (C.sizeof(a) == C.sizeof(b) and a._type_ == b._type_ and not hasattr(a, "contents") and not hasattr(b, "contents"))  # c_int is c_int32 here
    for name, (res, args) in _lib.SIGNATURES.items():
        params, ret = decls[name]
        rust_args = [a.split(":", 1)[1] for a in params.split(",")] if params.strip() else []
        assert len(rust_args) == len(args), name
        for i, (ra, ca) in enumerate(zip(rust_args, args)):
            got = _ctypes_of_rust(ra)
            ok = got is ca or (hasattr(got, "_type_") and hasattr(ca, "_type_") and getattr(got, "_type_", None) == getattr(ca, "_type_", None)) or \
                (hasattr(got, "contents") and hasattr(ca, "contents") and C.sizeof(got._type_) == C.sizeof(ca._type_) and getattr(got._type_, "_type_", 0) == getattr(ca._type_, "_type_", 1))
            assert ok, f"{name} argument {i}: Rust `{ra.strip()}` is {got}, the ctypes table has {ca}"
        want_ret = None if ret is None else _ctypes_of_rust(ret)
        assert (want_ret is None and res is None) or want_ret is res or same(want_ret, res), (name, ret, res)
    for sname, table in (("rlh_model_params", _lib.ModelParams), ("rlh_sampler_params", _lib.SamplerParams)):
        body = re.search(r"pub struct %s \{(.*?)\}" % sname, lib_rs, flags=re.S).group(1)
        fields = [(m.group(1), m.group(2)) for m in re.finditer(r"pub ([a-z_0-9]+): ([^,]+),", body)]
        assert [f for f, _ in fields] == [f for f, _ in table._fields_], sname          # same fields in the same order
        for (fname, rtype), (_, ctype) in zip(fields, table._fields_):
            got = _ctypes_of_rust(rtype)
            assert got is ctype or same(got, ctype), (sname, fname, rtype, ctype)
    # ctypes' layout of the two structs against gcc's of the header itself
    prog = '''#include <stdio.h>
#include <stddef.h>
#include "rllama_hip.h"
int main(void) {
    printf("%zu %zu %zu %zu %zu\\n", sizeof(rlh_model_params), offsetof(rlh_model_params, norm_eps), offsetof(rlh_model_params, force_f16),
           offsetof(rlh_model_params, percentage_to_gpu), offsetof(rlh_model_params, max_seq_len));
    printf("%zu %zu %zu\\n", sizeof(rlh_sampler_params), offsetof(rlh_sampler_params, top_k), offsetof(rlh_sampler_params, repetition_penalty));
    return 0;
}
'''
    with tempfile.TemporaryDirectory() as d:
        src, exe = os.path.join(d, "layout.c"), os.path.join(d, "layout")
        open(src, "w").write(prog)
        subprocess.check_call(["gcc", "-I", os.path.join(root, "include"), src, "-o", exe])
        out = subprocess.check_output([exe], text=True).split()
    M, S = _lib.ModelParams, _lib.SamplerParams
    assert [int(v) for v in out] == [C.sizeof(M), M.norm_eps.offset, M.force_f16.offset, M.percentage_to_gpu.offset, M.max_seq_len.offset,
                                     C.sizeof(S), S.top_k.offset, S.repetition_penalty.offset]


def test_no_oracle_in_product():
    """The shipped package and library must not reach into oracle/ (test infrastructure)."""
    pkg = os.path.dirname(_lib.__file__)
    for root, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                src = open(os.path.join(root, f), errors="replace").read()
                assert "import oracle" not in src and "from oracle" not in src and "rllama_oracle" not in src, f


def _have_gpu():
    return os.path.exists("/dev/kfd")


@pytest.mark.skipif(_have_gpu(), reason="checks the no-device error path")
def test_init_without_device_fails_loudly():
    with pytest.raises(rllama_amd.RllamaHipError) as ei:
        rllama_amd.Context(0)
    assert ei.value.code in (2, 3)          # RLH_ERR_NO_DEVICE (or a HIP runtime error string)
    assert "device" in str(ei.value).lower() or "hip" in str(ei.value).lower()


def test_synth_normal_statistics():
    bits = rllama_amd.synth_normal_f16(0, rllama_amd.W1, 3, 400_000, std=0.02)
    v = bits.view(np.float16).astype(np.float64)
    assert abs(v.mean()) < 2e-4
    assert abs(v.std() - 0.02) < 2e-4
    # normality of the underlying deviates (f16 rounding is far below the KS resolution at this n)
    ks = scipy.stats.kstest(v / 0.02, "norm")
    assert ks.pvalue > 1e-3, ks
    # element idx is a pure function of (seed, kind, layer, idx): windows agree with the whole
    win = rllama_amd.synth_normal_f16(0, rllama_amd.W1, 3, 1000, first_index=12345, std=0.02)
    assert np.array_equal(win, bits[12345:13345])
    # streams differ by seed, kind and layer
    for other in (rllama_amd.synth_normal_f16(1, rllama_amd.W1, 3, 1000), rllama_amd.synth_normal_f16(0, rllama_amd.W3, 3, 1000),
                  rllama_amd.synth_normal_f16(0, rllama_amd.W1, 4, 1000)):
        assert not np.array_equal(other, bits[:1000])
    # independence of the two outputs of one polar pair and of neighbouring pairs
    assert abs(np.corrcoef(v[0::2], v[1::2])[0, 1]) < 0.01
    assert abs(np.corrcoef(v[:-2:2], v[2::2])[0, 1]) < 0.01


def test_synth_tokens_range_and_uniformity():
    t = rllama_amd.synth_tokens(0, 200_000, 3, 32000)
    assert t.min() >= 3 and t.max() < 32000
    counts = np.bincount((t - 3) * 50 // (32000 - 3), minlength=50)
    assert scipy.stats.chisquare(counts).pvalue > 1e-3


def test_synth_golden_fixture():
    """The generator's output is frozen: the parity configs are defined by (seed, shape) alone."""
    fx = json.load(open(os.path.join(HERE, "golden", "synth_fixture.json")))
    for case in fx["normal_f16"]:
        bits = rllama_amd.synth_normal_f16(case["seed"], case["kind"], case["layer"], case["count"], first_index=case["first_index"], std=case["std"])
        assert bits[:8].tolist() == case["first8_bits"]
        assert hashlib.sha256(bits.tobytes()).hexdigest() == case["sha256"]
    for case in fx["tokens"]:
        t = rllama_amd.synth_tokens(case["seed"], case["count"], case["lo"], case["hi"])
        assert t.tolist() == case["ids"]
