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
