"""Pins the CPU oracle (oracle/rllama_oracle.c) without running the reference.

The reference (Noeda/rllama) ships no golden vectors and no seeded fixtures: its tests (src/tensor.rs:2548-3209)
are properties with tolerances.  Each oracle function is therefore pinned here by (a) those properties at the
reference's own tolerances, (b) closed forms / library routines in float64, and (c) hand-built cases in which
a plausible mistake (wrong lane order, missing FMA, wrong rounding mode, transposed operand, dropped term)
changes the answer.
"""
import math

import numpy as np
import pytest
import scipy.special

import oracle
from rllama_amd import TOK_EMB
from common import (SMALL, TINY, RefF64, make_oracle, max_rel_err, random_f32_weights, synth_weights)

f32 = np.float32


# ------------------------------------------------------------------------------------------------------
# f16 <-> f32  (simd_support.rs:45-52; tensor.rs:2226-2314; property tensor.rs:2881-2920)
# ------------------------------------------------------------------------------------------------------
def test_f16_to_f32_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = oracle.f16_bits_to_f32(bits)                      # F16C vector path
    got_sw = np.array([oracle.lib().orc_f16_bits_to_f32(int(b)) for b in bits], dtype=np.float32)
    for g in (got, got_sw):
        assert np.array_equal(g.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
        assert np.all(np.isnan(g[np.isnan(want)]))


def _f32_probe_values():
    """All f16 values, the midpoints between neighbours (ties), their f32 neighbours, and random bit patterns."""
    h = np.arange(0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)  # non-negative finite halves
    mids = (h[:-1] + h[1:]) / 2
    vals = [h, mids, np.nextafter(mids.astype(f32), f32(np.inf)).astype(np.float64),
            np.nextafter(mids.astype(f32), f32(-np.inf)).astype(np.float64),
            np.array([65504.0, 65519.99, 65520.0, 65536.0, 1e30, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0000001, 2.0 ** -26, 0.0])]
    v = np.concatenate(vals).astype(f32)
    v = np.concatenate([v, -v, np.array([np.inf, -np.inf], f32)])
    rng = np.random.default_rng(1)
    rnd = rng.integers(0, 2 ** 32, size=1_000_000, dtype=np.uint64).astype(np.uint32).view(f32)
    rnd = rnd[~np.isnan(rnd)]
    return np.concatenate([v, rnd])


def test_f32_to_f16_round_to_nearest_even():
    v = _f32_probe_values()
    with np.errstate(over="ignore"):
        want = v.astype(np.float16).view(np.uint16)          # numpy: IEEE RNE
    got_hw = oracle.f32_to_f16_bits(v)                       # _mm256_cvtps_ph(a, 0)
    assert np.array_equal(got_hw, want)
    sub = v[:: max(1, v.size // 200_000)]
    got_sw = np.array([oracle.lib().orc_f32_to_f16_bits(float(x)) for x in sub], dtype=np.uint16)
    with np.errstate(over="ignore"):
        assert np.array_equal(got_sw, sub.astype(np.float16).view(np.uint16))
    # a tie must go to even, not away from zero and not truncate: 1 + 2^-11 is halfway between 1 and 1 + 2^-10
    assert oracle.lib().orc_f32_to_f16_hw(1.0 + 2.0 ** -11) == 0x3C00
    assert oracle.lib().orc_f32_to_f16_hw(1.0 + 3 * 2.0 ** -11) == 0x3C02


def test_f16_round_trip_is_identity():
    bits = np.arange(65536, dtype=np.uint16)
    finite = ~np.isnan(bits.view(np.float16))
    assert np.array_equal(oracle.f32_to_f16_bits(oracle.f16_bits_to_f32(bits))[finite], bits[finite])


# ------------------------------------------------------------------------------------------------------
# hsum8 / dot8  (simd_support.rs:90-116; tensor.rs:1351-1447, 1577-1638, 1870-1902, 1957-1979)
# ------------------------------------------------------------------------------------------------------
def _hsum_ref(a):
    a = [f32(x) for x in a]
    return f32(f32(f32(a[0] + a[4]) + f32(a[1] + a[5])) + f32(f32(a[2] + a[6]) + f32(a[3] + a[7])))


def test_hsum8_association_order():
    # chosen so that sequential, adjacent-pairwise, (0+4),(2+6)-first and the reference's order all differ
    a = np.array([5.0, -2.0 ** 24, -1.0, 2.0 ** 25, -2.0 ** 25, -1.0, 3.0, 1.0], dtype=f32)
    got = oracle.lib().orc_hsum8(a.ctypes.data_as(oracle.C.POINTER(oracle.C.c_float)))
    want = _hsum_ref(a)
    seq = f32(0)
    for x in a:
        seq = f32(seq + x)
    adj = f32(f32(f32(a[0] + a[1]) + f32(a[2] + a[3])) + f32(f32(a[4] + a[5]) + f32(a[6] + a[7])))
    alt = f32(f32(f32(a[0] + a[4]) + f32(a[2] + a[6])) + f32(f32(a[1] + a[5]) + f32(a[3] + a[7])))
    assert got == want == f32(-16777212.0)
    assert len({float(want), float(seq), float(adj), float(alt)}) == 4, "test vector does not discriminate the association order"


def _dot8_ref_exact_products(a, b):
    """dot8 when every product is exactly representable (so FMA == multiply-then-add)."""
    acc = [f32(0)] * 8
    for p in range(0, len(a), 8):
        for l in range(8):
            if p + l < len(a):
                acc[l] = f32(acc[l] + f32(a[p + l]) * f32(b[p + l]))
    return _hsum_ref(acc)


def test_dot8_lane_order_discriminates():
    big = 2.0 ** 24
    # products: lane l accumulates k = l, l+8, l+16.  Absorption (2^24 + 1 == 2^24 in f32) makes the result
    # depend on which elements share a lane and on the hsum order.
    prods = np.array([big, 1, 1, 1, -big, 1, 1, 1,
                      1, 1, big, 1, 1, 1, -big, 1,
                      1, 1, 1, 1, 1, 1, 1, 1, 1], dtype=f32)  # K = 25: also exercises the zero-padded tail
    a = prods.copy()
    b = np.ones_like(a)
    want = _dot8_ref_exact_products(a, b)
    assert oracle.dot8_f32(a, b) == want
    assert oracle.dot8_f32_scalar(a, b) == want
    seq = f32(0)
    for x in prods:
        seq = f32(seq + x)
    # a 4-lane or 16-lane accumulator layout gives something else on this vector
    def lanes(nl):
        acc = [f32(0)] * nl
        for i, x in enumerate(prods):
            acc[i % nl] = f32(acc[i % nl] + x)
        s = f32(0)
        for x in acc:
            s = f32(s + x)
        return s
    assert want != seq and want != lanes(4) and want != lanes(16)


def test_dot8_uses_fused_multiply_add():
    a = np.array([1 + 2.0 ** -12, 1.0], dtype=f32)
    b = np.array([1 + 2.0 ** -12, -(1 + 2.0 ** -11)], dtype=f32)
    # lanes 0 and 1, one term each: fma keeps 2^-24 of the first product; a rounded product would lose it
    got = oracle.dot8_f32(a, b)
    # lane0 = fma(a0,b0,0) = round(1 + 2^-11 + 2^-24) = 1 + 2^-11 (tie to even); lane1 = -(1 + 2^-11): sum is 0 here,
    # so put both on the same lane (k = 0 and k = 8) to make the FMA visible:
    a2 = np.zeros(9, f32)
    b2 = np.zeros(9, f32)
    a2[0], b2[0] = -(1 + 2.0 ** -11), 1.0
    a2[8], b2[8] = 1 + 2.0 ** -12, 1 + 2.0 ** -12
    assert oracle.dot8_f32(a2, b2) == f32(2.0 ** -24)
    assert oracle.dot8_f32_scalar(a2, b2) == f32(2.0 ** -24)
    assert got == f32(0.0)


def test_dot8_intrinsics_equal_scalar_fmaf_and_f16_path():
    rng = np.random.default_rng(2)
    for k in (1, 7, 8, 9, 64, 100, 128, 1000, 4096):
        a = rng.uniform(-1, 1, k).astype(f32)
        b = rng.uniform(-1, 1, k).astype(f32)
        assert oracle.dot8_f32(a, b) == oracle.dot8_f32_scalar(a, b)
        ah, bh = oracle.f32_to_f16_bits(a), oracle.f32_to_f16_bits(b)
        assert oracle.dot8_f16(ah, bh) == oracle.dot8_f32(oracle.f16_bits_to_f32(ah), oracle.f16_bits_to_f32(bh))
        exact = float(np.dot(a.astype(np.float64), b.astype(np.float64)))
        assert abs(oracle.dot8_f32(a, b) - exact) <= 1e-5 * max(1.0, abs(exact))


# ------------------------------------------------------------------------------------------------------
# matmul family: the reference's own properties and tolerances (tensor.rs:2554-2856), plus exact structure
# ------------------------------------------------------------------------------------------------------
def test_matmul_transposed_f32_vs_naive_and_structure():
    rng = np.random.default_rng(3)
    for _ in range(40):
        n, m, k = (int(v) for v in rng.integers(1, 129, 3))
        x = rng.uniform(-1, 1, (n, k)).astype(f32)
        w = rng.uniform(-1, 1, (m, k)).astype(f32)
        got = oracle.matmul_transposed_f32(x, w)
        want = x.astype(np.float64) @ w.astype(np.float64).T     # naive, not transposed-operand
        assert np.allclose(got, want, rtol=1e-5, atol=1e-5)      # tensor.rs:2725-2747 (1e-5)
        r, c = int(rng.integers(0, n)), int(rng.integers(0, m))
        assert got[r, c] == f32(oracle.dot8_f32(x[r], w[c]))     # every element is exactly dot8
    # non-square, asymmetric case catches an accidentally transposed operand or output
    x = np.arange(6, dtype=f32).reshape(2, 3)
    w = np.array([[1, 0, 0], [0, 1, 0], [0, 0, 1], [1, 1, 1]], dtype=f32)
    assert np.array_equal(oracle.matmul_transposed_f32(x, w), np.array([[0, 1, 2, 3], [3, 4, 5, 12]], dtype=f32))


def test_matmul_transposed_f16_vs_f32_and_rounding():
    rng = np.random.default_rng(4)
    for _ in range(30):
        n, m, k = (int(v) for v in rng.integers(1, 129, 3))
        x = rng.uniform(-1, 1, (n, k)).astype(f32)
        w = rng.uniform(-1, 1, (m, k)).astype(f32)
        xh, wh = oracle.f32_to_f16_bits(x), oracle.f32_to_f16_bits(w)
        got_bits = oracle.matmul_transposed_f16(xh, wh)
        got = oracle.f16_bits_to_f32(got_bits)
        f32res = oracle.matmul_transposed_f32(x, w)
        assert np.allclose(got, f32res, rtol=1e-1, atol=1e-1)    # tensor.rs:2581-2609 (1e-1)
        # exact structure: f16(dot8 of the f16-rounded operands)
        want64 = oracle.f16_bits_to_f32(xh).astype(np.float64) @ oracle.f16_bits_to_f32(wh).astype(np.float64).T
        assert np.allclose(got, want64, rtol=2e-3, atol=2e-3)
        r, c = int(rng.integers(0, n)), int(rng.integers(0, m))
        assert got_bits[r, c] == oracle.f32_to_f16_bits(np.array([oracle.dot8_f16(xh[r], wh[c])], f32))[0]


def test_matmul_seqk_chain_and_vector_matrix_mul():
    rng = np.random.default_rng(5)
    for _ in range(20):
        m, n, k = (int(v) for v in rng.integers(1, 65, 3))
        a = rng.uniform(-1, 1, (m, k)).astype(f32)
        b = rng.uniform(-1, 1, (k, n)).astype(f32)
        got = oracle.matmul_f32_seqk(a, b)
        assert np.allclose(got, a.astype(np.float64) @ b.astype(np.float64), rtol=1e-5, atol=1e-5)  # tensor.rs:2749-2786
        v = oracle.vector_matrix_mul_f32(a[0], b)
        assert np.allclose(v, a[0].astype(np.float64) @ b.astype(np.float64), rtol=1e-5, atol=1e-5)  # tensor.rs:2803-2824
        c = int(rng.integers(0, n))
        assert v[c] == f32(oracle.dot8_f32(a[0], np.ascontiguousarray(b[:, c])))   # gather form == dot8 of the column
    # sequential-k chain with absorption: (2^24 + 1) + 1 ... stays 2^24 sequentially, but pairs would give 2^24 + 2
    a = np.array([[2.0 ** 24, 1, 1]], dtype=f32)
    b = np.ones((3, 1), dtype=f32)
    assert oracle.matmul_f32_seqk(a, b)[0, 0] == f32(2.0 ** 24)


# ------------------------------------------------------------------------------------------------------
# element-wise pieces: closed forms
# ------------------------------------------------------------------------------------------------------
def test_rmsnorm_closed_form():
    rng = np.random.default_rng(6)
    for d in (8, 64, 1000, 4096):
        x = rng.standard_normal(d).astype(f32) * 3
        w = rng.uniform(0.5, 1.5, d).astype(f32)
        eps = 1e-6
        got = oracle.rmsnorm_row(x, w, eps)
        x64 = x.astype(np.float64)
        want = x64 / np.sqrt(np.mean(x64 ** 2) + eps) * w
        assert np.allclose(got, want, rtol=2e-6, atol=1e-7)
    # constant row: c / sqrt(c^2 + eps) * w ; eps matters for small c (a dropped eps gives exactly +-1)
    c = 1e-3
    got = oracle.rmsnorm_row(np.full(16, c, f32), np.full(16, 2.0, f32), 1e-6)
    assert np.allclose(got, 2.0 * c / math.sqrt(c * c + 1e-6), rtol=1e-6)
    assert abs(got[0] - 2.0) > 0.1


def test_softmax_closed_form_and_no_max_subtraction():
    rng = np.random.default_rng(7)
    s = rng.uniform(-5, 5, 37).astype(f32)
    got = oracle.softmax_row(s)
    assert np.allclose(got, scipy.special.softmax(s.astype(np.float64)), rtol=1e-5)
    assert np.array_equal(oracle.softmax_row(np.zeros(16, f32)), np.full(16, 1 / 16, f32))
    assert np.allclose(oracle.softmax_row(np.full(13, 0.7, f32)), 1 / 13, rtol=1e-6)
    # tensor.rs:479-494 does not subtract the maximum: exp overflows to inf and inf/inf = NaN
    with np.errstate(all="ignore"):
        assert np.isnan(oracle.softmax_row(np.array([100.0, 0.0], f32))[0])
    # masked entries: exp(-inf) = 0
    assert oracle.softmax_row(np.array([0.0, -np.inf], f32)).tolist() == [1.0, 0.0]


def test_silu_closed_form():
    for v in (-10.0, -1.0, -0.1, 0.0, 0.1, 1.0, 3.5, 10.0):
        assert math.isclose(oracle.silu(v), v / (1 + math.exp(-v)), rel_tol=1e-6, abs_tol=1e-9)
    assert oracle.silu(0.0) == 0.0


def test_freqs_cis_and_rope_against_complex_rotation():
    hd, T = 64, 50
    fc = oracle.freqs_cis(hd, T)
    pos = np.arange(T)[:, None]
    ang = pos * (10000.0 ** (-np.arange(0, hd, 2) / hd))[None, :]
    assert np.allclose(fc[..., 0], np.cos(ang), atol=1e-12) and np.allclose(fc[..., 1], np.sin(ang), atol=1e-12)
    assert np.array_equal(fc[0, :, 0], np.ones(hd // 2)) and np.array_equal(fc[0, :, 1], np.zeros(hd // 2))
    rng = np.random.default_rng(8)
    H = 3
    x = rng.standard_normal((H, hd)).astype(f32)
    assert np.array_equal(oracle.rope_row(x, H, hd, fc[0]).reshape(H, hd), x)          # position 0 is the identity
    p = 17
    got = oracle.rope_row(x, H, hd, fc[p]).reshape(H, hd)
    xc = (x[:, 0::2].astype(np.float64) + 1j * x[:, 1::2].astype(np.float64)) * np.exp(1j * ang[p])[None, :]
    want = np.stack([xc.real, xc.imag], axis=-1).reshape(H, hd)                          # interleaved pairs
    assert np.allclose(got, want, rtol=1e-6, atol=1e-6)
    assert np.allclose(np.linalg.norm(got, axis=1), np.linalg.norm(x, axis=1), rtol=1e-6)  # rotations preserve norms
    # the half-split ("rotate_half") layout would pair (j, j + hd/2) instead: make sure that is not what we have
    xh = (x[:, : hd // 2].astype(np.float64) + 1j * x[:, hd // 2:].astype(np.float64)) * np.exp(1j * ang[p])[None, :]
    assert not np.allclose(got, np.concatenate([xh.real, xh.imag], axis=1), atol=1e-3)


def _sample_greedy_bruteforce(logits, temperature=1.0):
    """token_sampler.rs:83-174 at top_k = 1, restated independently with Python floats rounded through numpy f32."""
    l = [f32(v) for v in logits]
    if temperature > 0:
        inv = f32(1.0) / f32(temperature)
        l = [f32(v * inv) for v in l]
    maxv = f32(-np.inf)
    if l[0] > maxv:
        maxv = l[0]
    with np.errstate(invalid="ignore"):
        l[0] = f32(l[0] - maxv)
    with np.errstate(over="ignore", invalid="ignore"):
        e = np.exp(np.array(l, dtype=f32)).astype(f32)
        tot = f32(0)
        for v in e:
            tot = f32(tot + v)
        p = (e / tot).astype(f32)
    order = sorted(range(len(p)), key=lambda i: (math.isnan(p[i]), -p[i] if not math.isnan(p[i]) else 0, i))
    return order[0]


def test_greedy_sampler_bruteforce_and_token0_quirk():
    rng = np.random.default_rng(9)
    for _ in range(200):
        V = int(rng.integers(2, 40))
        logits = (rng.standard_normal(V) * 3).astype(f32)
        tok, prob, ties = oracle.sample_greedy(logits)
        assert tok == _sample_greedy_bruteforce(logits)
    # token 0's logit is replaced by 0.0: a hugely negative logit 0 still wins against all-negative others ...
    assert oracle.sample_greedy(np.array([-50.0, -1.0, -2.0], f32))[0] == 0
    # ... and a hugely positive logit 0 loses against any positive other
    assert oracle.sample_greedy(np.array([50.0, 1.0, 0.5], f32))[0] == 1
    # nothing else is shifted: plain argmax over the rest
    assert oracle.sample_greedy(np.array([0.0, 1.0, 7.0, 3.0], f32))[0] == 2
    # ties are reported and resolve to the lowest id
    tok, _, ties = oracle.sample_greedy(np.array([-9.0, 2.0, 2.0], f32))
    assert (tok, ties) == (1, 2)


# ------------------------------------------------------------------------------------------------------
# whole forward
# ------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("shape", [TINY, SMALL], ids=["tiny", "small"])
def test_forward_f32_mode_matches_independent_float64(shape):
    W = random_f32_weights(shape, seed=11, std=0.08)
    m = make_oracle(shape, W, force_f16=False)
    ref = RefF64(shape, W, f16_points=False)
    rng = np.random.default_rng(12)
    toks = rng.integers(0, shape.vocab_size, 9)
    c = m.make_caches()
    got = m.forward(toks[:6], 0, c)
    want = ref.forward(toks[:6], 0)
    assert max_rel_err(got, want) < 2e-5
    for i in range(6, 9):                                     # decode steps reuse the cache
        got = m.forward(toks[i:i + 1], i, c)
        want = ref.forward(toks[i:i + 1], i)
        assert max_rel_err(got, want) < 2e-5
    # cache contents: K is post-RoPE, position along columns (transformer.rs:143-154, 754-761)
    for l in range(shape.n_layers):
        for h in range(shape.n_heads):
            assert np.allclose(c.read(l, h, 0)[:, :9], ref.k[l, h, :9].T, rtol=1e-4, atol=1e-5)
            assert np.allclose(c.read(l, h, 1)[:, :9], ref.v[l, h, :9].T, rtol=1e-4, atol=1e-5)
            assert not np.any(c.read(l, h, 0)[:, 9:])         # untouched positions stay zero


@pytest.mark.parametrize("shape", [TINY, SMALL], ids=["tiny", "small"])
def test_forward_f16_mode_matches_float64_with_the_same_rounding_points(shape):
    W = synth_weights(shape, seed=3, std=0.08, norm_ones=False)
    m = make_oracle(shape, W, force_f16=True)
    ref = RefF64(shape, W, f16_points=True)
    rng = np.random.default_rng(13)
    toks = rng.integers(0, shape.vocab_size, 8)
    c = m.make_caches()
    got = m.forward(toks[:5], 0, c)
    want = ref.forward(toks[:5], 0)
    assert max_rel_err(got, want) < 1e-2                      # rounding flips at f16 points, nothing structural
    # without the rounding points the float64 model must be visibly further away than with them
    far = RefF64(shape, W, f16_points=False).forward(toks[:5], 0)
    assert max_rel_err(got, want) < max_rel_err(got, far) or max_rel_err(got, far) < 1e-3
    for i in range(5, 8):
        assert max_rel_err(m.forward(toks[i:i + 1], i, c), ref.forward(toks[i:i + 1], i)) < 1e-2
    # K and V are rounded to f16 on the cache write
    k0 = c.read(0, 0, 0)[:, :8]
    assert np.array_equal(k0, k0.astype(np.float16).astype(np.float32))


@pytest.mark.parametrize("force_f16", [False, True], ids=["f32", "f16"])
def test_forward_invariants(force_f16):
    shape = TINY
    W = synth_weights(shape, seed=5, std=0.1, norm_ones=False)
    m = make_oracle(shape, W, force_f16)
    toks = np.array([5, 17, 3, 90, 41, 8], dtype=np.int32)
    # prefill(n) == prefill(n-1) + decode(1) up to the score kernel's summation order (seq-k chain vs dot8)
    c1 = m.make_caches()
    a = m.forward(toks, 0, c1)
    c2 = m.make_caches()
    m.forward(toks[:-1], 0, c2)
    b = m.forward(toks[-1:], len(toks) - 1, c2)
    assert max_rel_err(a, b) < (5e-3 if force_f16 else 1e-5)
    # true_clone: independent copies, identical continuation; the original is not disturbed by the clone's step
    c3 = c2.true_clone()
    x = m.forward([7], len(toks), c2)
    y = m.forward([7], len(toks), c3)
    assert np.array_equal(x, y)
    z = m.forward([9], len(toks), c3)
    assert not np.array_equal(y, z)
    assert np.array_equal(m.forward([7], len(toks), c2), x)   # deterministic, thread-count independent
    oracle.set_threads(1)
    try:
        assert np.array_equal(m.forward([7], len(toks), c2), x)
    finally:
        oracle.set_threads(0)
    # calls the reference would panic on
    with pytest.raises(RuntimeError):
        m.forward([1, 2], 3, c2)
    with pytest.raises(RuntimeError):
        m.forward([1], shape.max_seq_len, c2)


def test_forward_with_zeroed_wo_and_w2_is_head_of_normed_embedding():
    from rllama_amd import NORM, OUTPUT, TOK_EMB, W2, WO
    shape = TINY
    W = synth_weights(shape, seed=6, std=0.1, norm_ones=False)
    for l in range(shape.n_layers):
        W[(WO, l)] = np.zeros_like(W[(WO, l)])
        W[(W2, l)] = np.zeros_like(W[(W2, l)])
    m = make_oracle(shape, W, force_f16=True)
    tok = 33
    got = m.forward([tok], 0, m.make_caches())
    e = W[(TOK_EMB, 0)][tok].view(np.float16).astype(np.float64)
    xn = e / np.sqrt(np.mean(e * e) + shape.norm_eps) * W[(NORM, 0)][0]
    want = W[(OUTPUT, 0)].view(np.float16).astype(np.float64) @ xn
    assert max_rel_err(got, want) < 1e-5


@pytest.mark.parametrize("force_f16", [False, True], ids=["f32", "f16"])
def test_forward_cut_at_the_layer_split_is_the_same_forward(force_f16):
    """embed -> forward_layers(0..k) -> forward_layers(k+1..L-1) -> head is forward bit for bit, for a prompt call and a
    single-token call, at every cut k (the pieces a layer split hands between devices, transformer.rs:262-279, 361-381)."""
    shape = SMALL
    W = synth_weights(shape, seed=5, std=0.05, norm_ones=False)
    m = make_oracle(shape, W, force_f16)
    toks = [int(t) for t in np.random.default_rng(3).integers(3, shape.vocab_size, 6)]
    c0 = m.make_caches()
    want_prompt, tap = m.forward(toks, 0, c0, layer_tap=True)
    want_next = m.forward([7], len(toks), c0)
    emb = W[(TOK_EMB, 0)].view(np.float16).astype(np.float32)
    assert np.array_equal(m.embed(toks), emb[toks])
    for k in range(shape.n_layers):
        c = m.make_caches()
        x = m.forward_layers(m.embed(toks), 0, c, 0, k)
        assert np.array_equal(x, tap[k]), k
        if k + 1 < shape.n_layers:
            x = m.forward_layers(x, 0, c, k + 1, shape.n_layers - 1)
        assert np.array_equal(m.head(x), want_prompt), k
        y = m.forward_layers(m.embed([7]), len(toks), c, 0, k)
        if k + 1 < shape.n_layers:
            y = m.forward_layers(y, len(toks), c, k + 1, shape.n_layers - 1)
        assert np.array_equal(m.head(y), want_next), k
        for l in range(shape.n_layers):
            assert np.array_equal(c.read(l, 1, 0), c0.read(l, 1, 0)) and np.array_equal(c.read(l, 2, 1), c0.read(l, 2, 1))


def test_cache_shift_left():
    shape = TINY
    W = synth_weights(shape, seed=7, std=0.1)
    m = make_oracle(shape, W, force_f16=True)
    c = m.make_caches()
    m.forward([1, 2, 3, 4, 5], 0, c)
    before = c.read(1, 1, 0).copy()
    c.shift_left(2)
    after = c.read(1, 1, 0)
    T = shape.max_seq_len
    assert np.array_equal(after[:, : T - 2], before[:, 2:])
    assert np.array_equal(after[:, T - 2:], np.repeat(before[:, T - 1:], 2, axis=1))   # last column keeps its value


# ---- committed fixtures (tests/golden/make_oracle_fixtures.py): the oracle must keep reproducing them -----------------

def _bits_to_f32(bits):
    return np.array(bits, dtype=np.uint32).view(np.float32)


def test_golden_config0_reproduced():
    import hashlib
    import json
    import os
    import rllama_amd
    from common import CONFIG0, make_oracle, synth_weights
    fx = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "config0_oracle.json")))
    W = synth_weights(CONFIG0, seed=fx["seed"], std=fx["std"])
    names = {rllama_amd.TOK_EMB: "tok_embeddings", rllama_amd.OUTPUT: "output", rllama_amd.WQ: "wq", rllama_amd.WK: "wk", rllama_amd.WV: "wv",
             rllama_amd.WO: "wo", rllama_amd.W1: "w1", rllama_amd.W2: "w2", rllama_amd.W3: "w3"}
    for (k, l), a in W.items():
        if k in names:
            assert hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest() == fx["weight_sha256"][f"{names[k]}.{l}"], (k, l)
    prompt = rllama_amd.synth_tokens(0, 16, 3, 32000)
    assert prompt.tolist() == fx["prompt_ids"]
    om = make_oracle(CONFIG0, W, True)
    oc = om.make_caches()
    toks, prev = list(fx["prompt_ids"]), 0
    for step in range(64):
        logits = om.forward(toks[prev:], prev, oc)
        tok, _, _ = oracle.sample_greedy(logits)
        want = _bits_to_f32(fx["sample_logits_f32_bits"][step])
        got = logits[fx["sample_token_ids"]]
        assert np.allclose(got, want, rtol=1e-6, atol=1e-7), step
        assert tok == fx["greedy_ids"][step], step
        toks.append(tok)
        prev = len(toks) - 1
    assert min(fx["top2_logit_gap"]) > 1e-4  # the greedy choice is nowhere near a tie, so f16-level noise cannot flip it


def test_golden_tiny_reproduced():
    import json
    import os
    from common import TINY, make_oracle, random_f32_weights, synth_weights
    fx = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tiny_oracle.json")))
    for mode, W, f16 in (("f16", synth_weights(TINY, seed=21, std=0.08, norm_ones=False), True), ("f32", random_f32_weights(TINY, seed=23, std=0.08), False)):
        om = make_oracle(TINY, W, f16)
        oc = om.make_caches()
        toks = fx[mode]["tokens"]
        assert np.allclose(om.forward(toks[:7], 0, oc), _bits_to_f32(fx[mode]["logits_after_7_f32_bits"]), rtol=1e-6, atol=1e-7)
        assert np.allclose(om.forward(toks[7:8], 7, oc), _bits_to_f32(fx[mode]["logits_after_8_f32_bits"]), rtol=1e-6, atol=1e-7)


# ---------------------------------------------------------------------------------------------------------
# The exact-sum probe (oracle.set_exact_sums): what the reference's arithmetic gives when no fp32 addition inside a sum
# rounds.  It is the yardstick of the full-depth GPU tests, so it is pinned here like the oracle proper.
# ---------------------------------------------------------------------------------------------------------
@pytest.fixture
def exact_sums():
    oracle.set_exact_sums(True)
    try:
        yield
    finally:
        oracle.set_exact_sums(False)


def test_exact_sums_are_the_correctly_rounded_sums(exact_sums):
    """Dot products against math.fsum of the exact products (products of two f32 are exact in float64), rounded to f32 once:
    a dropped term, a product rounded to f32 first, or an fp32 accumulator each fail on these vectors."""
    import math
    rng = np.random.default_rng(41)
    for k in (1, 7, 8, 9, 64, 333, 4096, 11008):
        a = (rng.standard_normal(k) * 3).astype(np.float32)
        b = rng.standard_normal(k).astype(np.float32)
        want = np.float32(math.fsum(float(x) * float(y) for x, y in zip(a, b)))
        assert np.float32(oracle.dot8_f32(a, b)) == want, k
        ah, bh = a.astype(np.float16), b.astype(np.float16)
        want_h = np.float32(math.fsum(float(x) * float(y) for x, y in zip(ah, bh)))
        assert np.float32(oracle.dot8_f16(ah.view(np.uint16), bh.view(np.uint16))) == want_h, k
    # a sum where every fp32 accumulation order loses the small terms and float64 keeps them
    a = np.array([1.0] + [2.0 ** -25] * 64, np.float32)
    b = np.ones(65, np.float32)
    assert oracle.dot8_f32(a, b) == float(np.float32(1.0 + 64 * 2.0 ** -25))
    oracle.set_exact_sums(False)
    assert oracle.dot8_f32(a, b) != float(np.float32(1.0 + 64 * 2.0 ** -25))
    oracle.set_exact_sums(True)
    # the matrix forms go through the same sums
    x = rng.standard_normal((3, 100)).astype(np.float32)
    w = rng.standard_normal((5, 100)).astype(np.float32)
    want = np.array([[np.float32(math.fsum(float(p) * float(q) for p, q in zip(xr, wr))) for wr in w] for xr in x], np.float32)
    assert np.array_equal(oracle.matmul_transposed_f32(x, w), want)
    xh, wh = x.astype(np.float16), w.astype(np.float16)
    want_h = np.array([[np.float32(math.fsum(float(p) * float(q) for p, q in zip(xr, wr))) for wr in wh] for xr in xh], np.float32)
    got_h = oracle.matmul_transposed_f16(xh.view(np.uint16), wh.view(np.uint16)).view(np.float16)
    assert np.array_equal(got_h, want_h.astype(np.float16))           # f32 first, then f16: the reference's two roundings
    kq = rng.standard_normal(24).astype(np.float32)
    km = rng.standard_normal((24, 13)).astype(np.float32)
    want_v = np.array([np.float32(math.fsum(float(kq[r]) * float(km[r, c]) for r in range(24))) for c in range(13)], np.float32)
    assert np.array_equal(oracle.vector_matrix_mul_f32(kq, km), want_v)
    assert np.array_equal(oracle.matmul_f32_seqk(kq.reshape(1, -1), km)[0], want_v)


def test_exact_sums_leave_everything_but_the_sums_alone(exact_sums):
    """RMSNorm and softmax keep the reference's f32 element-wise steps and libm calls; only the sum changes."""
    import math
    rng = np.random.default_rng(42)
    x = (rng.standard_normal(1000) * 2).astype(np.float32)
    w = rng.uniform(0.5, 1.5, 1000).astype(np.float32)
    ss = np.float32(math.fsum(float(v) * float(v) for v in x))
    rs = np.float32(1.0) / np.sqrt(np.float32(ss / np.float32(1000) + np.float32(1e-6)))
    want = (x * rs) * w                                               # two f32 roundings per element (tensor.rs:631, 672)
    assert np.array_equal(oracle.rmsnorm_row(x, w, 1e-6), want)
    s = rng.standard_normal(300).astype(np.float32)
    oracle.set_exact_sums(False)
    plain = oracle.softmax_row(s)
    oracle.set_exact_sums(True)
    got = oracle.softmax_row(s)
    # every ratio got / plain is one constant (the two denominators), to within the rounding of the divisions
    ratio = got.astype(np.float64) / plain.astype(np.float64)
    assert np.ptp(ratio) < 3e-7
    assert abs(float(np.sum(got.astype(np.float64))) - 1.0) < 2e-7    # the float64 denominator normalises better than 300 fp32 adds would need to


@pytest.mark.parametrize("shape", [TINY, SMALL], ids=["tiny", "small"])
def test_exact_sum_forward_sits_between_the_oracle_and_float64(shape, exact_sums):
    """Whole forward, f16 mode: with exact sums the restatement must land (much) closer to the independent float64 model with
    the same rounding points than the reference's own fp32 lane order does; f32 mode: closer still."""
    W = synth_weights(shape, seed=3, std=0.08, norm_ones=False)
    rng = np.random.default_rng(13)
    toks = rng.integers(0, shape.vocab_size, 8)
    for force_f16 in (False, True):
        m = make_oracle(shape, W, force_f16)
        ref = RefF64(shape, W, f16_points=force_f16, via_f32=True)
        c = m.make_caches()
        got = [m.forward(toks[:5], 0, c)] + [m.forward(toks[i:i + 1], i, c) for i in range(5, 8)]
        want = [ref.forward(toks[:5], 0)] + [ref.forward(toks[i:i + 1], i) for i in range(5, 8)]
        oracle.set_exact_sums(False)
        try:
            c2 = m.make_caches()
            plain = [m.forward(toks[:5], 0, c2)] + [m.forward(toks[i:i + 1], i, c2) for i in range(5, 8)]
        finally:
            oracle.set_exact_sums(True)
        d_exact = max(max_rel_err(a, b) for a, b in zip(got, want))
        d_plain = max(max_rel_err(a, b) for a, b in zip(plain, want))
        if force_f16:
            assert d_exact < 0.25 * d_plain < 1e-2, (d_exact, d_plain)   # measured: 1.7e-7 / 2.0e-5 against 4.6e-4 / 8.2e-4
        else:
            assert d_exact < 2e-6 and d_exact < d_plain, (d_exact, d_plain)
