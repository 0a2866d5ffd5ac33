"""Parity of the HIP path (through the C ABI) against the CPU oracle on the same seeded inputs.

Tolerances are the ones the task states: logits within max relative error 1e-2 for f16 weights and 1e-4 for f32
(relative to the largest |logit|), greedy token ids identical on config 0.  Op-level checks are tighter.
"""
import os

import numpy as np
import pytest

import oracle
import rllama_amd
from rllama_amd import Tensor, TensorDType
from common import (CONFIG0, PER_LAYER, SMALL, TINY, Shape, make_gpu, make_oracle, max_rel_err, options, random_f32_weights, synth_weights)

pytestmark = pytest.mark.gpu
f32 = np.float32

TOL_F16 = 1e-2
TOL_F32 = 1e-4


def close_f16(got, want, mag=None, what=""):
    """got within one f16 rounding step of want, plus fp32 summation noise proportional to the magnitude `mag`
    of the summed terms (a result that is small through cancellation is not accurate to its own ulp)."""
    tol = ulp_f16(want)
    if mag is not None:
        tol = tol + 2e-6 * np.asarray(mag, np.float32)
    bad = np.abs(np.asarray(got, np.float32) - np.asarray(want, np.float32)) > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.size} elements more than one f16 step from the oracle"


def ulp_f16(v):
    """spacing of f16 at |v| (for 'at most one rounding step apart' checks)"""
    a = np.abs(np.asarray(v, np.float32)).astype(np.float16)
    return (np.nextafter(a, np.float16(np.inf)).astype(np.float32) - a.astype(np.float32))


# ------------------------------------------------------------------------------------------------------
# synthetic inputs: the device generator is bit-identical to the host one
# ------------------------------------------------------------------------------------------------------
def test_device_synth_equals_host(ctx):
    shape = SMALL
    ds = rllama_amd.DataSettings(ctx).force_f16()
    m = rllama_amd.Transformer(ctx, shape.dim, shape.n_layers, shape.n_heads, shape.ffn_hidden, shape.vocab_size,
                               shape.max_seq_len, shape.norm_eps, ds)
    m.fill_synthetic(seed=4, std=0.02)
    W = synth_weights(shape, seed=4, std=0.02)
    for (kind, layer), arr in W.items():
        r, c = shape.tensor_shape(kind)
        got = m.get_tensor(kind, layer, r, c)
        want = arr.view(np.float16).astype(np.float32) if arr.dtype == np.uint16 else arr
        assert np.array_equal(got, want.reshape(r, c)), (kind, layer)
    m.free()


# ------------------------------------------------------------------------------------------------------
# op level (mirrors the reference's GPU-vs-CPU tests, tensor.rs:2924-3209, tolerance 1e-2 there)
# ------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("m_rows,k", [(1, 8), (3, 64), (64, 512), (100, 1000), (4096, 4096), (11008, 4096), (4096, 11008), (257, 2816)])
def test_gemv_f16_weights(ctx, m_rows, k):
    rng = np.random.default_rng(m_rows * 31 + k)
    w = (rng.standard_normal((m_rows, k)) * 0.05).astype(f32)
    x = rng.standard_normal((1, k)).astype(f32)
    wh = oracle.f32_to_f16_bits(w)
    xh = oracle.f32_to_f16_bits(x)
    W = Tensor.from_numpy(ctx, wh)
    X = Tensor.from_numpy(ctx, x)
    # f16 mode: x rounded to f16, product rounded to f16 (tensor.rs:1476-1666)
    got = W.gemv(X, round_x=True, round_y=True).to_numpy()[0]
    want = oracle.f16_bits_to_f32(oracle.matmul_transposed_f16(xh, wh))[0]
    mag = np.abs(oracle.f16_bits_to_f32(xh).astype(np.float64))[0] @ np.abs(oracle.f16_bits_to_f32(wh).astype(np.float64)).T
    close_f16(got, want, mag, "gemv f16")
    assert np.mean(got != want) < 0.02                      # rounding flips are rare
    assert np.array_equal(got, got.astype(np.float16).astype(f32))
    # no rounding of the product: fp32 accumulate against float64
    got32 = W.gemv(X, round_x=True, round_y=False).to_numpy()[0]
    exact = oracle.f16_bits_to_f32(xh).astype(np.float64)[0] @ oracle.f16_bits_to_f32(wh).astype(np.float64).T
    assert np.allclose(got32, exact, rtol=1e-5, atol=1e-5 * np.abs(exact).max())
    # f32 activations against f16 weights (the output head's combination, transformer.rs:381)
    got_head = W.gemv(X, round_x=False, round_y=False).to_numpy()[0]
    exact_head = x.astype(np.float64)[0] @ oracle.f16_bits_to_f32(wh).astype(np.float64).T
    assert np.allclose(got_head, exact_head, rtol=1e-5, atol=1e-5 * np.abs(exact_head).max())


@pytest.mark.parametrize("m_rows,k,burst", [(300, 11008, 11), (130, 5376, 11), (64, 4608, 9), (2100, 13824, 9), (77, 5120, 10), (40, 3584, 7), (9, 6656, 8)])
def test_gemv_burst_length_follows_the_row(ctx, m_rows, k, burst):
    """The single-row product issues its loads in bursts of 7, 9, 10 or 11 per lane where that divides the row's pieces of 512
    halves and 8 does not (a row that ends inside a piece counts as whole pieces: 11008 -> 22, 5376 -> 11); the last case has
    13 pieces and keeps 8 with a partial last burst.  Every lane still adds its products in the order of the pieces, so the
    bits are those of the fixed burst length; and against the oracle (tensor.rs:1476-1666)."""
    assert -(-k // 512) % burst == 0 or burst == 8
    rng = np.random.default_rng(m_rows + k)
    wh = oracle.f32_to_f16_bits((rng.standard_normal((m_rows, k)) * 0.05).astype(f32))
    x = rng.standard_normal((1, k)).astype(f32)
    xh = oracle.f32_to_f16_bits(x)
    W, X = Tensor.from_numpy(ctx, wh), Tensor.from_numpy(ctx, x)
    got = W.gemv(X, round_x=True, round_y=True).to_numpy()[0]
    got32 = W.gemv(X, round_x=False, round_y=False).to_numpy()[0]
    with options(ctx, GEMV_BURST="0"):
        assert np.array_equal(got, W.gemv(X, round_x=True, round_y=True).to_numpy()[0])
        assert np.array_equal(got32, W.gemv(X, round_x=False, round_y=False).to_numpy()[0])
    want = oracle.f16_bits_to_f32(oracle.matmul_transposed_f16(xh, wh))[0]
    mag = np.abs(oracle.f16_bits_to_f32(xh).astype(np.float64))[0] @ np.abs(oracle.f16_bits_to_f32(wh).astype(np.float64)).T
    close_f16(got, want, mag, "gemv f16, burst length by row")
    assert np.mean(got != want) < 0.02


@pytest.mark.parametrize("m_rows,k", [(5, 4), (64, 512), (1000, 1000), (4096, 4096)])
def test_gemv_f32_weights(ctx, m_rows, k):
    rng = np.random.default_rng(m_rows * 17 + k)
    w = rng.uniform(-1, 1, (m_rows, k)).astype(f32)
    x = rng.uniform(-1, 1, (1, k)).astype(f32)
    got = Tensor.from_numpy(ctx, w).gemv(Tensor.from_numpy(ctx, x), False, False).to_numpy()[0]
    want = oracle.matmul_transposed_f32(x, w)[0]
    scale = np.abs(want).max()
    assert np.allclose(got, want, rtol=0, atol=1e-5 * scale)  # tensor.rs:2701-2747 (1e-5)


def test_matrix_mul_transposed_multi_row(ctx):
    rng = np.random.default_rng(5)
    for n, m_rows, k in [(2, 3, 8), (5, 33, 64), (16, 100, 256)]:
        a = oracle.f32_to_f16_bits(rng.uniform(-1, 1, (n, k)).astype(f32))
        b = oracle.f32_to_f16_bits(rng.uniform(-1, 1, (m_rows, k)).astype(f32))
        got = Tensor.from_numpy(ctx, a).matrix_mul_transposed(Tensor.from_numpy(ctx, b)).to_numpy().astype(f32)
        want = oracle.f16_bits_to_f32(oracle.matmul_transposed_f16(a, b))
        assert got.shape == (n, m_rows)
        mag = np.abs(oracle.f16_bits_to_f32(a).astype(np.float64)) @ np.abs(oracle.f16_bits_to_f32(b).astype(np.float64)).T
        close_f16(got, want, mag, "matmul f16")
        a32 = rng.uniform(-1, 1, (n, k)).astype(f32)
        b32 = rng.uniform(-1, 1, (m_rows, k)).astype(f32)
        got32 = Tensor.from_numpy(ctx, a32).matrix_mul_transposed(Tensor.from_numpy(ctx, b32)).to_numpy()
        assert np.allclose(got32, oracle.matmul_transposed_f32(a32, b32), rtol=0, atol=1e-5 * k ** 0.5)
    # the reference's shape panics (tensor.rs:1261-1278) come back as errors
    with pytest.raises(rllama_amd.RllamaHipError):
        Tensor.from_numpy(ctx, np.zeros((2, 8), f32)).matrix_mul_transposed(Tensor.from_numpy(ctx, np.zeros((2, 16), f32)))
    with pytest.raises(rllama_amd.RllamaHipError):
        Tensor.from_numpy(ctx, np.zeros((2, 8), f32)).matrix_mul_transposed(Tensor.from_numpy(ctx, np.zeros((2, 8), np.uint16)))


def test_random_products_against_float64(ctx):
    """A seeded sweep over product shapes: 1 to 1300 rows (the values around the tile edges more often), ragged column counts,
    K any multiple of 8 (f16) or 4 (fp32) up to 4800; f16 results within one f16 step of the float64 product plus fp32
    summation noise, fp32 results within summation noise."""
    rng = np.random.default_rng(77)
    for case in range(48):
        f16 = bool(rng.integers(0, 2))
        m = int(rng.choice([1, 2, 3, 7, 31, 32, 33, 64, 65, 127, 128, 129, 255, 257, 500, 1024, 1100])) if rng.integers(0, 2) else int(rng.integers(1, 1300))
        n = int(rng.integers(1, 3000)) if rng.integers(0, 4) else int(rng.choice([64, 128, 192, 256, 3072, 4096]))
        k = (8 if f16 else 4) * int(rng.integers(1, 600)) if rng.integers(0, 2) else 64 * int(rng.integers(1, 70))
        what = f"case {case}: f16 {f16}, {m} x {n} x {k}"
        print(what, flush=True)
        a = rng.uniform(-1, 1, (m, k)).astype(f32)
        b = rng.uniform(-1, 1, (n, k)).astype(f32)
        if f16:
            a, b = a.astype(np.float16), b.astype(np.float16)
            got = Tensor.from_numpy(ctx, a.view(np.uint16)).matrix_mul_transposed(Tensor.from_numpy(ctx, b.view(np.uint16))).to_numpy().view(np.float16)
        else:
            got = Tensor.from_numpy(ctx, a).matrix_mul_transposed(Tensor.from_numpy(ctx, b)).to_numpy()
        want = a.astype(np.float64) @ b.astype(np.float64).T
        mag = np.abs(a.astype(np.float64)) @ np.abs(b.astype(np.float64)).T
        tol = np.abs(want) * 2.0 ** -10 + mag * 1.6e-6 + 1e-6 if f16 else mag * 3e-6 + 1e-7
        assert got.shape == want.shape and np.all(np.abs(got.astype(np.float64) - want) <= tol), what


def test_elementwise_ops(ctx):
    rng = np.random.default_rng(6)
    for rows, cols in [(1, 1), (3, 5), (64, 64), (37, 300)]:
        a = rng.uniform(-4, 4, (rows, cols)).astype(f32)
        b = rng.uniform(-4, 4, (rows, cols)).astype(f32)
        A, B = Tensor.from_numpy(ctx, a), Tensor.from_numpy(ctx, b)
        want_silu = np.array([[oracle.silu(v) for v in row] for row in a], dtype=f32)
        assert np.allclose(A.silu().to_numpy(), want_silu, rtol=1e-6, atol=1e-7)
        assert np.array_equal(A.hadamard_product(B).to_numpy(), a * b)
        assert np.array_equal(A.transpose().to_numpy(), a.T)
        assert np.array_equal(A.clone().to_numpy(), a)
        # f16 tensors: computed in f32, stored rounded (tensor_opencl_support.rs:668-697)
        ah, bh = a.astype(np.float16), b.astype(np.float16)
        AH, BH = Tensor.from_numpy(ctx, ah), Tensor.from_numpy(ctx, bh)
        assert np.array_equal(AH.hadamard_product(BH).to_numpy(), (ah.astype(f32) * bh.astype(f32)).astype(np.float16))
        assert np.array_equal(AH.transpose().to_numpy(), ah.T)
        got = AH.silu().to_numpy().astype(f32)
        want = np.array([[oracle.silu(float(v)) for v in row] for row in ah.astype(f32)], dtype=f32)
        close_f16(got, want, None, "silu f16")


def test_rmsnorm_and_rope_ops(ctx):
    rng = np.random.default_rng(7)
    for rows, d in [(1, 64), (4, 1024), (3, 4096)]:
        x = (rng.standard_normal((rows, d)) * 2).astype(f32)
        w = rng.uniform(0.5, 1.5, (1, d)).astype(f32)
        got = Tensor.from_numpy(ctx, x).rmsnorm(Tensor.from_numpy(ctx, w), 1e-6).to_numpy()
        want = np.stack([oracle.rmsnorm_row(x[r], w[0], 1e-6) for r in range(rows)])
        assert np.allclose(got, want, rtol=2e-6, atol=1e-7)
        gotr = Tensor.from_numpy(ctx, x).rmsnorm(Tensor.from_numpy(ctx, w), 1e-6, round_y=True).to_numpy()
        close_f16(gotr, oracle.f16r(want), None, "rmsnorm f16r")
    for H, hd, pos in [(2, 32, 0), (16, 64, 5), (32, 128, 1023)]:
        x = rng.standard_normal((1, H * hd)).astype(f32)
        T = Tensor.from_numpy(ctx, x)
        T.rope_inplace(H, hd, pos)
        fc = oracle.freqs_cis(hd, pos + 1)
        want = oracle.rope_row(x, H, hd, fc[pos])
        assert np.array_equal(T.to_numpy()[0], want)          # same table, same unfused f32 arithmetic: bit-exact


# ------------------------------------------------------------------------------------------------------
# forward
# ------------------------------------------------------------------------------------------------------
def _run_both(ctx, shape, W, force_f16, toks, n_prompt, tol):
    om = make_oracle(shape, W, force_f16)
    gm = make_gpu(ctx, shape, W, force_f16)
    oc, gc = om.make_caches(), gm.make_caches()
    worst = 0.0
    a = om.forward(toks[:n_prompt], 0, oc)
    b = gm.forward(toks[:n_prompt], 0, gc)
    worst = max(worst, max_rel_err(b, a))
    for i in range(n_prompt, len(toks)):
        a = om.forward(toks[i:i + 1], i, oc)
        b = gm.forward(toks[i:i + 1], i, gc)
        worst = max(worst, max_rel_err(b, a))
    assert worst < tol, f"max relative logit error {worst:.3e} (tolerance {tol})"
    return om, gm, oc, gc, worst


@pytest.mark.parametrize("shape", [TINY, SMALL], ids=["tiny", "small"])
def test_forward_f16_mode(ctx, shape):
    W = synth_weights(shape, seed=21, std=0.08, norm_ones=False)
    toks = np.random.default_rng(22).integers(0, shape.vocab_size, 12)
    om, gm, oc, gc, worst = _run_both(ctx, shape, W, True, toks, 7, TOL_F16)
    # KV cache: same layout view, f16-rounded, at most one f16 step from the oracle's
    T = len(toks)
    for l in range(shape.n_layers):
        for h in range(shape.n_heads):
            for which in (0, 1):
                g, o = gc.read(l, h, which), oc.read(l, h, which)
                assert np.array_equal(g, g.astype(np.float16).astype(f32))
                assert not np.any(g[:, T:])
                assert np.all(np.abs(g[:, :T] - o[:, :T]) <= 2 * ulp_f16(o[:, :T]) + 1e-3 * np.abs(o[:, :T]).max())
    gm.free()


@pytest.mark.parametrize("n_heads,n,cap", [(2, 300, 320), (2, 129, 320), (4, 64, 320), (4, 1, 320), (2, 289, 290), (4, 33, 35)],
                         ids=["hd128-n300", "hd128-n129", "hd64-n64", "hd64-n1", "hd128-n289-cap290", "hd64-n33-cap35"])
def test_prefill_fused_attention_head_dims(ctx, n_heads, n, cap):
    """The one-kernel causal attention of the multi-token forward (head_dim 128 and 64; ragged query and key tiles, also a
    cache whose capacity ends inside the last key tile) against the oracle."""
    shape = Shape(dim=256, n_layers=2, n_heads=n_heads, ffn_hidden=512, vocab_size=128, max_seq_len=cap)
    W = synth_weights(shape, seed=45, std=0.08, norm_ones=False)
    toks = np.random.default_rng(46).integers(0, shape.vocab_size, n + 1)
    om, gm = make_oracle(shape, W, True), make_gpu(ctx, shape, W, True)
    oc, gc = om.make_caches(), gm.make_caches()
    m = max(n, 2)  # a 1-token call is a decode step; make it a 2-token prefill instead
    want, got = om.forward(toks[:m], 0, oc), gm.forward(toks[:m], 0, gc)
    assert max_rel_err(got, want) < TOL_F16, max_rel_err(got, want)
    # and the step after it reads the cache the prefill wrote
    want, got = om.forward(toks[m:m + 1], m, oc) if m < len(toks) else want, gm.forward(toks[m:m + 1], m, gc) if m < len(toks) else got
    assert max_rel_err(got, want) < TOL_F16
    gm.free()


def test_prefill_attention_gemm_form_for_large_heads(ctx):
    """The PREFILL_ATTN=gemm switch keeps head_dim 64 / 128 on the two-GEMM form of the
    prefill attention (hi | lo halves of q and of P as K segments, tiles above the diagonal skipped, V^T in natural key
    order): same function as the one-kernel form and the oracle."""
    shape = Shape(dim=256, n_layers=2, n_heads=2, ffn_hidden=512, vocab_size=128, max_seq_len=320)   # head_dim 128
    W = synth_weights(shape, seed=53, std=0.08, norm_ones=False)
    toks = np.random.default_rng(54).integers(0, shape.vocab_size, 301)
    om = make_oracle(shape, W, True)
    gm = make_gpu(ctx, shape, W, True)
    for n in (300, 65):
        oc, ca, cb = om.make_caches(), gm.make_caches(), gm.make_caches()
        want = om.forward(toks[:n], 0, oc)
        a = gm.forward(toks[:n], 0, ca)
        with options(ctx, PREFILL_ATTN="gemm"):
            b = gm.forward(toks[:n], 0, cb)
        assert max_rel_err(a, want) < TOL_F16 and max_rel_err(b, want) < TOL_F16, (n, max_rel_err(a, want), max_rel_err(b, want))
        want1 = om.forward(toks[n:n + 1], n, oc)
        assert max_rel_err(gm.forward(toks[n:n + 1], n, cb), want1) < TOL_F16
    gm.free()


def test_prefill_odd_dims_register_staged_gemm(ctx):
    """dim 48 and ffn 104 are not multiples of the fast GEMM's K-tile, so every product of the multi-token forward (with the
    SiLU-gate and residual epilogues, and the two attention products at head_dim 16) runs on the register-staged kernel."""
    shape = Shape(dim=48, n_layers=2, n_heads=3, ffn_hidden=104, vocab_size=50, max_seq_len=40)
    W = synth_weights(shape, seed=55, std=0.1, norm_ones=False)
    toks = np.random.default_rng(56).integers(0, shape.vocab_size, 31)
    om, gm = make_oracle(shape, W, True), make_gpu(ctx, shape, W, True)
    for n in (30, 3):
        oc, gc = om.make_caches(), gm.make_caches()
        assert max_rel_err(gm.forward(toks[:n], 0, gc), om.forward(toks[:n], 0, oc)) < TOL_F16
        assert max_rel_err(gm.forward(toks[n:n + 1], n, gc), om.forward(toks[n:n + 1], n, oc)) < TOL_F16
    gm.free()


def test_prefill_short_prompt_split_k(ctx):
    """Few prompt rows leave few output tiles, so the projections run split along K (uneven pieces: 22 K-tiles over 5
    workgroups for w2) with a second kernel that adds the partial sums and applies the epilogue; against the oracle."""
    shape = Shape(dim=512, n_layers=2, n_heads=4, ffn_hidden=1408, vocab_size=64, max_seq_len=128)
    W = synth_weights(shape, seed=47, std=0.05, norm_ones=False)
    toks = np.random.default_rng(48).integers(0, shape.vocab_size, 101)
    om, gm = make_oracle(shape, W, True), make_gpu(ctx, shape, W, True)
    for n in (100, 5):
        oc, gc = om.make_caches(), gm.make_caches()
        got = gm.forward(toks[:n], 0, gc)
        assert max_rel_err(got, om.forward(toks[:n], 0, oc)) < TOL_F16
        assert max_rel_err(gm.forward(toks[n:n + 1], n, gc), om.forward(toks[n:n + 1], n, oc)) < TOL_F16
        # the kernel that adds the partial sums of wo / w2 also writes the RMSNorm that follows; with that switched off the
        # norm runs as a kernel of its own: same arithmetic in the same order, so the same bits
        with options(ctx, FINISH_NORM="0"):
            g2 = gm.make_caches()
            assert np.array_equal(gm.forward(toks[:n], 0, g2), got)
    gm.free()


def test_prefill_wide_ffn_largest_tile(ctx):
    """An FFN wide enough that w1 / w3 (1024 x 16384 outputs) take the 256 x 256 tile, whose SiLU-gate epilogue reads the gate
    in the epilogue instead of ahead of the K loop; against the oracle."""
    shape = Shape(dim=256, n_layers=1, n_heads=2, ffn_hidden=16384, vocab_size=64, max_seq_len=1024)
    W = synth_weights(shape, seed=49, std=0.03, norm_ones=False)
    toks = np.random.default_rng(50).integers(0, shape.vocab_size, 1024)
    om, gm = make_oracle(shape, W, True), make_gpu(ctx, shape, W, True)
    want = om.forward(toks, 0, om.make_caches())
    got = gm.forward(toks, 0, gm.make_caches())
    assert max_rel_err(got, want) < TOL_F16, max_rel_err(got, want)
    gm.free()


@pytest.mark.parametrize("dim,heads,ffn,n", [(256, 2, 1000, 300), (128, 2, 192, 256), (192, 3, 1544, 515)])
def test_prefill_w1_w3_in_one_pass(ctx, dim, heads, ffn, n):
    """w1 and w3 as one pass over the normalised rows (two accumulator sets per wavefront, SiLU(w1 x) * (w3 x) straight from
    them: transformer.rs:551-565), forced onto shapes the oracle handles quickly: ragged last row and column tiles (300 and
    515 rows on 256-row tiles, 1000 = 5 x 192 + 40 and 1544 = 8 x 192 + 8 columns), exactly one tile, three K-tiles.  Same
    MFMA sequence per output element as the two-launch form, so the same bits; and against the oracle."""
    shape = Shape(dim=dim, n_layers=2, n_heads=heads, ffn_hidden=ffn, vocab_size=64, max_seq_len=n + 2)
    W = synth_weights(shape, seed=61, std=0.05, norm_ones=False)
    toks = np.random.default_rng(62).integers(0, shape.vocab_size, n + 1)
    om, gm = make_oracle(shape, W, True), make_gpu(ctx, shape, W, True)
    got = {}
    # workgroups of 256 x 192 of both products (eight wavefronts), 128 x 192 (four), the short-prompt forms 32 / 64 / 128 x 64, two launches
    # (GEMM_KGROUP=0: the two-launch form on the tile-splitting kernel, whose sum over k runs in the same order as the one-pass kernel's)
    for mode in ("1", "2", "3", "4", "5", "0"):
        with options(ctx, GEMM_KGROUP="0", GEMM_DUAL=mode):
            gc = gm.make_caches()
            got[mode] = (gm.forward(toks[:n], 0, gc), gm.forward(toks[n:n + 1], n, gc))
    for mode in ("1", "2", "3", "4", "5"):
        assert np.array_equal(got[mode][0], got["0"][0]) and np.array_equal(got[mode][1], got["0"][1]), mode
    oc = om.make_caches()
    assert max_rel_err(got["1"][0], om.forward(toks[:n], 0, oc)) < TOL_F16
    assert max_rel_err(got["1"][1], om.forward(toks[n:n + 1], n, oc)) < TOL_F16
    gm.free()


@pytest.mark.parametrize("dim,heads,ffn,n", [(256, 2, 384, 300), (128, 2, 256, 70), (64, 4, 128, 130), (192, 3, 256, 515), (512, 4, 640, 1024)])
def test_prefill_rope_and_cache_write_in_the_projection(ctx, dim, heads, ffn, n):
    """RoPE, the hi + lo halves of q, the cache rows and V^T written by the epilogue of the wq|wk|wv product (transformer.rs:
    694-761 with seq_len > 1) against the same steps as a kernel of their own on the stored product: same values at the
    same rounding points, so the same bits in the logits, in the token step that follows, and in every cache row.  Head
    dimensions 128, 64 and 16 (the last takes the two-GEMM attention, which reads V^T in plain position order); ragged row
    tiles; wavefront tiles that straddle the q | k and k | v column boundaries; and against the oracle."""
    shape = Shape(dim=dim, n_layers=2, n_heads=heads, ffn_hidden=ffn, vocab_size=64, max_seq_len=n + 3)
    W = synth_weights(shape, seed=71, std=0.05, norm_ones=False)
    toks = np.random.default_rng(72).integers(0, shape.vocab_size, n + 1)
    om, gm = make_oracle(shape, W, True), make_gpu(ctx, shape, W, True)
    got = {}
    # (GEMM_KGROUP=0: the stored product on the tile-splitting kernel, whose sum over k runs in the same order as the kernel with the epilogue)
    for mode in ("1", "0"):
        with options(ctx, GEMM_KGROUP="0", GEMM_ROPE=mode):
            gc = gm.make_caches()
            a, b = gm.forward(toks[:n], 0, gc), gm.forward(toks[n:n + 1], n, gc)
            got[mode] = (a, b, [gc.read(l, h, w) for l in range(2) for h in range(heads) for w in (0, 1)])
    assert np.array_equal(got["1"][0], got["0"][0]) and np.array_equal(got["1"][1], got["0"][1])
    for x, y in zip(got["1"][2], got["0"][2]):
        assert np.array_equal(x, y)
    oc = om.make_caches()
    assert max_rel_err(got["1"][0], om.forward(toks[:n], 0, oc)) < TOL_F16
    assert max_rel_err(got["1"][1], om.forward(toks[n:n + 1], n, oc)) < TOL_F16
    gm.free()


@pytest.mark.parametrize("dim,heads,ffn,n", [(256, 2, 704, 300), (512, 4, 1408, 520), (128, 2, 192, 130)])
def test_prefill_k_steps_split_among_wavefronts(ctx, dim, heads, ffn, n):
    """wo and w2 (and the other projections at these sizes) on the kernel whose wavefronts split the K-steps of a 128 x 128 tile
    and add their four partial sums through LDS: against the oracle, and close to the tile-splitting kernel (the order of the
    fp32 additions differs, so single f16 rounding decisions may)."""
    shape = Shape(dim=dim, n_layers=2, n_heads=heads, ffn_hidden=ffn, vocab_size=64, max_seq_len=n + 2)
    W = synth_weights(shape, seed=81, std=0.05, norm_ones=False)
    toks = np.random.default_rng(82).integers(0, shape.vocab_size, n + 1)
    om, gm = make_oracle(shape, W, True), make_gpu(ctx, shape, W, True)
    got = {}
    for mode in ("1", "0"):
        with options(ctx, GEMM_KGROUP=mode):
            gc = gm.make_caches()
            got[mode] = (gm.forward(toks[:n], 0, gc), gm.forward(toks[n:n + 1], n, gc))
    oc = om.make_caches()
    want = (om.forward(toks[:n], 0, oc), om.forward(toks[n:n + 1], n, oc))
    for i in (0, 1):
        assert max_rel_err(got["1"][i], want[i]) < TOL_F16
        assert max_rel_err(got["1"][i], got["0"][i]) < 2e-3
    gm.free()


def test_prefill_long_prompt_causal_tiles(ctx):
    """A prompt long enough that the score matrix spans several GEMM tiles per head (tiles above the diagonal are
    skipped, the probability product stops at the diagonal) on the large-tile path; compared with the oracle."""
    shape = Shape(dim=1024, n_layers=1, n_heads=16, ffn_hidden=256, vocab_size=64, max_seq_len=1024)
    W = synth_weights(shape, seed=43, std=0.05, norm_ones=False)
    toks = np.random.default_rng(44).integers(0, shape.vocab_size, 1024)
    om, gm = make_oracle(shape, W, True), make_gpu(ctx, shape, W, True)
    for n in (1024, 700):
        want = om.forward(toks[:n], 0, om.make_caches())
        got = gm.forward(toks[:n], 0, gm.make_caches())
        assert max_rel_err(got, want) < TOL_F16, (n, max_rel_err(got, want))
    gm.free()


@pytest.mark.parametrize("shape", [TINY, SMALL], ids=["tiny", "small"])
def test_forward_f32_mode(ctx, shape):
    W = random_f32_weights(shape, seed=23, std=0.08)
    toks = np.random.default_rng(24).integers(0, shape.vocab_size, 12)
    om, gm, oc, gc, worst = _run_both(ctx, shape, W, False, toks, 7, TOL_F32)
    T = len(toks)
    for l in range(shape.n_layers):
        for h in range(shape.n_heads):
            for which in (0, 1):
                assert np.allclose(gc.read(l, h, which)[:, :T], oc.read(l, h, which)[:, :T], rtol=1e-4, atol=1e-5)
    gm.free()


def test_forward_f32_mode_with_f16_file_weights(ctx):
    """No --f16: the f16 file contents are widened to f32 tensors (tensor.rs:2467) and nothing is rounded."""
    shape = SMALL
    W = synth_weights(shape, seed=25, std=0.08)
    toks = np.random.default_rng(26).integers(0, shape.vocab_size, 10)
    _, gm, _, _, _ = _run_both(ctx, shape, W, False, toks, 6, TOL_F32)
    gm.free()


def test_long_context_split_attention(ctx):
    """Enough positions that the single-query attention splits the sequence over several blocks per head."""
    shape = Shape(dim=256, n_layers=2, n_heads=2, ffn_hidden=512, vocab_size=300, max_seq_len=700)  # head_dim 128
    for force_f16, tol in ((True, TOL_F16), (False, TOL_F32)):
        W = synth_weights(shape, seed=27, std=0.1, norm_ones=False)
        toks = np.random.default_rng(28).integers(0, shape.vocab_size, 660)
        om, gm = make_oracle(shape, W, force_f16), make_gpu(ctx, shape, W, force_f16)
        oc, gc = om.make_caches(), gm.make_caches()
        a = om.forward(toks[:650], 0, oc)
        b = gm.forward(toks[:650], 0, gc)
        assert max_rel_err(b, a) < tol
        for i in range(650, 660):
            assert max_rel_err(gm.forward(toks[i:i + 1], i, gc), om.forward(toks[i:i + 1], i, oc)) < tol
        gm.free()


def test_very_long_context_capped_splits(ctx):
    """Positions beyond (splits cap) x (chunk): every attention block takes a longer share; also a 4300-token prompt through
    the one-kernel prefill attention (68 key tiles) and the KV cache it leaves.  f16 mode, head_dim 64."""
    shape = Shape(dim=128, n_layers=1, n_heads=2, ffn_hidden=256, vocab_size=200, max_seq_len=4400)
    W = synth_weights(shape, seed=29, std=0.1, norm_ones=False)
    toks = np.random.default_rng(30).integers(0, shape.vocab_size, 4320)
    om, gm = make_oracle(shape, W, True), make_gpu(ctx, shape, W, True)
    oc, gc = om.make_caches(), gm.make_caches()
    assert max_rel_err(gm.forward(toks[:4300], 0, gc), om.forward(toks[:4300], 0, oc)) < TOL_F16
    for i in range(4300, 4320):
        assert max_rel_err(gm.forward(toks[i:i + 1], i, gc), om.forward(toks[i:i + 1], i, oc)) < TOL_F16, i
    gm.free()


def test_config0_greedy_tokens_identical(ctx):
    """Config 0: d=1024, L=8, H=16, F=2816, V=32000, f16, seed 0; 16 prompt ids, then 64 greedy steps."""
    shape = CONFIG0
    W = synth_weights(shape, seed=0, std=0.02)
    prompt = rllama_amd.synth_tokens(0, 16, 3, 32000)
    om, gm = make_oracle(shape, W, True), make_gpu(ctx, shape, W, True)
    # oracle token loop (rllama_main.rs:821-897 at top_k = 1)
    oc = om.make_caches()
    toks = list(prompt)
    prev = 0
    want_ids, gaps, o_logits = [], [], []
    for _ in range(64):
        logits = om.forward(toks[prev:], prev, oc)
        tok, _, ties = oracle.sample_greedy(logits)
        l2 = logits.copy()
        l2[0] = 0.0
        top2 = np.sort(l2)[-2:]
        gaps.append(float(top2[1] - top2[0]))
        assert ties == 1, "exact probability tie in the oracle: the reference's sort order is unspecified here"
        want_ids.append(tok)
        o_logits.append(logits)
        toks.append(tok)
        prev = len(toks) - 1
    # device loop: one call
    gc = gm.make_caches()
    got_ids, ms_first, ms_tok = gm.generate_greedy(prompt, 64, gc)
    assert got_ids.tolist() == want_ids, f"first divergence at step {next(i for i in range(64) if got_ids[i] != want_ids[i])}, min top-2 gap {min(gaps):.3e}"
    # the same loop driven through forward(): logits within tolerance at every step
    gc2 = gm.make_caches()
    toks2 = list(prompt)
    prev = 0
    worst = 0.0
    for step in range(64):
        lg = gm.forward(toks2[prev:], prev, gc2)
        worst = max(worst, max_rel_err(lg, o_logits[step]))
        toks2.append(want_ids[step])
        prev = len(toks2) - 1
    assert worst < TOL_F16, worst
    # forward_greedy agrees with generate_greedy
    gc3 = gm.make_caches()
    assert gm.forward_greedy(prompt, 0, gc3) == want_ids[0]
    assert gm.forward_greedy([want_ids[0]], 16, gc3) == want_ids[1]
    print(f"config0: worst logit rel err {worst:.2e}, min top-2 gap {min(gaps):.2e}, {ms_tok:.3f} ms/token")
    gm.free()


def test_config0_f32_mode_end_to_end(ctx):
    """Config 0 in the reference's default mode (no --f16: fp32 weights, activations and cache; the file's f16 values widened,
    transformer.rs:38-49, tensor.rs:2467): all 8 layers end to end, 16 prompt ids on the fp32 matrix cores, then 64 greedy
    steps; logits within 1e-4 of the oracle's at every call, ids identical."""
    shape = CONFIG0
    W = synth_weights(shape, seed=0, std=0.02)
    prompt = [int(t) for t in rllama_amd.synth_tokens(0, 16, 3, 32000)]
    om, gm = make_oracle(shape, W, False), make_gpu(ctx, shape, W, False)
    oc, gc = om.make_caches(), gm.make_caches()
    want = om.forward(prompt, 0, oc)
    worst = max_rel_err(gm.forward(prompt, 0, gc), want)
    ids = []
    for step in range(64):
        tok, _, ties = oracle.sample_greedy(want)
        assert ties == 1
        ids.append(tok)
        if step == 63:
            break
        want = om.forward([tok], 16 + step, oc)
        worst = max(worst, max_rel_err(gm.forward([tok], 16 + step, gc), want))
    assert worst < 1e-4, worst
    got, _, _ = gm.generate_greedy(prompt, 64, gm.make_caches())
    assert got.tolist() == ids
    print(f"config 0, f32 mode: worst logit rel err {worst:.2e}")
    gm.free()


def test_set_option_names_and_values(ctx):
    """rlh_set_option: the switches rlh_init reads from RLLAMA_HIP_<NAME> once, changed per context afterwards; unknown names
    and unusable values are refused and leave the switch as it was."""
    for name, good, bad in (("GEMM_DUAL", "3", "9"), ("ATTN_MERGE", "0", "1"), ("ATTN_CHUNK", "64", "5"), ("GEMM_TILE", "2", "7"),
                            ("PREFILL_ATTN", "gemm", "whatever"), ("PREFILL_ATTN_ORDER", "1", "3")):
        ctx.set_option(name, good)
        with pytest.raises(rllama_amd.RllamaHipError) as ei:
            ctx.set_option(name, bad)
        assert ei.value.code == 1 and name in str(ei.value)
        ctx.set_option(name, None)
    for name in ("NO_SUCH_SWITCH", "FUSED", "GEMM_SIMPLE", ""):
        with pytest.raises(rllama_amd.RllamaHipError):
            ctx.set_option(name, "1")
    # a switch takes effect on the next call of an existing model and goes back with None: the split attention merged by a
    # second launch and inside the kernel give the same bits (the same partial results, added in the same order)
    shape = Shape(dim=128, n_layers=1, n_heads=2, ffn_hidden=256, vocab_size=64, max_seq_len=600)
    gm = make_gpu(ctx, shape, synth_weights(shape, seed=9, std=0.08), True)
    toks = np.random.default_rng(10).integers(0, 64, 500)
    c = gm.make_caches()
    gm.forward(toks, 0, c)
    c2 = c.true_clone()
    a = gm.forward([5], 500, c)
    with options(ctx, ATTN_MERGE="0", ATTN_CHUNK="64"):
        b = gm.forward([5], 500, c2)
    assert np.array_equal(gm.forward([7], 501, c), gm.forward([7], 501, c2)) and max_rel_err(a, b) < 1e-3
    gm.free()


def test_cache_services_and_errors(ctx):
    shape = TINY
    W = synth_weights(shape, seed=31, std=0.1)
    om, gm = make_oracle(shape, W, True), make_gpu(ctx, shape, W, True)
    oc, gc = om.make_caches(), gm.make_caches()
    toks = [5, 17, 3, 90, 41]
    om.forward(toks, 0, oc)
    gm.forward(toks, 0, gc)
    # true_clone: independent deep copy (transformer.rs:207-213)
    g2 = gc.true_clone()
    a = gm.forward([7], 5, gc)
    b = gm.forward([7], 5, g2)
    assert np.array_equal(a, b)
    c = gm.forward([9], 5, g2)
    assert np.array_equal(gm.forward([7], 5, gc), a) and not np.array_equal(c, a)
    # shift_left (transformer.rs:180-205)
    before = gc.read(1, 1, 0).copy()
    gc.shift_left(2)
    after = gc.read(1, 1, 0)
    T = shape.max_seq_len
    assert np.array_equal(after[:, :T - 2], before[:, 2:])
    assert np.array_equal(after[:, T - 2:], np.repeat(before[:, T - 1:], 2, axis=1))
    oc.shift_left(2)
    om.forward([7], 5, oc)  # keep the oracle's position 5 comparable
    assert np.all(np.abs(after[:, :3] - oc.read(1, 1, 0)[:, :3]) <= 2 * ulp_f16(after[:, :3]) + 1e-3)
    # the reference's panics are errors here, and nothing is launched
    for bad in (lambda: gm.forward([1, 2], 3, gc), lambda: gm.forward([1], shape.max_seq_len, gc),
                lambda: gm.forward([shape.vocab_size], 0, gc), lambda: gm.forward([], 0, gc)):
        with pytest.raises(rllama_amd.RllamaHipError):
            bad()
    other = make_gpu(ctx, shape, W, True)
    with pytest.raises(rllama_amd.RllamaHipError):
        other.forward([1], 0, gc)                         # caches of another model
    ds = rllama_amd.DataSettings(ctx).force_f16()
    empty = rllama_amd.Transformer(ctx, shape.dim, shape.n_layers, shape.n_heads, shape.ffn_hidden, shape.vocab_size,
                                   shape.max_seq_len, shape.norm_eps, ds)
    with pytest.raises(rllama_amd.RllamaHipError):
        empty.forward([1], 0, empty.make_caches())       # weights never set
    with pytest.raises(rllama_amd.RllamaHipError):
        empty.set_tensor(rllama_amd.WQ, 0, np.zeros((3, 3), np.uint16))
    gm.free()
    other.free()
    empty.free()


def test_percentage_to_gpu_rule(ctx):
    """DataSettings::percentage_to_gpu clamp (transformer.rs:91-103) and the split rule (:262-279)."""
    shape = TINY
    for p, want in [(1.0, 1), (7.0, 1), (0.0, 0), (-3.0, 0), (float("nan"), 0), (0.5, 1), (0.49, 0)]:
        ds = rllama_amd.DataSettings(ctx).force_f16().percentage_to_gpu(p)
        m = rllama_amd.Transformer(ctx, shape.dim, shape.n_layers, shape.n_heads, shape.ffn_hidden, shape.vocab_size,
                                   shape.max_seq_len, shape.norm_eps, ds)
        assert m.last_layer_on_gpu() == want, p
        m.free()


def test_random_small_shapes_against_the_oracle(ctx):
    """A seeded sweep over model shapes nobody would pick by hand: head dims 16 to 128, one to five heads, ffn widths that are
    only multiples of 8, odd vocabularies and sequence capacities, prompts up to the capacity, both modes and both prefill
    paths; logits of the prompt call and of single-token calls after it, and the last head's cache planes, against the oracle."""
    rng = np.random.default_rng(2024)
    for case in range(32):
        hd = int(rng.choice([16, 32, 64, 128]))
        H = int(rng.integers(1, 6))
        ffn = 8 * int(rng.integers(1, 200))
        vocab = int(rng.integers(5, 700))
        L = int(rng.integers(1, 4))
        max_seq = int(rng.integers(4, 150)) if rng.integers(0, 3) else int(rng.integers(150, 700))
        n_prompt = int(rng.integers(1, max_seq - 2))
        f16 = bool(rng.integers(0, 2))
        tbt = bool(rng.integers(0, 2))
        n_dec = int(min(max_seq - n_prompt - 1, rng.integers(1, 5)))
        what = f"case {case}: head_dim {hd} heads {H} ffn {ffn} vocab {vocab} layers {L} max_seq {max_seq} prompt {n_prompt} f16 {f16} token-by-token {tbt}"
        print(what, flush=True)
        shape = Shape(hd * H, L, H, ffn, vocab, max_seq)
        W = synth_weights(shape, seed=case, std=0.05, norm_ones=False)
        om, gm = make_oracle(shape, W, f16), make_gpu(ctx, shape, W, f16)
        gm.set_prefill_mode(tbt)
        oc, gc = om.make_caches(), gm.make_caches()
        tol = TOL_F16 if f16 else TOL_F32
        toks = [int(t) for t in rng.integers(0, vocab, n_prompt)]
        assert max_rel_err(gm.forward(toks, 0, gc), om.forward(toks, 0, oc)) < tol, what
        for i in range(n_dec):
            t = int(rng.integers(0, vocab))
            assert max_rel_err(gm.forward([t], n_prompt + i, gc), om.forward([t], n_prompt + i, oc)) < tol, what
        for l in range(L):
            for which in (0, 1):
                assert max_rel_err(gc.read(l, H - 1, which), oc.read(l, H - 1, which)) < tol, what
        gc.free()
        gm.free()


def test_concurrent_calls_from_threads(ctx):
    """The reference shares its device handle between rayon workers (transformer.rs:52-53, 783-815).  Calls from several
    threads on one context and one model, each thread with caches and tensors of its own, give bit for bit what the same calls
    give one after another."""
    from concurrent.futures import ThreadPoolExecutor
    shape = SMALL
    W = synth_weights(shape, seed=71, std=0.05, norm_ones=False)
    gm = make_gpu(ctx, shape, W, True)
    rng = np.random.default_rng(72)
    jobs = []
    for i in range(12):
        n = int(rng.integers(1, 40))
        jobs.append(([int(t) for t in rng.integers(0, shape.vocab_size, n)], [int(t) for t in rng.integers(0, shape.vocab_size, 4)],
                     oracle.f32_to_f16_bits(rng.uniform(-1, 1, (7 + i, 64)).astype(f32)), oracle.f32_to_f16_bits(rng.uniform(-1, 1, (33, 64)).astype(f32))))

    def run(job):
        prompt, follow, a, b = job
        c = gm.make_caches()
        out = [gm.forward(prompt, 0, c)]
        for i, t in enumerate(follow[:2]):
            out.append(gm.forward([t], len(prompt) + i, c))
        c2 = c.true_clone()
        out.append(np.int32(gm.forward_greedy([follow[2]], len(prompt) + 2, c2)))
        out.append(np.int32(gm.forward_greedy([follow[3]], len(prompt) + 3, c2)))
        out.append(Tensor.from_numpy(ctx, a).matrix_mul_transposed(Tensor.from_numpy(ctx, b)).to_numpy())
        out.append(c.read(shape.n_layers - 1, 1, 0))
        c.free()
        c2.free()
        return out

    serial = [run(j) for j in jobs]
    for _ in range(3):
        with ThreadPoolExecutor(max_workers=6) as ex:
            threaded = list(ex.map(run, jobs))
        for a, b in zip(serial, threaded):
            for x, y in zip(a, b):
                assert np.array_equal(x, y)
    gm.free()


def _make_split_gpu(ctx, shape, W, force_f16, p):
    ds = rllama_amd.DataSettings(ctx).percentage_to_gpu(p)
    if force_f16:
        ds = ds.force_f16()
    m = rllama_amd.Transformer(ctx, shape.dim, shape.n_layers, shape.n_heads, shape.ffn_hidden, shape.vocab_size, shape.max_seq_len,
                               shape.norm_eps, ds)
    last = m.last_layer_on_gpu()
    for (kind, layer), arr in W.items():
        if kind in PER_LAYER or kind in (rllama_amd.ATTN_NORM, rllama_amd.FFN_NORM):
            if layer <= last:
                m.set_tensor(kind, layer, arr)
    return m, last


@pytest.mark.parametrize("force_f16,token_by_token", [(True, False), (True, True), (False, False), (False, True)],
                         ids=["f16-matrix-core", "f16-token-by-token", "f32-matrix-core", "f32-token-by-token"])
def test_hybrid_layer_split(ctx, force_f16, token_by_token):
    """--percentage-to-gpu (transformer.rs:262-279): blocks 0..=last_layer_on_gpu through rlh_forward_layers, the remaining
    blocks, the final norm and the head on the host (here the oracle stands in for the reference's own CPU path).  The stream
    handed over, the device's cache planes and the final logits are compared with the all-host forward, for a prompt call and
    for single-token calls after it."""
    shape = SMALL
    tol = TOL_F16 if force_f16 else TOL_F32
    W = synth_weights(shape, seed=9, std=0.05, norm_ones=False)
    om = make_oracle(shape, W, force_f16)
    toks = [int(t) for t in np.random.default_rng(11).integers(3, shape.vocab_size, 9)]
    follow = [17, 4, 300]
    for p in (0.0, 0.5):
        gm, last = _make_split_gpu(ctx, shape, W, force_f16, p)
        assert last == round(p * (shape.n_layers - 1)) and last < shape.n_layers - 1
        gm.set_prefill_mode(token_by_token)
        gc = gm.make_caches()
        oc_full, oc_tail = om.make_caches(), om.make_caches()
        calls = [(toks, 0)] + [([t], len(toks) + i) for i, t in enumerate(follow)]
        for call_toks, start in calls:
            want, tap = om.forward(call_toks, start, oc_full, layer_tap=True)
            x = gm.forward_layers(om.embed(call_toks), start, gc, 0, last)
            assert max_rel_err(x, tap[last]) < tol, (p, start, max_rel_err(x, tap[last]))
            y = om.forward_layers(x, start, oc_tail, last + 1, shape.n_layers - 1)
            got = om.head(y)
            assert max_rel_err(got, want) < tol, (p, start, max_rel_err(got, want))
        T = len(toks) + len(follow)
        for l in range(last + 1):
            for which in (0, 1):
                a, b = gc.read(l, 1, which), oc_full.read(l, 1, which)
                assert max_rel_err(a[:, :T], b[:, :T]) < tol
                assert not a[:, T:].any()
        # what a split model refuses: whole forwards, tensors and cache planes of host-side layers
        with pytest.raises(rllama_amd.RllamaHipError, match="percentage_to_gpu"):
            gm.forward(toks, 0, gc)
        with pytest.raises(rllama_amd.RllamaHipError, match="percentage_to_gpu"):
            gm.generate_greedy(toks, 2, gc)
        with pytest.raises(rllama_amd.RllamaHipError, match="stays on the host"):
            gm.set_tensor(rllama_amd.WO, last + 1, W[(rllama_amd.WO, last + 1)])
        with pytest.raises(rllama_amd.RllamaHipError, match="stays on the host"):
            gm.forward_layers(om.embed(toks), 0, gc, 0, last + 1)
        with pytest.raises(rllama_amd.RllamaHipError):
            gc.read(last + 1, 0, 0)
        with pytest.raises(rllama_amd.RllamaHipError):
            gm.forward_layers(om.embed(toks), 1, gc, 0, last)       # n > 1 needs start_pos == 0
        gc.free()
        gm.free()


@pytest.mark.parametrize("force_f16", [True, False], ids=["f16", "f32"])
def test_each_layer_alone_against_the_oracle(ctx, force_f16):
    """Config-0 shape, one block at a time: layer l gets the oracle's own stream after layer l - 1 as its input, so every
    block is compared on identical inputs and no difference is carried from layer to layer (prompt call through the
    matrix-core path, then single-token calls through the decode kernels, which read the cache planes the prompt call left)."""
    shape = CONFIG0
    W = synth_weights(shape, seed=0)
    om = make_oracle(shape, W, force_f16)
    gm = make_gpu(ctx, shape, W, force_f16)
    oc, gc = om.make_caches(), gm.make_caches()
    prompt = [int(t) for t in rllama_amd.synth_tokens(0, 16, 3, shape.vocab_size)]
    calls = [(prompt, 0), ([77], 16), ([31000], 17)]
    # one block on identical inputs: only the order of fp32 additions differs, plus in f16 mode the rounding decisions that flips
    tol = 2e-3 if force_f16 else 2e-6
    for toks, start in calls:
        _, tap = om.forward(toks, start, oc, layer_tap=True)
        x_in = om.embed(toks)
        for l in range(shape.n_layers):
            got = gm.forward_layers(x_in, start, gc, l, l)
            err = max_rel_err(got, tap[l])
            assert err < tol, (start, l, err)
            x_in = tap[l]
    T = 18
    for l in (0, shape.n_layers - 1):
        for which in (0, 1):
            a, b = gc.read(l, 3, which)[:, :T], oc.read(l, 3, which)[:, :T]
            # f16 mode: a one-step difference in wk's f16 output passes through the rotation with its pair partner's scale
            bound = 2 * ulp_f16(b) + 1e-3 * np.abs(b).max() if force_f16 else 1e-5 * np.abs(b).max()
            assert np.all(np.abs(a - b) <= bound), (l, which, float(np.abs(a - b).max()))
    gc.free()
    gm.free()


def test_layer_span_on_a_whole_model_equals_its_forward(ctx):
    """On a fully resident model any span runs: two spans back to back give the stream whose norm + head are the logits
    of rlh_forward, and a span over layers that were never set is refused."""
    shape = SMALL
    W = synth_weights(shape, seed=2, std=0.05, norm_ones=False)
    om = make_oracle(shape, W, True)
    gm = make_gpu(ctx, shape, W, True)
    toks = [int(t) for t in np.random.default_rng(5).integers(3, shape.vocab_size, 33)]
    c1, c2 = gm.make_caches(), gm.make_caches()
    want = gm.forward(toks, 0, c1)
    x = gm.forward_layers(om.embed(toks), 0, c2, 0, 0)
    x = gm.forward_layers(x, 0, c2, 1, shape.n_layers - 1)
    got = om.head(x)                                   # final norm + f32 head: the host's part in the reference
    assert max_rel_err(got, want) < 1e-5, max_rel_err(got, want)
    for l in range(shape.n_layers):
        assert np.array_equal(c1.read(l, 0, 0), c2.read(l, 0, 0)) and np.array_equal(c1.read(l, 3, 1), c2.read(l, 3, 1))
    # the caches of a span call continue under the whole forward
    a = gm.forward([9], len(toks), c1)
    b = gm.forward([9], len(toks), c2)
    assert np.array_equal(a, b)
    empty = rllama_amd.Transformer(ctx, shape.dim, shape.n_layers, shape.n_heads, shape.ffn_hidden, shape.vocab_size, shape.max_seq_len,
                                   shape.norm_eps, rllama_amd.DataSettings(ctx).force_f16())
    ce = empty.make_caches()
    with pytest.raises(rllama_amd.RllamaHipError, match="never set"):
        empty.forward_layers(om.embed(toks), 0, ce, 0, 0)
    ce.free()
    empty.free()
    c1.free()
    c2.free()
    gm.free()


# the last four are sized so that the tile choice lands on the 256 x 192, 256 x 256 and 256 x 128 tiles (with ragged edges)
@pytest.mark.parametrize("n,m_rows,k", [(2, 3, 8), (33, 65, 72), (128, 128, 64), (130, 200, 192), (16, 2816, 1024), (257, 384, 4096), (1024, 256, 11008),
                                        (1024, 12288, 64), (1000, 12290, 160), (1024, 16384, 96), (512, 16384, 96)])
@pytest.mark.parametrize("kgroup", ["1", "0"], ids=["k-steps-split", "tile-split"])
def test_mfma_gemm_f16(ctx, n, m_rows, k, kgroup):
    """src [n x k] . other[m x k]^T with n > 1 runs on the matrix cores; every element against the oracle's
    f16-rounded dot8 (tensor.rs:1476-1666), including tiles that straddle the matrix edges.  Products that take 128 x 128
    tiles with k a multiple of 64 run on the kernel whose wavefronts split the K-steps of a tile (four partial sums per
    element, added in a fixed order) unless that is switched off; both forms are checked."""
    rng = np.random.default_rng(n * 7 + m_rows * 3 + k)
    a = oracle.f32_to_f16_bits(rng.uniform(-1, 1, (n, k)).astype(f32))
    b = oracle.f32_to_f16_bits((rng.standard_normal((m_rows, k)) * 0.05).astype(f32))
    with options(ctx, GEMM_KGROUP=kgroup):
        got = Tensor.from_numpy(ctx, a).matrix_mul_transposed(Tensor.from_numpy(ctx, b)).to_numpy().astype(f32)
    want = oracle.f16_bits_to_f32(oracle.matmul_transposed_f16(a, b))
    mag = np.abs(oracle.f16_bits_to_f32(a).astype(np.float64)) @ np.abs(oracle.f16_bits_to_f32(b).astype(np.float64)).T
    close_f16(got, want, mag, f"mfma gemm {n}x{m_rows}x{k}")
    assert np.mean(got != want) < 0.03


@pytest.mark.parametrize("n,m_rows,k", [(2, 40, 32), (130, 200, 96), (300, 129, 512), (1024, 384, 256)])
def test_mfma_gemm_f32(ctx, n, m_rows, k):
    """fp32 src [n x k] . other[m x k]^T with n > 1 and k a multiple of 32 runs on the matrix cores (fp32 products, fp32
    accumulation: only the order of the additions differs from tensor.rs:1282-1475); every element against a float64
    product, with the tolerance the reference's own test uses (1e-5 scaled, tensor.rs:2554-2650), tiles straddling the edges."""
    rng = np.random.default_rng(n * 11 + m_rows * 5 + k)
    a = rng.uniform(-1, 1, (n, k)).astype(f32)
    b = (rng.standard_normal((m_rows, k)) * 0.5).astype(f32)
    got = Tensor.from_numpy(ctx, a).matrix_mul_transposed(Tensor.from_numpy(ctx, b)).to_numpy()
    want64 = a.astype(np.float64) @ b.astype(np.float64).T
    mag = np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64).T
    assert got.shape == (n, m_rows)
    assert np.all(np.abs(got - want64) <= 3e-6 * mag + 1e-30), float(np.max(np.abs(got - want64) / mag))
    if n * m_rows * k <= 130 * 200 * 96:   # and the oracle's own lane-ordered sum on the sizes it finishes quickly
        assert np.allclose(got, oracle.matmul_transposed_f32(a, b), rtol=0, atol=1e-5 * k ** 0.5)


def test_prefill_f32_mode_matrix_core_path(ctx):
    """n > 1 at start_pos 0 in f32 mode (fp32 weights, activations and cache): the fp32 matrix-core prefill against the
    token-by-token path and the oracle's prefill, logits and KV cache; ragged n, several row tiles, decode continues."""
    shape = Shape(dim=256, n_layers=3, n_heads=4, ffn_hidden=704, vocab_size=512, max_seq_len=330)
    W = random_f32_weights(shape, seed=51, std=0.08)
    toks = np.random.default_rng(52).integers(0, shape.vocab_size, 321)
    om, gm = make_oracle(shape, W, False), make_gpu(ctx, shape, W, False)
    for n in (2, 33, 150, 320):
        oc = om.make_caches()
        want = om.forward(toks[:n], 0, oc)
        ga, gb = gm.make_caches(), gm.make_caches()
        gm.set_prefill_mode(False)
        a = gm.forward(toks[:n], 0, ga)
        gm.set_prefill_mode(True)
        b = gm.forward(toks[:n], 0, gb)
        gm.set_prefill_mode(False)
        assert max_rel_err(a, want) < TOL_F32 and max_rel_err(b, want) < TOL_F32, (n, max_rel_err(a, want), max_rel_err(b, want))
        for l in (0, shape.n_layers - 1):
            for which in (0, 1):
                ca, cb, co = ga.read(l, 1, which), gb.read(l, 1, which), oc.read(l, 1, which)
                assert not np.any(ca[:, n:])
                assert np.allclose(ca[:, :n], co[:, :n], rtol=1e-4, atol=1e-5)
                assert np.allclose(cb[:, :n], co[:, :n], rtol=1e-4, atol=1e-5)
        nxt = [int(toks[n])]
        want1 = om.forward(nxt, n, oc)
        assert max_rel_err(gm.forward(nxt, n, ga), want1) < TOL_F32
        assert max_rel_err(gm.forward(nxt, n, gb), want1) < TOL_F32
    gm.free()


def test_prefill_matrix_core_path_against_token_by_token_and_oracle(ctx):
    """n > 1 at start_pos 0 in f16 mode: the matrix-core prefill and the token-by-token path are the same function
    (transformer.rs:343-383); both stay within tolerance of the oracle's prefill, and leave the same KV cache."""
    shape = Shape(dim=256, n_layers=3, n_heads=4, ffn_hidden=704, vocab_size=512, max_seq_len=200)
    W = synth_weights(shape, seed=41, std=0.08, norm_ones=False)
    toks = np.random.default_rng(42).integers(0, shape.vocab_size, 150)
    om, gm = make_oracle(shape, W, True), make_gpu(ctx, shape, W, True)
    for n in (2, 33, 129, 150):
        want = om.forward(toks[:n], 0, om.make_caches())
        ga, gb = gm.make_caches(), gm.make_caches()
        gm.set_prefill_mode(False)
        a = gm.forward(toks[:n], 0, ga)
        gm.set_prefill_mode(True)
        b = gm.forward(toks[:n], 0, gb)
        gm.set_prefill_mode(False)
        assert max_rel_err(a, want) < TOL_F16 and max_rel_err(b, want) < TOL_F16, (n, max_rel_err(a, want), max_rel_err(b, want))
        assert max_rel_err(a, b) < TOL_F16
        for l in (0, shape.n_layers - 1):
            for which in (0, 1):
                ca, cb = ga.read(l, 1, which), gb.read(l, 1, which)
                assert not np.any(ca[:, n:]) and not np.any(cb[:, n:])
                assert np.all(np.abs(ca[:, :n] - cb[:, :n]) <= 2 * ulp_f16(cb[:, :n]) + 2e-3 * np.abs(cb[:, :n]).max())
        # decode continues from a matrix-core prefill exactly as from a token-by-token one
        nxt = int(toks[n % len(toks)])
        assert max_rel_err(gm.forward([nxt], n, ga), gm.forward([nxt], n, gb)) < TOL_F16
    gm.free()


def test_decode_step_graph_replay(ctx):
    """DECODE_GRAPH=1 replays the captured decode step (one graph per attention grid shape): the ids are those of
    the eager loop on every replay, across a change of grid shape, with eager work on other caches between the replays."""
    shape = Shape(dim=256, n_layers=2, n_heads=2, ffn_hidden=512, vocab_size=300, max_seq_len=460)
    W = synth_weights(shape, seed=61, std=0.08, norm_ones=False)
    gm = make_gpu(ctx, shape, W, True)
    prompt = np.random.default_rng(62).integers(0, shape.vocab_size, 376)
    want, _, _ = gm.generate_greedy(prompt, 60, gm.make_caches())
    with options(ctx, DECODE_GRAPH="1"):
        c = gm.make_caches()
        got, _, _ = gm.generate_greedy(prompt, 20, c)           # positions 376 .. 395: the attention grid changes at 384
        assert np.array_equal(got, want[:20])
        for lo in (20, 40):
            other = gm.make_caches()
            gm.forward(prompt[:17], 0, other)                    # eager work between the replays (it drops the greedy state)
            gm.forward([5], 17, other)
            # token want[lo - 1] sits at position 376 + lo - 1; forwarding it again yields want[lo] and re-seeds the greedy state
            assert gm.forward_greedy([int(want[lo - 1])], 376 + lo - 1, c) == want[lo]
            if lo == 40:
                c = c.true_clone()                               # a clone replays its own captures, not its source's
                assert gm.forward_greedy([int(want[lo - 1])], 376 + lo - 1, c) == want[lo]
            ids, _ = gm.decode_greedy(19, c)
            assert np.array_equal(ids, want[lo + 1:lo + 20])
    gm.free()


@pytest.mark.parametrize("force_f16", [True, False], ids=["f16", "f32"])
def test_decode_step_without_launches_for_the_embedding_row_and_the_pick(ctx, force_f16):
    """A greedy decode step reads its embedding row inside layer 0's wq|wk|wv launch and makes its pick inside the output
    head's launch (the last workgroup to finish reduces the workgroups' candidates and advances the token-step state).  With
    DECODE_FOLD=0 both are launches of their own, as they were: same arithmetic on the same values, so the same ids, the same
    logits and the same cache rows bit for bit (as a replayed graph: the same ids), on a vocabulary that does not divide
    into the workgroups evenly and one smaller than the grid."""
    for vocab in (32003, 300):
        shape = Shape(dim=256, n_layers=2, n_heads=2, ffn_hidden=512, vocab_size=vocab, max_seq_len=80)
        W = synth_weights(shape, seed=63, std=0.08, norm_ones=False) if force_f16 else random_f32_weights(shape, 63)
        gm = make_gpu(ctx, shape, W, force_f16)
        prompt = np.random.default_rng(64).integers(0, vocab, 9)
        runs = {}
        for name, opts in (("separate", dict(DECODE_FOLD="0")), ("folded", {}), ("folded-graph", dict(DECODE_GRAPH="1"))):
            with options(ctx, **opts):
                c = gm.make_caches()
                ids, _, _ = gm.generate_greedy(prompt, 40, c)
                more, _ = gm.decode_greedy(20, c)
                last = gm.forward([int(more[-1])], 9 + 40 + 20 - 1, c)   # the logits behind the next pick
                runs[name] = (np.concatenate([ids, more]), last, c.read(1, 1, 0), c.read(1, 1, 1))
        for name in ("folded", "folded-graph"):
            assert np.array_equal(runs[name][0], runs["separate"][0]), (vocab, name)
        for a, b in zip(runs["folded"][1:], runs["separate"][1:]):
            assert np.array_equal(a, b), vocab
        # (a replayed graph keeps the attention kernel's batch size of the step it was captured at, so its fp32 sums may
        # run in another order than the eager loop's at a later position)
        for a, b in zip(runs["folded-graph"][1:], runs["separate"][1:]):
            assert max_rel_err(a, b) < (2e-3 if force_f16 else 2e-6), vocab
        gm.free()


@pytest.mark.parametrize("n_prompt", [200, 1100], ids=["200-tokens", "1100-tokens"])
def test_full_size_7b_properties(ctx, n_prompt):
    """At the full size of the headline configuration (LLaMA-7B shape, f16 mode, synthetic weights) the oracle is out of reach,
    so this checks what holds at any size: the matrix-core prefill and the token-by-token path are the same function (logits
    within the f16-mode tolerance, same greedy continuation), the greedy loop is deterministic, and a true_clone of the caches
    continues exactly like the original."""
    dim, L, H, F, V = 4096, 32, 32, 11008, 32000
    m = rllama_amd.Transformer(ctx, dim, L, H, F, V, n_prompt + 64, 1e-6, rllama_amd.DataSettings(ctx).force_f16())
    m.fill_synthetic(0, 0.02)
    prompt = rllama_amd.synth_tokens(0, n_prompt, 3, V)
    ca, cb = m.make_caches(), m.make_caches()
    a = m.forward(prompt, 0, ca)                       # matrix-core prefill
    m.set_prefill_mode(True)
    b = m.forward(prompt, 0, cb)                       # token by token with the decode kernels
    m.set_prefill_mode(False)
    assert max_rel_err(a, b) < TOL_F16, max_rel_err(a, b)
    assert int(np.argmax(a[1:])) == int(np.argmax(b[1:]))
    for l in (0, L - 1):                               # the caches the two paths leave agree to f16 rounding noise
        for which in (0, 1):
            ka, kb = ca.read(l, 5, which), cb.read(l, 5, which)
            assert not np.any(ka[:, n_prompt:]) and not np.any(kb[:, n_prompt:])
            # layer 0 sees identical inputs; by the last layer 31 layers of f16 rounding decisions have diverged
            slack = 2e-3 if l == 0 else TOL_F16
            assert np.all(np.abs(ka[:, :n_prompt] - kb[:, :n_prompt]) <= 2 * ulp_f16(kb[:, :n_prompt]) + slack * np.abs(kb[:, :n_prompt]).max())
    c1, c2 = m.make_caches(), m.make_caches()
    ids1, _, _ = m.generate_greedy(prompt, 24, c1)
    ids2, _, _ = m.generate_greedy(prompt, 24, c2)
    assert np.array_equal(ids1, ids2)                  # same kernels, same order of additions: bit-identical runs
    c3 = c2.true_clone()
    nxt = int(ids2[-1])
    la = m.forward([nxt], n_prompt + 23, c2)
    lb = m.forward([nxt], n_prompt + 23, c3)
    assert np.array_equal(la, lb)
    m.free()


@pytest.mark.parametrize("force_f16,prompts", [(True, (5, 40, 130, 300, 1024)), (False, (40, 300, 520))], ids=["f16", "f32"])
def test_7b_layer_dimensions_against_the_oracle(ctx, force_f16, prompts):
    """Two layers with the real dimensions of the headline configuration (dim 4096, 32 heads of 128, ffn 11008, vocabulary
    32000, f16 mode): few enough layers for the oracle, and every kernel runs at the row lengths, tile choices and grids it has
    in the 7B model.  Prompts of 5, 40, 130, 300 and 1024 tokens take the 32 x 64, 64 x 64, 128 x 64, 128 x 128 and 256 x 192
    tile paths (the short ones cut along K) and the one-kernel attention at its real head count; single-token calls after each
    prompt run the decode kernels on the cache the prompt call left.  In f32 mode the same dimensions run the fp32 matrix-core
    path: 40 rows on the 64 x 64 tile cut along K, 300 on 128 x 128, 520 on the 128 x 64 tile that only fp32 operands choose."""
    shape = Shape(dim=4096, n_layers=2, n_heads=32, ffn_hidden=11008, vocab_size=32000, max_seq_len=1030)
    W = synth_weights(shape, seed=0)
    if not force_f16:  # the embedding table and the head as fp32 tensors, the way the reference holds them (transformer.rs:302-308)
        for kind in (rllama_amd.TOK_EMB, rllama_amd.OUTPUT):
            W[(kind, 0)] = W[(kind, 0)].view(np.float16).astype(np.float32)
    om = make_oracle(shape, W, force_f16)
    gm = make_gpu(ctx, shape, W, force_f16)
    TOL = TOL_F16 if force_f16 else TOL_F32
    for n_prompt in prompts:
        toks = [int(t) for t in rllama_amd.synth_tokens(n_prompt, n_prompt, 3, shape.vocab_size)]
        oc, gc = om.make_caches(), gm.make_caches()
        print(f"prompt of {n_prompt} tokens", flush=True)
        want, got = om.forward(toks, 0, oc), gm.forward(toks, 0, gc)
        assert max_rel_err(got, want) < TOL, (n_prompt, max_rel_err(got, want))
        top = np.sort(np.where(np.arange(want.size) == 0, 0.0, want))[::-1]                  # the sampler's view: token 0 reads 0.0
        if top[0] - top[1] > 2 * TOL * np.abs(want).max():                               # a clear winner is the same winner
            assert int(np.argmax(got[1:])) == int(np.argmax(want[1:]))
        for i, t in enumerate((17, 31999)):
            want, got = om.forward([t], n_prompt + i, oc), gm.forward([t], n_prompt + i, gc)
            assert max_rel_err(got, want) < TOL, (n_prompt, i, max_rel_err(got, want))
        for l in range(shape.n_layers):
            for which in (0, 1):
                a, b = gc.read(l, 31, which), oc.read(l, 31, which)
                assert max_rel_err(a, b) < TOL, (n_prompt, l, which)
        gc.free()
    gm.free()


@pytest.mark.parametrize("dim,H,F,prompts", [(5120, 40, 13824, (64, 2100)), (8192, 64, 22016, (33, 256))], ids=["13B-dimensions", "65B-dimensions"])
def test_larger_layer_dimensions_against_the_oracle(ctx, dim, H, F, prompts):
    """One layer with the dimensions of the 13B and 65B configurations against the oracle: their tile choices and attention
    grids (40 / 64 heads), and at the 13B dimensions single-token calls at sequence length 2101 and 2102, where the decode
    attention is split into 17 blocks per head and merged, as in the 2048-token-context configuration."""
    shape = Shape(dim=dim, n_layers=1, n_heads=H, ffn_hidden=F, vocab_size=4000, max_seq_len=max(prompts) + 4)
    W = synth_weights(shape, seed=3)
    om = make_oracle(shape, W, True)
    gm = make_gpu(ctx, shape, W, True)
    for n_prompt in prompts:
        toks = [int(t) for t in rllama_amd.synth_tokens(n_prompt, n_prompt, 3, shape.vocab_size)]
        oc, gc = om.make_caches(), gm.make_caches()
        print(f"prompt of {n_prompt} tokens", flush=True)
        want, got = om.forward(toks, 0, oc), gm.forward(toks, 0, gc)
        assert max_rel_err(got, want) < TOL_F16, (n_prompt, max_rel_err(got, want))
        for i, t in enumerate((17, 3999)):
            want, got = om.forward([t], n_prompt + i, oc), gm.forward([t], n_prompt + i, gc)
            assert max_rel_err(got, want) < TOL_F16, (n_prompt, i, max_rel_err(got, want))
        for which in (0, 1):
            assert max_rel_err(gc.read(0, H - 1, which), oc.read(0, H - 1, which)) < TOL_F16, (n_prompt, which)
        gc.free()
    gm.free()


def test_full_size_7b_layer_split(ctx):
    """7B shape split by percentage_to_gpu 0.5 (17 of 32 layers resident): its span calls give bit for bit the stream the same
    span gives on a whole model with the same weights (a prompt call and single-token calls); on the whole model two spans
    back to back, then the final norm and the head in numpy, give the logits of rlh_forward."""
    dim, L, H, F, V, n_prompt = 4096, 32, 32, 11008, 32000, 72
    whole = rllama_amd.Transformer(ctx, dim, L, H, F, V, n_prompt + 8, 1e-6, rllama_amd.DataSettings(ctx).force_f16())
    whole.fill_synthetic(0, 0.02)
    split = rllama_amd.Transformer(ctx, dim, L, H, F, V, n_prompt + 8, 1e-6, rllama_amd.DataSettings(ctx).force_f16().percentage_to_gpu(0.5))
    split.fill_synthetic(0, 0.02)
    last = split.last_layer_on_gpu()
    assert last == 16
    prompt = rllama_amd.synth_tokens(0, n_prompt, 3, V)
    emb = whole.get_tensor(rllama_amd.TOK_EMB, 0, V, dim)
    cw, cs, cf = whole.make_caches(), split.make_caches(), whole.make_caches()
    x = emb[prompt]
    xs = split.forward_layers(x, 0, cs, 0, last)
    xw = whole.forward_layers(x, 0, cw, 0, last)
    assert np.array_equal(xs, xw)
    xw = whole.forward_layers(xw, 0, cw, last + 1, L - 1)
    want = whole.forward(prompt, 0, cf)

    def head(row):
        row = row.astype(np.float64)
        xn = (row / np.sqrt(np.mean(row * row) + 1e-6)).astype(np.float32)          # final norm, weights 1.0
        return whole.get_tensor(rllama_amd.OUTPUT, 0, V, dim) @ xn

    assert max_rel_err(head(xw[-1]), want) < 1e-4
    for step, tok in enumerate((11, 12345)):
        r = emb[[tok]]
        rs = split.forward_layers(r, n_prompt + step, cs, 0, last)
        rw = whole.forward_layers(r, n_prompt + step, cw, 0, last)
        assert np.array_equal(rs, rw)
        rw = whole.forward_layers(rw, n_prompt + step, cw, last + 1, L - 1)
        assert max_rel_err(head(rw[0]), whole.forward([tok], n_prompt + step, cf)) < 1e-4
    assert np.array_equal(cs.read(last, 7, 1), cw.read(last, 7, 1))
    split.free()
    whole.free()


@pytest.mark.parametrize("dim,L,H,F,n_prompt", [(5120, 40, 40, 13824, 300), (8192, 80, 64, 22016, 96)], ids=["13B-shape", "65B-shape"])
def test_full_size_larger_shapes_prefill_equals_token_by_token(ctx, dim, L, H, F, n_prompt):
    """The 13B and 65B shapes of the other configurations (other GEMM tile choices, split factors and attention grids than 7B):
    the matrix-core prefill against the token-by-token path, i.e. two device paths against each other.  How far each may sit
    from the reference at these depths is what test_gpu_fulldepth.py measures against the oracle and its exact-sum form; this
    test adds no tolerance of its own on the logits.  What it checks is what a wrong tile, split or grid would break: the
    difference between the two paths' cache rows grows smoothly with the layer (a mistake shows as a jump at the layer where it
    happens and stays), and both paths pick the same next token where the top-2 gap is larger than their difference."""
    V = 32000
    m = rllama_amd.Transformer(ctx, dim, L, H, F, V, n_prompt + 16, 1e-6, rllama_amd.DataSettings(ctx).force_f16())
    m.fill_synthetic(0, 0.02)
    prompt = rllama_amd.synth_tokens(0, n_prompt, 3, V)
    ca, cb = m.make_caches(), m.make_caches()
    a = m.forward(prompt, 0, ca)
    m.set_prefill_mode(True)
    b = m.forward(prompt, 0, cb)
    m.set_prefill_mode(False)
    noise = {}
    for l in (0, 1, L // 4, L // 2, L - 1):
        for which in (0, 1):
            ka, kb = ca.read(l, 5, which)[:, :n_prompt], cb.read(l, 5, which)[:, :n_prompt]
            noise[(l, which)] = float(np.abs(ka - kb).mean() / np.sqrt((kb.astype(np.float64) ** 2).mean()))
            assert noise[(l, which)] < 2e-3 * (l + 1) ** 0.5, (l, which, noise)
    print(f"logits of the two paths differ by {max_rel_err(a, b):.3e}; cache rows by {noise}")
    assert max_rel_err(a, b) < 0.05                       # sanity only (an unrelated result is O(1) away)
    la, lb = a.copy(), b.copy()
    la[0] = lb[0] = 0.0
    top2 = np.sort(lb)[-2:]
    if top2[1] - top2[0] > 2.0 * float(np.max(np.abs(a - b))):
        assert int(np.argmax(la)) == int(np.argmax(lb))
    m.free()


@pytest.mark.timeout(300)
def test_13b_shape_at_2048_tokens_of_context(ctx):
    """The 13B shape where its configuration operates: a 2048-token prompt, then 8 single-token steps at sequence lengths
    2049 .. 2056 (device-only properties; the comparison with the oracle at this shape is test_gpu_fulldepth.py, 450-token
    prompt).  (i) The split single-query attention gives the same bits whether its pieces are merged inside the kernel or by
    a second launch, (ii) the same greedy ids and logits within fp32 summation noise of the f16 rounding points when the
    sequence is cut into other pieces, (iii) repeated runs are bit-identical, and (iv) the matrix-core prompt pass and the
    token-by-token path agree on the cache rows of the first layers to within rounding flips."""
    dim, L, H, F, V, n_prompt, n_dec = 5120, 40, 40, 13824, 32000, 2048, 8
    m = rllama_amd.Transformer(ctx, dim, L, H, F, V, n_prompt + n_dec + 1, 1e-6, rllama_amd.DataSettings(ctx).force_f16())
    m.fill_synthetic(0, 0.02)
    prompt = rllama_amd.synth_tokens(0, n_prompt, 3, V)
    base = m.make_caches()
    first = m.forward_greedy(prompt, 0, base)

    def steps(**opts):
        with options(ctx, **opts):
            c = base.true_clone()
            logits, tok = [], first
            for i in range(n_dec):
                lg = m.forward([tok], n_prompt + i, c)
                logits.append(lg)
                l2 = lg.copy()
                l2[0] = 0.0
                tok = int(np.argmax(l2))
            planes = (c.read(L - 1, H - 1, 0)[:, n_prompt:n_prompt + n_dec], c.read(L - 1, H - 1, 1)[:, n_prompt:n_prompt + n_dec])
            c.free()
            return logits, planes

    ref, ref_planes = steps()
    again, again_planes = steps()
    for x, y in zip(ref, again):
        assert np.array_equal(x, y)                              # (iii)
    sep, sep_planes = steps(ATTN_MERGE="0")
    for x, y in zip(ref, sep):
        assert np.array_equal(x, y)                              # (i): the same partial results, merged in the same order
    assert np.array_equal(ref_planes[0], sep_planes[0]) and np.array_equal(ref_planes[1], sep_planes[1])
    for chunk in ("128", "96"):
        other, _ = steps(ATTN_CHUNK=chunk)                       # 17 and 22 pieces per head instead of 6
        for i, (x, y) in enumerate(zip(ref, other)):
            # another cut of the sequence changes fp32 sums in front of the f16 rounding of the attention output (a5): flips
            # of single f16 values, 40 layers deep (measured 4.3e-3).  The reference's own arithmetic sits 8e-3 from its
            # exact-sum form at this depth (test_gpu_fulldepth.py).
            assert max_rel_err(x, y) < 8e-3, (chunk, i, max_rel_err(x, y))
    # (iv) prompt pass on the matrix cores against the decode kernels, first layers (differences compound with depth)
    m.set_prefill_mode(True)
    tb = m.make_caches()
    short = 300                                                  # the token-by-token path costs a token step per prompt token
    m.forward(prompt[:short], 0, tb)
    m.set_prefill_mode(False)
    for l in (0, 1):
        for which in (0, 1):
            ka, kb = base.read(l, 7, which)[:, :short], tb.read(l, 7, which)[:, :short]
            assert float(np.abs(ka - kb).mean() / np.sqrt((kb.astype(np.float64) ** 2).mean())) < 2e-3 * (l + 1) ** 0.5, (l, which)
    m.free()


def _checkpoint_tensors(shape, W):
    """The reference's tensor names -> f16 bits, from a weight dict of common.synth_weights (norms rounded to f16)."""
    names = {rllama_amd.TOK_EMB: "tok_embeddings.weight", rllama_amd.NORM: "norm.weight", rllama_amd.OUTPUT: "output.weight"}
    per_layer = {rllama_amd.WQ: "attention.wq", rllama_amd.WK: "attention.wk", rllama_amd.WV: "attention.wv", rllama_amd.WO: "attention.wo",
                 rllama_amd.W1: "feed_forward.w1", rllama_amd.W2: "feed_forward.w2", rllama_amd.W3: "feed_forward.w3",
                 rllama_amd.ATTN_NORM: "attention_norm", rllama_amd.FFN_NORM: "ffn_norm"}
    T, W16 = {}, {}
    for (kind, layer), arr in W.items():
        bits = arr if arr.dtype == np.uint16 else arr.astype(np.float16).view(np.uint16)
        W16[(kind, layer)] = bits
        name = names[kind] if kind in names else f"layers.{layer}.{per_layer[kind]}.weight"
        T[name] = bits.reshape(-1) if "norm" in name else bits
    return T, W16


@pytest.mark.parametrize("shards", [1, 2])
def test_model_loaded_from_checkpoint_directory(ctx, tmp_path, shards):
    """params.json + consolidated.NN (src/data_source.rs:166-210) -> device model: the loader hands over exactly the bits
    of the files, so logits equal those of a model filled tensor by tensor; the C++ host loader generates the same ids."""
    import subprocess
    from rllama_amd import build, checkpoint
    shape = SMALL
    T, W16 = _checkpoint_tensors(shape, synth_weights(shape, seed=51, std=0.08, norm_ones=False))
    path = str(tmp_path / "model")
    checkpoint.write_checkpoint(path, {"dim": shape.dim, "multiple_of": 32, "n_heads": shape.n_heads, "n_layers": shape.n_layers,
                                       "norm_eps": shape.norm_eps, "vocab_size": shape.vocab_size}, T, n_shards=shards)
    ds = rllama_amd.DataSettings(ctx).force_f16()
    loaded = checkpoint.load_transformer(ctx, path, ds, shape.max_seq_len)
    direct = make_gpu(ctx, shape, W16, True)
    n_prompt, n_new = 9, 12
    prompt = rllama_amd.synth_tokens(0, n_prompt, 3, shape.vocab_size)
    a = loaded.forward(prompt, 0, loaded.make_caches())
    b = direct.forward(prompt, 0, direct.make_caches())
    assert np.array_equal(a, b)
    want_ids, _, _ = direct.generate_greedy(prompt, n_new, direct.make_caches())
    # the same directory under a layer split: only the device's layers are loaded, and they run as a span
    part = checkpoint.load_transformer(ctx, path, rllama_amd.DataSettings(ctx).force_f16().percentage_to_gpu(0.5), shape.max_seq_len)
    last = part.last_layer_on_gpu()
    assert last == 1 and shape.n_layers == 3
    x = W16[(rllama_amd.TOK_EMB, 0)].view(np.float16).astype(np.float32)[prompt]
    assert np.array_equal(part.forward_layers(x, 0, part.make_caches(), 0, last), direct.forward_layers(x, 0, direct.make_caches(), 0, last))
    part.free()
    loaded.free()
    direct.free()
    r = subprocess.run([build.build_host(), "--model-path", path, str(n_prompt), str(n_new), "0"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    line = [ln for ln in r.stdout.splitlines() if ln.startswith("tokens:")][0]
    assert [int(t) for t in line.split()[1:]] == [int(t) for t in want_ids]


def test_forward_sample(ctx):
    """rlh_forward_sample = forward + TokenSampler::sample (src/rllama_main.rs:846-860): with top_k 1 it is the device argmax,
    otherwise the host sampler on the downloaded logits; both agree with the oracle sampler run on these logits."""
    shape = SMALL
    W = synth_weights(shape, seed=61, std=0.08, norm_ones=False)
    gm = make_gpu(ctx, shape, W, True)
    toks = np.random.default_rng(62).integers(0, shape.vocab_size, 7)

    class _U:
        def __init__(self, u):
            self.u = u

        def random(self, dtype=None):
            return np.float32(self.u)

    logits = gm.forward(toks, 0, gm.make_caches())
    greedy = gm.forward_greedy(toks, 0, gm.make_caches())
    for ts in (rllama_amd.TokenSampler(), rllama_amd.TokenSampler().temperature(3.0).repetition_penalty(1.0)):
        tok, prob = gm.forward_sample(toks, 0, gm.make_caches(), ts, toks, _U(0.4))
        oi, op, ot = oracle.sample_candidates(logits, ts.get_temperature(), ts.get_top_p(), ts.get_top_k(), ts.get_repetition_penalty(), toks)
        assert tok == greedy == oi[0] and prob == 1.0
    ts = rllama_amd.TokenSampler().temperature(1.5).top_k(8).top_p(0.9).repetition_penalty(1.2)
    for u in (0.0, 0.35, 0.8, 1.0):
        tok, prob = gm.forward_sample(toks, 0, gm.make_caches(), ts, toks, _U(u))
        oi, op, ot = oracle.sample_candidates(logits, 1.5, 0.9, 8, 1.2, toks)
        assert (tok, prob) == oracle.sample_pick(oi, op, ot, u)
    gm.free()


def test_against_committed_oracle_fixtures(ctx):
    """The committed outputs of the oracle (tests/golden/*.json; no oracle run here): config 0's 64 greedy ids identical,
    its sampled logits and the tiny shapes' full logits within the f16 / f32 tolerances."""
    import json
    import os
    gold = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    fx = json.load(open(os.path.join(gold, "config0_oracle.json")))
    bits = lambda b: np.array(b, dtype=np.uint32).view(np.float32)  # noqa: E731
    gm = make_gpu(ctx, CONFIG0, synth_weights(CONFIG0, seed=fx["seed"], std=fx["std"]), True)
    ids, _, _ = gm.generate_greedy(fx["prompt_ids"], 64, gm.make_caches())
    assert ids.tolist() == fx["greedy_ids"]
    gc, toks, prev = gm.make_caches(), list(fx["prompt_ids"]), 0
    for step in range(64):
        lg = gm.forward(toks[prev:], prev, gc)
        want = bits(fx["sample_logits_f32_bits"][step])
        assert np.max(np.abs(lg[fx["sample_token_ids"]] - want)) <= TOL_F16 * np.max(np.abs(want)), step
        toks.append(fx["greedy_ids"][step])
        prev = len(toks) - 1
    gm.free()
    tiny = json.load(open(os.path.join(gold, "tiny_oracle.json")))
    for mode, W, f16, tol in (("f16", synth_weights(TINY, seed=21, std=0.08, norm_ones=False), True, TOL_F16),
                              ("f32", random_f32_weights(TINY, seed=23, std=0.08), False, TOL_F32)):
        gm = make_gpu(ctx, TINY, W, f16)
        gc = gm.make_caches()
        t = tiny[mode]["tokens"]
        assert max_rel_err(gm.forward(t[:7], 0, gc), bits(tiny[mode]["logits_after_7_f32_bits"])) < tol
        assert max_rel_err(gm.forward(t[7:8], 7, gc), bits(tiny[mode]["logits_after_8_f32_bits"])) < tol
        gm.free()
