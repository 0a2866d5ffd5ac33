"""Op-level parity of the kernels the reference runs on its host path: single-query attention, the prompt's causal
attention, RoPE + cache write, the residual add, the FFN gate and the greedy pick -- each on crafted inputs against the
oracle's restatement of the reference ops it replaces (through the C ABI).

Attention on one head, as the reference does it for one token (src/transformer.rs:762-781): scores =
vector_matrix_mul(q, K) * (1 / sqrt(hd)) (src/tensor.rs:1923-1983), softmax without a maximum subtracted (:479-494),
out[j] = dot8(p, V[j, :]) (:1282-1475).
"""
import numpy as np
import pytest

import oracle
import rllama_amd
from rllama_amd import Tensor, TensorDType
from common import options

pytestmark = pytest.mark.gpu
f32 = np.float32


def _oracle_attn_decode(q, K, V, T, hd):
    """q [H x hd] f32; K, V [H x max_seq x hd] f32 (values as the cache holds them) -> [H x hd] f32 and the scores."""
    H = q.shape[0]
    out = np.zeros((H, hd), f32)
    smax = -np.inf
    for h in range(H):
        keys = np.ascontiguousarray(K[h, :T].T)                       # the reference's [hd x T] view of the cache
        s = oracle.vector_matrix_mul_f32(q[h:h + 1], keys) * f32(1.0 / np.sqrt(f32(hd)))
        smax = max(smax, float(s.max()))
        p = oracle.softmax_row(s)
        vals = np.ascontiguousarray(V[h, :T].T)                       # [hd x T]
        for j in range(hd):
            out[h, j] = oracle.dot8_f32(p, vals[j])
    return out, smax


def _planes(ctx, K, V, f16):
    H, S, hd = K.shape
    if f16:
        return (Tensor.from_numpy(ctx, K.reshape(H * S, hd).astype(np.float16)), Tensor.from_numpy(ctx, V.reshape(H * S, hd).astype(np.float16)))
    return Tensor.from_numpy(ctx, K.reshape(H * S, hd)), Tensor.from_numpy(ctx, V.reshape(H * S, hd))


@pytest.mark.parametrize("hd,H,f16", [(128, 3, True), (64, 5, True), (128, 2, False), (32, 4, True), (16, 6, False)])
def test_attn_decode_against_the_reference_ops(ctx, hd, H, f16):
    """Every sequence length around the edges of the block's chunking (16-position rounding, one / several steps of the
    loop, 2 / 4 / 8 rows in flight) and every way of splitting it, against the oracle's ops on the same cache contents."""
    rng = np.random.default_rng(hd * 7 + H)
    S = 1100
    K = (rng.standard_normal((H, S, hd)) * 0.7).astype(f32)
    V = rng.standard_normal((H, S, hd)).astype(f32)
    if f16:
        K, V = K.astype(np.float16).astype(f32), V.astype(np.float16).astype(f32)
    q = rng.standard_normal((H, hd)).astype(f32)
    ck, cv = _planes(ctx, K, V, f16)
    Q = Tensor.from_numpy(ctx, q.reshape(1, -1))
    per_step = 8 * 512 // hd
    Ts = sorted({1, 2, 15, 16, 17, 31, 33, per_step - 1, per_step, per_step + 1, 2 * per_step, 2 * per_step + 1, 4 * per_step + 3,
                 8 * per_step, 8 * per_step + 1, 383, 384, 385, 513, 1024, 1100} & set(range(1, S + 1)))
    worst = 0.0
    for T in Ts:
        want, _ = _oracle_attn_decode(q, K, V, T, hd)
        for n_splits in (0, 1, 2, 3, 7, 16, 64):
            if n_splits > 1 and T < 4:
                continue
            got = Q.attn_decode(ck, cv, H, S, T, n_splits=n_splits).to_numpy().reshape(H, hd)
            err = float(np.max(np.abs(got - want)) / np.max(np.abs(want)))
            worst = max(worst, err)
            assert err < 2e-6, (T, n_splits, err)
    # the rounding point before wo (src/transformer.rs:793-796): the same values rounded to f16
    got = Q.attn_decode(ck, cv, H, S, 700, n_splits=0, round_out=True).to_numpy().reshape(H, hd)
    plain = Q.attn_decode(ck, cv, H, S, 700, n_splits=0).to_numpy().reshape(H, hd)
    assert np.array_equal(got, plain.astype(np.float16).astype(f32))
    print(f"attn_decode hd {hd}: worst relative error {worst:.2e}")


def test_attn_decode_repeats_bit_for_bit(ctx):
    """The merge of a split sequence runs in split order whichever block finishes last: repeated calls agree bit for bit."""
    rng = np.random.default_rng(3)
    H, hd, S, T = 8, 128, 2304, 2111
    K = rng.standard_normal((H, S, hd)).astype(np.float16).astype(f32)
    V = rng.standard_normal((H, S, hd)).astype(np.float16).astype(f32)
    ck, cv = _planes(ctx, K, V, True)
    Q = Tensor.from_numpy(ctx, rng.standard_normal((1, H * hd)).astype(f32))
    first = Q.attn_decode(ck, cv, H, S, T, n_splits=17).to_numpy()
    for _ in range(20):
        assert np.array_equal(Q.attn_decode(ck, cv, H, S, T, n_splits=17).to_numpy(), first)


def test_attn_decode_where_the_reference_overflows(ctx):
    """Scores above ln(FLT_MAX) = 88.72: the reference's exp(s) is inf and its probabilities NaN (src/tensor.rs:479-494, pinned
    here on the oracle); the kernel subtracts the running maximum and returns the finite softmax -- the documented
    divergence -- which is checked against a float64 softmax."""
    rng = np.random.default_rng(11)
    H, hd, S, T = 2, 64, 96, 80
    K = rng.standard_normal((H, S, hd)).astype(np.float16).astype(f32)
    V = rng.standard_normal((H, S, hd)).astype(np.float16).astype(f32)
    q = (rng.standard_normal((H, hd)) * 40.0).astype(f32)             # |score| reaches several hundred
    want_ref, smax = _oracle_attn_decode(q, K, V, T, hd)
    assert smax > 89.0 and np.isnan(want_ref).any(), "the crafted scores must overflow the reference's softmax"
    ck, cv = _planes(ctx, K, V, True)
    got = Tensor.from_numpy(ctx, q.reshape(1, -1)).attn_decode(ck, cv, H, S, T, n_splits=3).to_numpy().reshape(H, hd)
    assert np.isfinite(got).all()
    s = np.einsum("hd,htd->ht", q.astype(np.float64), K[:, :T].astype(np.float64)) / np.sqrt(hd)
    p = np.exp(s - s.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    want = np.einsum("ht,htd->hd", p, V[:, :T].astype(np.float64))
    assert np.max(np.abs(got - want)) < 1e-4 * np.max(np.abs(want))
    # and just below the overflow both agree
    q2 = (q * (80.0 / smax)).astype(f32)
    want2, smax2 = _oracle_attn_decode(q2, K, V, T, hd)
    assert smax2 < 88.0 and np.isfinite(want2).all()
    got2 = Tensor.from_numpy(ctx, q2.reshape(1, -1)).attn_decode(ck, cv, H, S, T, n_splits=2).to_numpy().reshape(H, hd)
    assert np.max(np.abs(got2 - want2)) < 1e-5 * np.max(np.abs(want2))


def test_attn_decode_rejects_what_does_not_fit(ctx):
    H, hd, S = 2, 64, 32
    z = Tensor.zeros(ctx, H * S, hd, TensorDType.Float16)
    q = Tensor.zeros(ctx, 1, H * hd, TensorDType.Float32)
    for bad in (dict(T=0), dict(T=S + 1), dict(T=4, n_splits=65), dict(T=4, n_splits=-1)):
        with pytest.raises(rllama_amd.RllamaHipError):
            q.attn_decode(z, z, H, S, **bad)
    with pytest.raises(rllama_amd.RllamaHipError):
        q.attn_decode(z, Tensor.zeros(ctx, H * S, hd, TensorDType.Float32), H, S, 4)     # planes of two dtypes
    with pytest.raises(rllama_amd.RllamaHipError):
        Tensor.zeros(ctx, 1, H * hd + 8, TensorDType.Float32).attn_decode(z, z, H, S, 4)  # q of another size
    with pytest.raises(rllama_amd.RllamaHipError):
        q.attn_decode(Tensor.zeros(ctx, H * S, 48, TensorDType.Float16), Tensor.zeros(ctx, H * S, 48, TensorDType.Float16), H, S, 4)  # head_dim 48


@pytest.mark.parametrize("f16", [True, False])
def test_rope_kvwrite_against_the_oracle(ctx, f16):
    """RoPE bit-exact with the oracle's apply_rotary_emb (no FMA, f64 table cast to f32), cache rows = f16r of the rotated k
    and of v, other positions untouched."""
    rng = np.random.default_rng(21)
    H, hd, S = 4, 64, 40
    fc = oracle.freqs_cis(hd, S)
    dt = TensorDType.Float16 if f16 else TensorDType.Float32
    ck, cv = Tensor.zeros(ctx, H * S, hd, dt), Tensor.zeros(ctx, H * S, hd, dt)
    wantK = np.zeros((H, S, hd), f32)
    wantV = np.zeros((H, S, hd), f32)
    for pos in (0, 1, 7, 39):
        q, k, v = (rng.standard_normal((1, H * hd)).astype(f32) for _ in range(3))
        Q = Tensor.from_numpy(ctx, q)
        Q.rope_kvwrite(Tensor.from_numpy(ctx, k), Tensor.from_numpy(ctx, v), ck, cv, H, S, pos)
        assert np.array_equal(Q.to_numpy()[0], oracle.rope_row(q, H, hd, fc[pos]))
        kr = oracle.rope_row(k, H, hd, fc[pos]).reshape(H, hd)
        wantK[:, pos] = oracle.f16r(kr) if f16 else kr
        wantV[:, pos] = oracle.f16r(v.reshape(H, hd)) if f16 else v.reshape(H, hd)
    assert np.array_equal(ck.to_numpy().astype(f32).reshape(H, S, hd), wantK)
    assert np.array_equal(cv.to_numpy().astype(f32).reshape(H, S, hd), wantV)
    with pytest.raises(rllama_amd.RllamaHipError):
        Tensor.zeros(ctx, 1, H * hd, TensorDType.Float32).rope_kvwrite(Tensor.zeros(ctx, 1, H * hd, TensorDType.Float32),
                                                                       Tensor.zeros(ctx, 1, H * hd, TensorDType.Float32), ck, cv, H, S, S)


def test_add_and_silu_mul(ctx):
    rng = np.random.default_rng(8)
    a = rng.standard_normal((3, 1000)).astype(f32)
    b = rng.standard_normal((3, 1000)).astype(f32)
    assert np.array_equal(Tensor.from_numpy(ctx, a).add(Tensor.from_numpy(ctx, b)).to_numpy(), a + b)    # src/tensor.rs:573-593
    # f32: (g / (1 + exp(-g))) * u, each step rounded to f32 (src/tensor.rs:826-827, 729); the device's expf may differ from
    # the host's in the last place
    silu = np.array([oracle.silu(float(x)) for x in a.ravel()], f32).reshape(a.shape)
    got = Tensor.from_numpy(ctx, a).silu_mul(Tensor.from_numpy(ctx, b)).to_numpy()
    assert np.allclose(got, silu * b, rtol=3e-7, atol=1e-9)
    # f16 tensors: inputs are f16 values, one rounding of the f32 product (src/transformer.rs:557-565)
    ah, bh = a.astype(np.float16), b.astype(np.float16)
    silu_h = np.array([oracle.silu(float(x)) for x in ah.astype(f32).ravel()], f32).reshape(a.shape)
    want = (silu_h * bh.astype(f32)).astype(np.float16)
    got = Tensor.from_numpy(ctx, ah).silu_mul(Tensor.from_numpy(ctx, bh)).to_numpy()
    assert np.mean(got != want) < 2e-3 and np.all(np.abs(got.astype(f32) - want.astype(f32)) <= np.spacing(np.abs(want)).astype(f32))
    with pytest.raises(rllama_amd.RllamaHipError):
        Tensor.from_numpy(ctx, ah).add(Tensor.from_numpy(ctx, bh))                                   # the residual stream is f32


@pytest.mark.parametrize("n,m,k", [(300, 1000, 256), (256, 192, 64), (70, 520, 128), (513, 392, 192), (8, 264, 256), (100, 136, 192)])
def test_ffn_gate_against_the_reference_ops(ctx, n, m, k):
    """FeedForward up to its gate for n rows (src/transformer.rs:551-565): the oracle's f16 matmul (src/tensor.rs:1282-1475,
    result rounded to f16), silu and hadamard product in f32, one rounding to f16.  The matrix cores add the k products in
    another order than the reference's lanes, so a product near an f16 rounding boundary may land on the neighbouring value:
    at most one f16 step, on few elements.  The one-pass form (forced) and the two-product form give the same bits."""
    import os
    rng = np.random.default_rng(n + m + k)
    x = (rng.standard_normal((n, k)) * 0.5).astype(np.float16)
    w1 = (rng.standard_normal((m, k)) * 0.1).astype(np.float16)
    w3 = (rng.standard_normal((m, k)) * 0.1).astype(np.float16)
    g = oracle.matmul_transposed_f16(x.view(np.uint16), w1.view(np.uint16)).view(np.float16).astype(f32)
    u = oracle.matmul_transposed_f16(x.view(np.uint16), w3.view(np.uint16)).view(np.float16).astype(f32)
    silu = np.array([oracle.silu(float(v)) for v in g.ravel()], f32).reshape(g.shape)
    want = (silu * u).astype(np.float16)
    X, W1, W3 = Tensor.from_numpy(ctx, x), Tensor.from_numpy(ctx, w1), Tensor.from_numpy(ctx, w3)
    got = {}
    for mode in ("1", "2", "3", "4", "5", "0"):  # five shapes of the one-pass workgroup, two launches
        # (GEMM_KGROUP=0: the two-launch form on the kernel whose sum over k runs in the one-pass kernel's order)
        with options(ctx, GEMM_KGROUP="0", GEMM_DUAL=mode):
            got[mode] = X.ffn_gate(W1, W3).to_numpy()
    assert np.array_equal(got["1"].view(np.uint16), got["0"].view(np.uint16))
    for mode in ("2", "3", "4", "5"):
        assert np.array_equal(got[mode].view(np.uint16), got["0"].view(np.uint16)), mode
    one = got["1"]
    step = np.spacing(np.maximum(np.abs(want), np.abs(one))).astype(f32)
    assert np.mean(one != want) < 2e-2 and np.all(np.abs(one.astype(f32) - want.astype(f32)) <= 2 * step)
    with pytest.raises(rllama_amd.RllamaHipError):
        X.ffn_gate(W1, Tensor.from_numpy(ctx, w3[:-1]))                                              # w1 and w3 of two shapes
    with pytest.raises(rllama_amd.RllamaHipError):
        Tensor.from_numpy(ctx, x.astype(f32)).ffn_gate(W1, W3)                                       # f16 mode only


def test_ffn_gate_whole_rounds_in_one_pass_and_the_rest_in_two_launches(ctx):
    """2048 rows x 13824 columns are 576 workgroups of the one-pass form, 2.25 rounds of the 256 compute units: the pass takes
    the 12288 columns that make two whole rounds and the last 1536 go through w1's product and w3's with the gate epilogue
    (src/transformer.rs:551-565 either way).  Against the two-launch form over all columns (a few f16 steps apart on few
    elements: the remaining columns add their k products in another order, and a gate or product that lands on the neighbouring
    f16 value moves the result by up to its own relative step each) and, on a sample, against float64."""
    import os
    n, m, k = 2048, 13824, 1024
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((n, k)) * 0.5).astype(np.float16)
    w1 = (rng.standard_normal((m, k)) * 0.05).astype(np.float16)
    w3 = (rng.standard_normal((m, k)) * 0.05).astype(np.float16)
    X, W1, W3 = Tensor.from_numpy(ctx, x), Tensor.from_numpy(ctx, w1), Tensor.from_numpy(ctx, w3)
    got = X.ffn_gate(W1, W3).to_numpy()
    with options(ctx, GEMM_DUAL="0"):
        two = X.ffn_gate(W1, W3).to_numpy()
    step = np.spacing(np.maximum(np.abs(got), np.abs(two))).astype(f32)
    assert np.array_equal(got[:, :12288], two[:, :12288])   # the pass: the two-launch form's order of additions
    assert np.mean(got[:, 12288:] != two[:, 12288:]) < 5e-3 and np.all(np.abs(got.astype(f32) - two.astype(f32)) <= 8 * step)
    rows = rng.integers(0, n, 600)
    cols = np.concatenate([rng.integers(0, 12288, 300), rng.integers(12288, m, 300)])  # both sides of the cut
    xs, a, b = x[rows].astype(np.float64), w1[cols].astype(np.float64), w3[cols].astype(np.float64)
    g = np.einsum("ik,ik->i", xs, a).astype(np.float16).astype(np.float64)
    u = np.einsum("ik,ik->i", xs, b).astype(np.float16).astype(np.float64)
    want = (g / (1.0 + np.exp(-g)) * u)
    have = got[rows, cols].astype(np.float64)
    assert np.all(np.abs(have - want) <= 4e-3 * np.abs(want) + 1e-4), float(np.max(np.abs(have - want)))


@pytest.mark.parametrize("hd,H,n", [(128, 2, 200), (64, 3, 65), (128, 1, 64), (64, 2, 1), (128, 2, 333)])
def test_attn_prefill_against_the_reference_ops(ctx, hd, H, n):
    """The prompt's attention block between the projections and wo against the oracle's restatement of
    src/transformer.rs:704-796: RoPE, f16 cache rows, per row scores by the sequential-k product (src/tensor.rs:1050-1115),
    mask, softmax, P.V by dot8, heads concatenated and rounded to f16.  Ragged query / key tiles included."""
    rng = np.random.default_rng(hd + H * 13 + n)
    d, S = H * hd, 352
    qkv = (rng.standard_normal((n, 3 * d)) * 0.8).astype(np.float16)
    ck, cv = Tensor.zeros(ctx, H * S, hd, TensorDType.Float16), Tensor.zeros(ctx, H * S, hd, TensorDType.Float16)
    got = Tensor.from_numpy(ctx, qkv).attn_prefill(ck, cv, H, S).to_numpy().astype(f32)
    fc = oracle.freqs_cis(hd, S)
    q32, k32, v32 = (qkv[:, i * d:(i + 1) * d].astype(f32) for i in range(3))
    qr = np.stack([oracle.rope_row(q32[i:i + 1], H, hd, fc[i]) for i in range(n)]).reshape(n, H, hd)
    kr = oracle.f16r(np.stack([oracle.rope_row(k32[i:i + 1], H, hd, fc[i]) for i in range(n)])).reshape(n, H, hd)
    vr = v32.reshape(n, H, hd)                                        # already f16 values
    # the cache planes hold the rotated, rounded k and v rows
    assert np.array_equal(ck.to_numpy().astype(f32).reshape(H, S, hd)[:, :n], kr.transpose(1, 0, 2))
    assert np.array_equal(cv.to_numpy().astype(f32).reshape(H, S, hd)[:, :n], vr.transpose(1, 0, 2))
    want = np.zeros((n, H, hd), f32)
    scale = f32(1.0 / np.sqrt(f32(hd)))
    for h in range(H):
        keys = np.ascontiguousarray(kr[:, h].T)                       # [hd x n]
        sc = oracle.matmul_f32_seqk(np.ascontiguousarray(qr[:, h]), keys) * scale      # [n x n]
        vals = np.ascontiguousarray(vr[:, h].T)                       # [hd x n]
        for r in range(n):
            s = sc[r].copy()
            s[r + 1:] = -np.inf                                       # full_triu mask (src/tensor.rs:496-508)
            p = oracle.softmax_row(s)
            for j in range(hd):
                want[r, h, j] = oracle.dot8_f32(p, vals[j])
    want = want.reshape(n, d)
    scale_out = np.abs(want).max()
    # q and the probabilities travel as hi + lo f16 halves through the matrix cores: the difference from the fp32 ops is the
    # order of fp32 additions plus 2^-22 relative per operand, then one f16 rounding of the output
    tol = np.abs(want) * 2.0 ** -10 + 2e-5 * scale_out
    assert np.all(np.abs(got - want) <= tol), float(np.max(np.abs(got - want) / scale_out))


def _greedy_cases():
    V = 1000
    rng = np.random.default_rng(0)
    base = (rng.standard_normal(V) * 3.0).astype(f32)
    cases = {}
    cases["plain"] = base.copy()
    c = base.copy(); c[0] = 50.0; cases["token0_largest_logit_is_shifted_to_zero"] = c          # the quirk bites: 0 must NOT win
    c = -np.abs(base) - 1.0; c[0] = -7.0; cases["token0_wins_when_all_others_negative"] = c      # 0 - 0 = 0 is the largest
    c = base.copy(); c[[17, 400, 999]] = 9.5; cases["exact_tie_lowest_id"] = c
    c = base.copy(); c[123] = np.nan; cases["one_nan_poisons_the_sum"] = c
    c = base.copy(); c[0] = np.nan; cases["token0_nan"] = c
    c = base.copy(); c[0] = np.inf; cases["token0_inf_minus_inf"] = c
    c = base.copy(); c[77] = 89.0; cases["one_logit_overflows_exp"] = c
    c = base.copy(); c[77] = 88.7; cases["just_below_the_overflow"] = c
    c = base.copy(); c[5] = np.inf; cases["plus_inf"] = c
    c = base.copy(); c[5] = -np.inf; cases["minus_inf_is_harmless"] = c
    c = np.full(V, 85.0, f32); c[300] = 86.0; cases["sum_overflows_without_any_term_overflowing"] = c
    c = np.full(V, 80.0, f32); c[300] = 81.5; cases["large_but_finite_sum"] = c
    c = np.full(V, np.nan, f32); cases["all_nan"] = c
    return cases


@pytest.mark.parametrize("name", sorted(_greedy_cases()))
@pytest.mark.parametrize("temperature", [1.0, 0.2])
def test_device_greedy_pick_on_crafted_logits(ctx, name, temperature):
    """The device pick (the kernel every greedy entry point ends with) against the oracle's TokenSampler::sample at top_k 1
    (src/token_sampler.rs:99-147) and against the library's host sampler, on the cases where an arg-max of the logits and the
    reference's sort of un-stabilised softmax probabilities part ways."""
    logits = _greedy_cases()[name]
    want, _, ties = oracle.sample_greedy(logits, temperature)
    got = Tensor.from_numpy(ctx, logits.reshape(1, -1)).argmax_greedy(temperature)
    assert got == want, (name, temperature, got, want, ties)
    sampler = rllama_amd.TokenSampler().temperature(temperature).top_k(1).top_p(1.0).repetition_penalty(1.0)
    host, _ = sampler.sample(logits, [], np.random.default_rng(0))
    assert host == want, (name, temperature, host, want)


@pytest.mark.parametrize("name", sorted(_greedy_cases()))
def test_greedy_pick_inside_the_output_head_on_crafted_logits(ctx, name):
    """The pick that a decode step makes inside the output head's launch, on the same crafted cases: a one-layer f32-mode model
    whose wo and w2 are zero and whose embedding rows all hold one non-zero element, so that every step's logits are
    W_out[:, 0] times one constant -- the crafted values.  The second id of a greedy run comes from a decode step; it must
    be what the oracle's sampler picks on the logits the device itself returns."""
    from rllama_amd import ATTN_NORM, FFN_NORM, NORM, OUTPUT, TOK_EMB, W1, W2, W3, WK, WO, WQ, WV
    logits = _greedy_cases()[name]
    V, d, F = logits.size, 64, 64
    gm = rllama_amd.Transformer(ctx, d, 1, 2, F, V, 8, 1e-6, rllama_amd.DataSettings(ctx))
    rng = np.random.default_rng(3)
    emb = np.zeros((V, d), f32)
    emb[:, 0] = 8.0                                         # mean(x^2) = 1: the final norm leaves 8 / sqrt(1 + eps) in element 0
    xn0 = f32(8.0) * (f32(1.0) / np.sqrt(f32(1.0) + f32(1e-6)))
    out = np.zeros((V, d), f32)
    with np.errstate(invalid="ignore", over="ignore"):
        out[:, 0] = logits / xn0
    gm.set_tensor(TOK_EMB, 0, emb)
    gm.set_tensor(OUTPUT, 0, out)
    gm.set_tensor(NORM, 0, np.ones((1, d), f32))
    for kind, shape in ((WQ, (d, d)), (WK, (d, d)), (WV, (d, d)), (W1, (F, d)), (W3, (F, d))):
        gm.set_tensor(kind, 0, (rng.standard_normal(shape) * 0.1).astype(f32))
    gm.set_tensor(WO, 0, np.zeros((d, d), f32))
    gm.set_tensor(W2, 0, np.zeros((d, F), f32))
    for kind in (ATTN_NORM, FFN_NORM):
        gm.set_tensor(kind, 0, np.ones((1, d), f32))
    have = gm.forward([5], 0, gm.make_caches())
    finite = np.isfinite(logits)
    assert np.allclose(have[finite], logits[finite], rtol=1e-6, atol=1e-6) and np.array_equal(np.isnan(have), np.isnan(logits))
    want, _, _ = oracle.sample_greedy(have, 1.0)
    ids, _, _ = gm.generate_greedy([5], 3, gm.make_caches())
    assert ids.tolist() == [want, want, want], (name, ids.tolist(), want)   # the prompt pass's pick, then two decode steps
    with options(ctx, DECODE_FOLD="0"):
        ids2, _, _ = gm.generate_greedy([5], 3, gm.make_caches())
    assert ids2.tolist() == ids.tolist()
    gm.free()


def test_device_greedy_pick_full_vocab_and_odd_sizes(ctx):
    rng = np.random.default_rng(5)
    for V in (32000, 31999, 7, 1):
        for _ in range(3):
            logits = (rng.standard_normal(V) * 4.0).astype(f32)
            want, _, _ = oracle.sample_greedy(logits, 1.0)
            assert Tensor.from_numpy(ctx, logits.reshape(-1, 1)).argmax_greedy() == want


def test_gemv_phase_probe_reads_a_consistent_clock(ctx):
    """rlh_probe_gemv_phases (measurement only): the wall-clock readings inside the kernel are ordered as the kernel runs --
    every phase non-negative and shorter than the launch it belongs to, the launch as the device sees it no longer than what
    HIP events measure around it plus the gap in front -- and bad arguments are refused."""
    rows, k = 2048, 4096
    r = ctx.probe_gemv_phases(rows, k, n_buffers=4, launches=16)
    assert set(r) == set(rllama_amd.Context.GEMV_PHASES) and all(np.isfinite(v) and v >= 0.0 for v in r.values()), r
    whole = r["first_entry_to_last_exit"]
    assert 1.0 < whole < 200.0, r
    for name in ("dispatch_ramp", "prologue", "first_byte_latency", "streaming", "epilogue", "tail_skew"):
        assert r[name] <= whole, (name, r)
    events = ctx.time_gemv(rows, k, TensorDType.Float16, False, False, n_buffers=4, iters=50)
    assert whole + r["gap_after_previous_launch"] < 3.0 * events + 5.0, (r, events)     # stamps cost a little; same order of magnitude
    for bad in ((0, k, 4, 16), (rows, 12, 4, 16), (rows, k, 0, 16), (rows, k, 4, 1)):
        with pytest.raises(rllama_amd.RllamaHipError):
            ctx.probe_gemv_phases(bad[0], bad[1], n_buffers=bad[2], launches=bad[3])
