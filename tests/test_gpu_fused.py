"""The fused layer kernel (one launch for wo, w1|w3, w2 and the next block's wq|wk|wv, device-wide barriers between
them; off by default, RLLAMA_HIP_FUSED=1): bit-identical to the one-launch-per-product path, and a barrier that cannot
complete ends every workgroup and comes back as an error."""
import numpy as np
import pytest

import rllama_amd
from common import CONFIG0, SMALL, TINY, Shape, make_gpu, random_f32_weights, synth_weights

pytestmark = pytest.mark.gpu


def _pair(ctx, monkeypatch, shape, W, force_f16):
    monkeypatch.setenv("RLLAMA_HIP_FUSED", "0")
    plain = make_gpu(ctx, shape, W, force_f16)
    monkeypatch.setenv("RLLAMA_HIP_FUSED", "1")
    fused = make_gpu(ctx, shape, W, force_f16)
    return plain, fused


@pytest.mark.parametrize("shape,force_f16", [(TINY, True), (SMALL, True), (SMALL, False), (Shape(320, 1, 5, 872, 333, 40), True),
                                              (CONFIG0, True)], ids=["tiny-f16", "small-f16", "small-f32", "one-layer-ragged", "config0"])
def test_fused_layer_kernel_equals_the_separate_kernels(ctx, monkeypatch, shape, force_f16):
    """Same arithmetic in the same order (one shared device function), so logits, cache contents and greedy ids must agree
    bit for bit: token-by-token prompt (the variant without a last phase), single-token calls, the device-side greedy loop."""
    W = synth_weights(shape, seed=5, std=0.06) if force_f16 else random_f32_weights(shape, seed=5)
    plain, fused = _pair(ctx, monkeypatch, shape, W, force_f16)
    for m in (plain, fused):
        m.set_prefill_mode(True)                      # prompt tokens one by one: every token step runs the layer kernels
    toks = rllama_amd.synth_tokens(3, 12, 3, shape.vocab_size)
    cp, cf = plain.make_caches(), fused.make_caches()
    assert np.array_equal(fused.forward(toks[:7], 0, cf), plain.forward(toks[:7], 0, cp))
    for i in range(7, 12):
        assert np.array_equal(fused.forward(toks[i:i + 1], i, cf), plain.forward(toks[i:i + 1], i, cp)), i
    for l in range(shape.n_layers):
        for which in (0, 1):
            assert np.array_equal(cf.read(l, shape.n_heads - 1, which), cp.read(l, shape.n_heads - 1, which)), (l, which)
    n_new = min(20, shape.max_seq_len - 7)
    ids_p, _, _ = plain.generate_greedy(toks[:6], n_new, plain.make_caches())
    ids_f, _, _ = fused.generate_greedy(toks[:6], n_new, fused.make_caches())
    assert ids_f.tolist() == ids_p.tolist()
    plain.free()
    fused.free()


def test_fused_barrier_that_cannot_complete_is_an_error(ctx, monkeypatch):
    """A wait limit of zero ticks makes the first barrier give up at once (forced from the host; every workgroup still
    leaves the kernel normally): the call reports it, and a model with the normal limit works afterwards."""
    shape = SMALL
    W = synth_weights(shape, seed=2, std=0.06)
    monkeypatch.setenv("RLLAMA_HIP_FUSED", "1")
    monkeypatch.setenv("RLLAMA_HIP_FUSED_LIMIT_TICKS", "0")
    broken = make_gpu(ctx, shape, W, True)
    with pytest.raises(rllama_amd.RllamaHipError) as ei:
        broken.forward([5], 0, broken.make_caches())
    assert ei.value.code == 3 and "barrier" in str(ei.value)
    with pytest.raises(rllama_amd.RllamaHipError):
        broken.forward_greedy([5], 0, broken.make_caches())     # and again: the barrier words were cleared, the limit is still zero
    broken.free()
    monkeypatch.delenv("RLLAMA_HIP_FUSED_LIMIT_TICKS")
    good = make_gpu(ctx, shape, W, True)
    monkeypatch.setenv("RLLAMA_HIP_FUSED", "0")
    plain = make_gpu(ctx, shape, W, True)
    assert np.array_equal(good.forward([5, 9, 11], 0, good.make_caches()), plain.forward([5, 9, 11], 0, plain.make_caches()))
