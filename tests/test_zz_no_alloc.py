"""The allocation-free variant of rlh_attn_decode (static device work memory) against rlh_attn_decode itself, through the
C ABI: same kernels, so bit-identical outputs; two calls in a row, the second on a smaller input, and the size limit."""
import numpy as np
import pytest

import rllama_amd
from rllama_amd import Tensor, TensorDType

pytestmark = pytest.mark.gpu
f32 = np.float32


def _case(ctx, rng, H, hd, S, f16):
    K = rng.standard_normal((H * S, hd)).astype(f32)
    V = rng.standard_normal((H * S, hd)).astype(f32)
    if f16:
        K, V = K.astype(np.float16), V.astype(np.float16)
    q = rng.standard_normal((1, H * hd)).astype(f32)
    return Tensor.from_numpy(ctx, q), Tensor.from_numpy(ctx, K), Tensor.from_numpy(ctx, V)


def test_attn_decode_noalloc_equals_attn_decode(ctx):
    rng = np.random.default_rng(42)
    # first call: 8 heads of 128 dims, 1500 positions in 12 blocks per head; second call right after it: a smaller input
    # (fewer heads, shorter sequence, fewer blocks), which must not see anything the first call left in the work memory
    for (H, hd, S, T, n_splits, f16) in ((8, 128, 1536, 1500, 12, True), (3, 64, 400, 333, 5, True), (2, 128, 64, 40, 1, False),
                                          (5, 32, 900, 900, 0, False), (8, 128, 1536, 1500, 12, True)):
        q, ck, cv = _case(ctx, rng, H, hd, S, f16)
        want = q.attn_decode(ck, cv, H, S, T, n_splits=n_splits, round_out=f16).to_numpy()
        out = Tensor.zeros(ctx, 1, H * hd, TensorDType.Float32)
        q.attn_decode_noalloc(out, ck, cv, H, S, T, n_splits=n_splits, round_out=f16)
        got = out.to_numpy()
        assert np.isfinite(got).all()
        assert np.array_equal(got, want), (H, hd, T, n_splits, float(np.max(np.abs(got - want))))
        # and again on the same input: the counters the first call left behind must not matter
        q.attn_decode_noalloc(out, ck, cv, H, S, T, n_splits=n_splits, round_out=f16)
        assert np.array_equal(out.to_numpy(), want)


def test_attn_decode_noalloc_rejects_sizes_beyond_its_work_memory(ctx):
    H, hd, S = 128, 128, 128                       # 128 heads x 64 splits x 130 floats = 1,064,960 > 1,048,576
    z = Tensor.zeros(ctx, H * S, hd, TensorDType.Float16)
    q = Tensor.zeros(ctx, 1, H * hd, TensorDType.Float32)
    out = Tensor.zeros(ctx, 1, H * hd, TensorDType.Float32)
    with pytest.raises(rllama_amd.RllamaHipError) as ei:
        q.attn_decode_noalloc(out, z, z, H, S, 128, n_splits=64)
    assert ei.value.code == 6 and "static work memory" in str(ei.value)
    q.attn_decode_noalloc(out, z, z, H, S, 128, n_splits=63)      # 1,048,320 floats fit
    with pytest.raises(rllama_amd.RllamaHipError):
        q.attn_decode_noalloc(out, z, z, H, S, S + 1)             # the checks of rlh_attn_decode apply


def test_attn_decode_noalloc_allocates_nothing(ctx):
    """What the entry point exists for: no device allocation inside the call.  The free device memory the HIP runtime reports
    (hipMemGetInfo, called on the runtime library this process already has loaded) does not move over 50 calls at growing
    split counts, where the allocating entry point, asked for more work memory than it holds, makes it move."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    hip.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]

    def free_bytes():
        ctx.sync()
        free, total = C.c_size_t(0), C.c_size_t(0)
        assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
        return free.value

    rng = np.random.default_rng(43)
    H, hd, S, T = 64, 128, 2048, 2040
    q, ck, cv = _case(ctx, rng, H, hd, S, True)
    out = Tensor.zeros(ctx, 1, H * hd, TensorDType.Float32)
    q.attn_decode_noalloc(out, ck, cv, H, S, T, n_splits=2)       # first use
    before = free_bytes()
    for i in range(50):
        q.attn_decode_noalloc(out, ck, cv, H, S, T, n_splits=2 + i % 62)
    assert free_bytes() == before
    # the probe does see an allocation of the size in question: 64 heads x 64 splits x 130 floats = 2.1 MB of work memory
    held = Tensor.zeros(ctx, 64 * 64, 130 * 4, TensorDType.Float32)      # 8.5 MB: more than the allocator's granularity
    assert free_bytes() < before
    held.free()
