"""The decode-attention entry point that allocates nothing (its scratch is an array inside the library) against the
allocating one: two calls in a row on one GPU, the second smaller, so that whatever the first call left in the shared
array must not matter."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_noalloc_decode_attention_equals_the_allocating_entry_point():
    import flexllm_amd as fx
    rng = np.random.default_rng(77)
    for length, qh, kvh, max_pos in [(4096, 32, 8, 4096), (700, 8, 2, 1024)]:
        print("decode attention without allocation: len", length, "heads", qh, kvh, flush=True)
        q_s = rng.uniform(0.003, 0.005, qh).astype(np.float32); k_s = rng.uniform(0.02, 0.04, kvh).astype(np.float32)
        v_s = rng.uniform(0.02, 0.04, kvh).astype(np.float32); a_s = np.full(qh, 1.0 / 255, np.float32)
        sc = fx.ops.Scales(q_s, k_s, v_s, a_s)
        q8 = fx.to_device(rng.integers(-128, 128, (qh, 64)).astype(np.int8))
        kc, vc = fx.ops.kv_cache(kvh, max_pos)
        k8 = rng.integers(-60, 60, (length, kvh, 64)).astype(np.int8); v8 = rng.integers(-128, 128, (length, kvh, 64)).astype(np.int8)
        fx.ops.kv_store_i8(fx.to_device(k8), fx.to_device(v8), kc, vc, 0)
        o_ref, p_ref = fx.ops.mha_i8_decode(q8, kc, vc, sc, length, want_p=True)
        o = fx.zeros((qh, 64), np.float32); p8 = fx.zeros((qh, length), np.uint8)
        fx.ops.mha_i8_decode_noalloc(q8, kc, vc, sc, length, o, p8)
        assert np.array_equal(p8.numpy(), p_ref.numpy())
        assert np.array_equal(o.numpy(), o_ref.numpy())
        assert np.abs(o.numpy()).max() > 0
    # sizes beyond the built-in scratch are refused with a message, not served
    kc, vc = fx.ops.kv_cache(16, 64)
    sc = fx.ops.Scales(np.ones(64, np.float32), np.ones(16, np.float32), np.ones(16, np.float32), np.ones(64, np.float32))
    with pytest.raises(Exception, match="exceeds the built-in scratch"):
        fx.ops.mha_i8_decode_noalloc(fx.zeros((64, 64), np.int8), kc, vc, sc, 8, fx.zeros((64, 64), np.float32))


def _free_bytes(fx):
    import ctypes as C
    free, total = C.c_size_t(), C.c_size_t()
    fx.check(fx.lib().flexllm_rt_mem_info(C.byref(free), C.byref(total)))
    return free.value


def test_noalloc_entry_point_allocates_nothing_on_a_fresh_stream():
    """The property the entry point exists for.  On a stream that no attention call has used (so no per-stream
    scratch exists for it), at the largest size the built-in array holds, the free device memory the runtime reports is
    the same before and after the call (the one-time symbol look-up is done first); the result equals the allocating
    entry point's.  The instrument is checked as well: the allocating entry point on another fresh stream, whose first
    call there must allocate its scratch, lowers the reported free memory."""
    import flexllm_amd as fx
    rng = np.random.default_rng(78)
    length, qh, kvh, max_pos = 8192, 32, 8, 8192
    sc = fx.ops.Scales(rng.uniform(0.003, 0.005, qh).astype(np.float32), rng.uniform(0.02, 0.04, kvh).astype(np.float32),
                       rng.uniform(0.02, 0.04, kvh).astype(np.float32), np.full(qh, 1.0 / 255, np.float32))
    q8 = fx.to_device(rng.integers(-128, 128, (qh, 64)).astype(np.int8))
    kc, vc = fx.ops.kv_cache(kvh, max_pos)
    fx.ops.kv_store_i8(fx.to_device(rng.integers(-60, 60, (length, kvh, 64)).astype(np.int8)),
                       fx.to_device(rng.integers(-128, 128, (length, kvh, 64)).astype(np.int8)), kc, vc, 0)
    o = fx.zeros((qh, 64), np.float32); p8 = fx.zeros((qh, length), np.uint8)
    fx.ops.mha_i8_decode_noalloc(q8, kc, vc, sc, 64, o)                 # symbol look-up of this device, default stream
    s1, s2 = fx.Stream(), fx.Stream()
    fx.device.device_sync()
    free0 = _free_bytes(fx)
    fx.ops.mha_i8_decode_noalloc(q8, kc, vc, sc, length, o, p8, stream=s1)
    s1.sync()
    free1 = _free_bytes(fx)
    assert free1 == free0, "the call changed the free device memory by %d bytes" % (free0 - free1)
    o_ref, p_ref = fx.ops.mha_i8_decode(q8, kc, vc, sc, length, want_p=True, stream=s2)   # allocates o, p8 and its scratch
    s2.sync()
    assert _free_bytes(fx) < free1 - qh * length * 4 // 2, "the allocating entry point's scratch does not show in the free memory"
    assert np.array_equal(p8.numpy(), p_ref.numpy()) and np.array_equal(o.numpy(), o_ref.numpy())
    assert np.abs(o.numpy()).max() > 0
