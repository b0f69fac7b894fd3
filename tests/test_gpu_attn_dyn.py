"""Attention with dynamic per-(token, head) Q/K/V scales (the library's own quantiser on every tensor, scores
dequantised per key, V's scale folded into the probabilities) against the oracle: prefill up to 1024 and 4096
tokens, decode of one token against 4096 cached positions."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fx():
    import flexllm_amd
    return flexllm_amd


def quantised_inputs(fx, oracle, s, qh, kvh, seed, max_pos=None):
    """fp32 q/k/v ~ N(0,1) with a per-token amplitude (so that the scales really differ), quantised on the device with
    flexllm_head_quant_sym_i8 and laid out in the caches; bit-identical to the oracle's tensors."""
    r = np.random.default_rng(seed)
    q = (r.standard_normal((s, qh, 64)) * r.uniform(0.3, 2.0, (s, qh, 1))).astype(np.float32)
    k = (r.standard_normal((s, kvh, 64)) * r.uniform(0.3, 2.0, (s, kvh, 1))).astype(np.float32)
    v = (r.standard_normal((s, kvh, 64)) * r.uniform(0.3, 2.0, (s, kvh, 1))).astype(np.float32)
    max_pos = max_pos or ((s + 63) // 64) * 64
    q8, q_s = fx.ops.head_quant_sym_i8(fx.to_device(q))
    k8, k_s = fx.ops.head_quant_sym_i8(fx.to_device(k))
    v8, v_s = fx.ops.head_quant_sym_i8(fx.to_device(v))
    kc, vc = fx.ops.kv_cache(kvh, max_pos)
    fx.ops.kv_store_i8(k8, v8, kc, vc, 0)
    ks_full = np.zeros((max_pos, kvh), np.float32); vs_full = np.zeros((max_pos, kvh), np.float32)
    ks_full[:s] = k_s.numpy(); vs_full[:s] = v_s.numpy()
    return (q, k, v), q8, q_s, kc, fx.to_device(ks_full), vc, fx.to_device(vs_full)


def check_against(p8, p_s, o, ref_p8, ref_p_s, ref_o, v8, group):
    """P within one step (rounding ties), the row scale to fp32 rounding, the integer P.V stage exact given the
    kernel's own bytes and scale, and the output within what the flipped steps explain."""
    np.testing.assert_allclose(p_s, ref_p_s, rtol=1e-5)       # sums of up to 4096 exponentials, associated differently
    d = np.abs(p8.astype(np.int32) - ref_p8.astype(np.int32))
    assert d.max() <= 1 and (d != 0).mean() < 2e-3, (d.max(), (d != 0).mean())
    assert p8.min() >= 0 and p8.max() == 127
    qh = p8.shape[0]
    acc = np.stack([p8[h].astype(np.float64) @ v8[:, h // group].astype(np.float64) for h in range(qh)], axis=1)   # [rows][qh][64], exact
    o_from_p = acc.astype(np.float32) * p_s[..., None]
    assert np.array_equal(o, o_from_p.astype(np.float32))
    flips = d.sum(-1).T[:, :, None]
    tol = ref_p_s[..., None] * 128
    err = np.abs(o.astype(np.float64) - ref_o) - flips * tol
    assert err.max() <= 1.2e-5 * np.abs(ref_o).max(), err.max()          # the row scale carries the row sum's rounding


@pytest.mark.parametrize("s,qh,kvh", [(32, 4, 1), (96, 8, 2), (256, 32, 8), (1024, 32, 8), (1088, 4, 1), (4096, 4, 1)])
def test_mha_prefill_dyn_vs_oracle(fx, oracle, s, qh, kvh):
    (q, k, v), q8, q_s, kc, k_s, vc, v_s = quantised_inputs(fx, oracle, s, qh, kvh, 100 + s)
    ref = oracle.mha_prefill_dyn(q, k, v, want_p=True)
    assert np.array_equal(q8.numpy(), ref["q8"]) and np.array_equal(q_s.numpy() / np.float32(8), ref["q_s"])
    assert np.array_equal(kc.numpy()[:, :s], ref["k8"].transpose(1, 0, 2)) and np.array_equal(k_s.numpy()[:s], ref["k_s"])
    o, p8, p_s = fx.ops.mha_i8_prefill_dyn(q8, q_s, kc, k_s, vc, v_s, want_p=True)
    p8 = p8.numpy()
    assert not np.triu(p8[0], 1).any()
    check_against(p8, p_s.numpy(), o.numpy(), ref["p8"], ref["p_s"], ref["o"], ref["v8"], qh // kvh)


def test_mha_prefill_dyn_per_channel_v_scale(fx, oracle):
    s, qh, kvh = 64, 8, 2
    (q, k, v), q8, q_s, kc, k_s, vc, v_s = quantised_inputs(fx, oracle, s, qh, kvh, 7)
    vch = np.random.default_rng(8).uniform(0.5, 2.0, (kvh, 64)).astype(np.float32)
    o0, _, _ = fx.ops.mha_i8_prefill_dyn(q8, q_s, kc, k_s, vc, v_s)
    o1, _, _ = fx.ops.mha_i8_prefill_dyn(q8, q_s, kc, k_s, vc, v_s, v_ch_s=fx.to_device(vch))
    assert np.array_equal(o1.numpy(), (o0.numpy() * np.repeat(vch, qh // kvh, axis=0)[None]).astype(np.float32))


@pytest.mark.parametrize("length,qh,kvh", [(1, 8, 2), (5, 4, 4), (127, 32, 8), (129, 32, 8), (1000, 8, 2), (4096, 32, 8)])
def test_mha_decode_dyn_vs_oracle(fx, oracle, length, qh, kvh):
    """One query against `length` cached positions (4096: the benchmark's decode case), cache tail poisoned."""
    r = np.random.default_rng(200 + length)
    max_pos = ((length + 63) // 64) * 64 + 64
    q8 = r.integers(-127, 128, (qh, 64)).astype(np.int8); q8[:, 0] = 127
    q_s = r.uniform(0.005, 0.02, qh).astype(np.float32)
    k8 = r.integers(-127, 128, (max_pos, kvh, 64)).astype(np.int8); v8 = r.integers(-127, 128, (max_pos, kvh, 64)).astype(np.int8)
    k_s = r.uniform(0.005, 0.03, (max_pos, kvh)).astype(np.float32); v_s = r.uniform(0.005, 0.03, (max_pos, kvh)).astype(np.float32)
    k_s[length:] = 1e30; v_s[length:] = 1e30                               # nothing beyond len may be read into the result
    kc, vc = fx.ops.kv_cache(kvh, max_pos)
    fx.ops.kv_store_i8(fx.to_device(k8), fx.to_device(v8), kc, vc, 0)
    o, p8, p_s = fx.ops.mha_i8_decode_dyn(fx.to_device(q8), fx.to_device(q_s), kc, fx.to_device(k_s), vc, fx.to_device(v_s), length, want_p=True)
    o_ref, p_ref, ps_ref = oracle.mha_decode_dyn(q8, q_s / np.float32(8), k8[:length], k_s[:length], v8[:length], v_s[:length], want_p=True)
    check_against(p8.numpy()[:, None, :], p_s.numpy()[None], o.numpy()[None], p_ref[:, None, :], ps_ref[None], o_ref[None], v8[:length], qh // kvh)


def test_mha_decode_dyn_equals_prefill_dyn_row(fx, oracle):
    """Size-independent property at the benchmark's shape: decode of query i over the first i+1 positions reproduces
    row i of the 1024-token prefill (same probability bytes up to tie flips, hence the same output)."""
    s, qh, kvh = 1024, 32, 8
    (q, k, v), q8, q_s, kc, k_s, vc, v_s = quantised_inputs(fx, oracle, s, qh, kvh, 55)
    o, p8, p_s = fx.ops.mha_i8_prefill_dyn(q8, q_s, kc, k_s, vc, v_s, want_p=True)
    o, p8, p_s = o.numpy(), p8.numpy(), p_s.numpy()
    q8h, qsh = q8.numpy(), q_s.numpy()
    for i in (0, 31, 32, 500, 1023):
        od, pd, psd = fx.ops.mha_i8_decode_dyn(fx.to_device(q8h[i]), fx.to_device(qsh[i]), kc, k_s, vc, v_s, i + 1, want_p=True)
        np.testing.assert_allclose(psd.numpy(), p_s[i], rtol=2e-6)
        d = np.abs(pd.numpy().astype(np.int32) - p8[:, i, :i + 1])
        assert d.max() <= 1 and (d != 0).mean() < 2e-3
        if not d.any():
            np.testing.assert_allclose(od.numpy(), o[i], rtol=2e-6, atol=1e-9)
