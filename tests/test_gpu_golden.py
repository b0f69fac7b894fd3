"""The device path against the committed vectors of tests/golden/modules_small.npz (inputs and expected outputs; no
oracle involved at run time).  Integer results bit for bit; floating point to the tolerance given at each check."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "modules_small.npz")


@pytest.fixture(scope="module")
def fx():
    import flexllm_amd as fx
    return fx


@pytest.fixture(scope="module")
def g():
    return np.load(GOLDEN)


def test_quant(fx, g):
    x = fx.to_device(g["quant_in_x"])
    q, s = fx.ops.quant_sym_i8(x)
    assert np.array_equal(q.numpy(), g["quant_out_q8"]) and np.array_equal(s.numpy(), g["quant_out_s8"])
    q4, s4, b4 = fx.ops.quant_asym_u8(x, bits=4)
    assert np.array_equal(q4.numpy(), g["quant_out_q4"])
    assert np.array_equal(s4.numpy(), g["quant_out_s4"]) and np.array_equal(b4.numpy(), g["quant_out_b4"])


def test_linear(fx, g):
    a, w = fx.to_device(g["linear_in_a"]), fx.to_device(g["linear_in_w"])
    assert np.array_equal(fx.ops.linear_i8_gemm(a, w).numpy(), g["linear_out_acc"])
    y = fx.ops.linear_i8_gemm_dequant(a, fx.to_device(g["linear_in_sx"]), w, fx.to_device(g["linear_in_ws"]))
    assert np.array_equal(y.numpy(), g["linear_out_y"])                        # (float(acc) * s_x) * w_s: same two roundings
    for row in range(2):                                                        # decode form, one token at a time
        acc = fx.ops.linear_i8_gemv(fx.to_device(g["linear_in_a"][row]), w)
        assert np.array_equal(acc.numpy().reshape(-1), g["linear_out_acc"][row])


def test_fht_rmsnorm_rope_swiglu(fx, g):
    assert np.array_equal(fx.ops.fht_f32(fx.to_device(g["fht_in_x"]), 32.0).numpy(), g["fht_out_y"])      # same stage order: exact
    y = fx.ops.rmsnorm_f32(fx.to_device(g["rmsnorm_in_x"]), fx.to_device(g["rmsnorm_in_gamma"]), eps=1e-5).numpy()
    np.testing.assert_allclose(y, g["rmsnorm_out_y"], rtol=2e-6, atol=1e-7)    # tree-reduced sum of squares
    y = fx.ops.rope_f32(fx.to_device(g["rope_in_x"]), fx.to_device(g["rope_in_sin"]), fx.to_device(g["rope_in_cos"]), 64).numpy()
    assert np.array_equal(y, g["rope_out_y"])
    h = fx.ops.swiglu_f32(fx.to_device(g["swiglu_in_gate"]), fx.to_device(g["swiglu_in_up"])).numpy()
    np.testing.assert_allclose(h, g["swiglu_out_h"], rtol=1e-6, atol=1e-7)     # device exponential within a few ulp of expf


def test_attention(fx, g):
    S, QH, HD = g["mha_in_q"].shape
    KVH = g["mha_in_k"].shape[1]
    sc = fx.ops.Scales(g["mha_in_qs"], g["mha_in_ks"], g["mha_in_vs"], g["mha_in_as"])
    q8 = fx.ops.static_quant_i8(fx.to_device(g["mha_in_q"]), fx.to_device(g["mha_in_qs"]), factor=8.0)
    assert np.array_equal(q8.numpy(), g["mha_out_q8"])
    kc, vc = fx.ops.kv_cache(KVH, 64)
    fx.ops.kv_append_i8(fx.to_device(g["mha_in_k"]), fx.to_device(g["mha_in_v"]), kc, vc, sc, 0)
    k_got = kc.numpy().transpose(1, 0, 2)[:S]
    v_got = vc.numpy().transpose(1, 3, 0, 2).reshape(64, KVH, HD)[:S]
    assert np.array_equal(k_got, g["mha_out_k8"]) and np.array_equal(v_got, g["mha_out_v8"])
    # prefill rows are padded to the 32-query tile: 48 -> 64 rows, the 16 extra ones are ignored
    q_pad = np.zeros((64, QH, HD), np.int8); q_pad[:S] = g["mha_out_q8"]
    o, p8 = fx.ops.mha_i8_prefill(fx.to_device(q_pad), kc, vc, sc, want_p=True)
    p_got = p8.numpy()[:, :S, :S]
    d = np.abs(p_got.astype(np.int32) - g["mha_out_p8"].astype(np.int32))
    assert d.max() <= 1 and (d != 0).mean() < 2e-3                             # rounding ties of p / A_s only
    tol = float(g["mha_in_as"][0] * g["mha_in_vs"][0] * 127) * (1 + d.sum())
    assert np.abs(o.numpy()[:S] - g["mha_out_o"]).max() <= tol + 1e-6
    od, pd = fx.ops.mha_i8_decode(fx.to_device(g["mhadec_in_q8"]), kc, vc, sc, S, want_p=True)
    dd = np.abs(pd.numpy().astype(np.int32) - g["mhadec_out_p8"].astype(np.int32))
    assert dd.max() <= 1 and (dd != 0).mean() < 1e-2
    assert np.abs(od.numpy() - g["mhadec_out_o"]).max() <= float(g["mha_in_as"][0] * g["mha_in_vs"][0] * 127) * (1 + dd.sum()) + 1e-6


def test_head_and_sampler(fx, g):
    logits = fx.ops.lm_head_f16(fx.to_device(g["head_in_table"].view(np.float16)), fx.to_device(g["head_in_n"])).numpy()
    np.testing.assert_allclose(logits, g["head_out_logits"], rtol=1e-5, atol=1e-6)       # fp32 sums in a different order
    lg = fx.to_device(g["topk_in_logits"])
    for i, rnd in enumerate(g["topk_in_rand"]):
        tok, idx, val, prob = fx.ops.sample_topk_f32(lg, 5, float(rnd))
        assert np.array_equal(idx, g["topk_out_idx"][i]) and np.array_equal(val, g["topk_out_val"][i])
        np.testing.assert_allclose(prob, g["topk_out_prob"][i], rtol=2e-6)
        assert tok == int(g["topk_out_token"][i])


def test_w4a4_and_hmt(fx, g):
    x = fx.to_device(g["w4a4_in_x"])
    q, s, b = fx.ops.quant_asym_u8(x, bits=4)
    w4 = fx.ops.pack_nibbles(fx.to_device(g["w4a4_in_w"]))
    y = fx.ops.linear_u4i4_gemm_dequant(fx.ops.pack_nibbles(q), s, b, w4, fx.to_device(g["w4a4_in_ws"]), fx.to_device(g["w4a4_in_wsum"]))
    assert np.array_equal(y.numpy(), g["w4a4_out_y"])
    from flexllm_amd import hmt
    a, p = hmt.hmt_retrieve(fx.to_device(g["hmt_in_q"]), fx.to_device(g["hmt_in_kmem"]), fx.to_device(g["hmt_in_mmem"]), 8.0)
    np.testing.assert_allclose(a.numpy(), g["hmt_out_a"], rtol=1e-4, atol=1e-7)          # fp32 dot products in lane order
    np.testing.assert_allclose(p.numpy(), g["hmt_out_p"], rtol=1e-4, atol=1e-6)
