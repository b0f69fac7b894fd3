"""Pins the CPU oracle (oracle/flexllm_oracle.c) against facts that do not come from
the oracle's own formulas: closed forms, invariants, special cases, textbook routines
and brute force.  The reference ships no stored golden vectors for this path (its
testbenches synthesise inputs and compute goldens in-process), so these checks plus the
testbench-style float64 "fake-quant" goldens below are what anchors the oracle."""
import numpy as np
import pytest
import scipy.linalg
import scipy.special

rng = np.random.default_rng(1234)


# ------------------------------------------------------------------ quant
def test_quant_sym_special_cases(oracle):
    x = np.zeros((3, 16), np.float32)
    x[1, 3] = -2.54; x[1, 5] = 1.0
    x[2] = np.linspace(-1, 1, 16)
    q, s = oracle.quant_sym(x)
    assert s[0] == 1.0 and not q[0].any()              # all-zero row: scale 1, zeros
    assert q[1, 3] == -127 and s[1] == np.float32(2.54) / np.float32(127)
    assert q[2, 0] == -127 and q[2, -1] == 127         # absmax maps to +-127 exactly
    # dequantised error bounded by half a step
    assert np.all(np.abs(q[2] * s[2] - x[2]) <= s[2] * 0.5 * (1 + 1e-6))


def test_quant_sym_ties_round_away_from_zero(oracle):
    # scale = 127/127 = 1 exactly, so x/s = x and .5 values are exact ties
    x = np.array([[127.0, 0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 0.49999997]], np.float32)
    q, s = oracle.quant_sym(x)
    assert s[0] == 1.0
    assert q[0].tolist() == [127, 1, -1, 2, -2, 3, -3, 0]


def test_quant_sym_matches_numpy_float32(oracle):
    x = rng.standard_normal((64, 2048)).astype(np.float32)
    q, s = oracle.quant_sym(x)
    s_np = (np.abs(x).max(axis=1) / np.float32(127)).astype(np.float32)
    t = (x / s_np[:, None]).astype(np.float32)
    q_np = (np.sign(t) * np.floor(np.abs(t) + np.float32(0.5))).astype(np.int8)
    assert np.array_equal(s, s_np) and np.array_equal(q, q_np)


def test_quant_asym_range_and_endpoints(oracle):
    x = rng.uniform(-1, 1, (8, 256)).astype(np.float32)
    q, s, b = oracle.quant_asym(x, bits=4)
    assert q.min() == 0 and q.max() == 15
    assert np.array_equal(b, x.min(axis=1))
    assert np.all(q[np.arange(8), x.argmax(axis=1)] == 15)
    assert np.all(np.abs(q * s[:, None] + b[:, None] - x) <= s[:, None] * 0.5 * (1 + 1e-5))


def test_dequant_order_and_asym_term(oracle):
    acc = rng.integers(-2**20, 2**20, (4, 32)).astype(np.int32)
    s_x = rng.uniform(1e-3, 1e-2, 4).astype(np.float32)
    w_s = rng.uniform(1e-3, 1e-2, 32).astype(np.float32)
    y = oracle.dequant(acc, s_x, w_s)
    ref = (acc.astype(np.float32) * s_x[:, None]).astype(np.float32) * w_s[None, :]
    assert np.array_equal(y, ref.astype(np.float32))
    b = rng.uniform(-1, 1, 4).astype(np.float32); ws = rng.uniform(-5, 5, 32).astype(np.float32)
    y2 = oracle.dequant(acc, s_x, w_s, b, ws)
    np.testing.assert_allclose(y2, ref.astype(np.float64) + b[:, None].astype(np.float64) * ws[None, :], rtol=1e-6, atol=1e-7)


def test_static_quant_clamps(oracle):
    x = np.array([[[1000.0, -1000.0, 0.26, -0.26, 0.25, 127.49 * 0.5]]], np.float32)
    q = oracle.static_quant(x, np.array([0.5], np.float32), factor=1.0, signed=True)
    assert q[0, 0].tolist() == [127, -128, 1, -1, 1, 127]
    p = np.array([[[1.0, 0.5, 0.0, 1.5 / 256, 200.0 / 256]]], np.float32)
    u = oracle.static_quant(p, np.array([1.0 / 256], np.float32), signed=False)
    assert u.dtype == np.uint8 and u[0, 0].tolist() == [255, 128, 0, 2, 200]
    # unsigned branch clamps high only at 2^8-1
    u2 = oracle.static_quant(np.array([[[3.0]]], np.float32), np.array([1.0 / 255], np.float32), signed=False)
    assert u2[0, 0, 0] == 255
    # q uses factor*scale as the divisor (sqrt(head_dim) folded into the Q scale)
    q2 = oracle.static_quant(np.array([[[8.0]]], np.float32), np.array([0.5], np.float32), factor=8.0)
    assert q2[0, 0, 0] == 2


# ------------------------------------------------------------------ integer GEMM
def test_linear_i8_exact(oracle):
    a = rng.integers(-128, 128, (5, 300)).astype(np.int8)
    w = rng.integers(-128, 128, (7, 300)).astype(np.int8)
    assert np.array_equal(oracle.linear_i8(a, w), a.astype(np.int64) @ w.astype(np.int64).T)
    au = rng.integers(0, 256, (5, 300)).astype(np.uint8)
    assert np.array_equal(oracle.linear_i8(au, w), au.astype(np.int64) @ w.astype(np.int64).T)
    # extreme values at K=8192 stay inside int32
    a = np.full((1, 8192), -128, np.int8); w = np.full((1, 8192), -128, np.int8)
    assert oracle.linear_i8(a, w)[0, 0] == 8192 * 128 * 128


# ------------------------------------------------------------------ FHT
@pytest.mark.parametrize("n", [2, 4, 8, 16, 64])
def test_fht_equals_sylvester_matrix_exactly_on_integers(oracle, n):
    x = rng.integers(-50, 50, (6, n)).astype(np.float32)
    H = scipy.linalg.hadamard(n).astype(np.float64)
    assert np.array_equal(oracle.fht(x), (x.astype(np.float64) @ H.T).astype(np.float32))


@pytest.mark.parametrize("n", [2048, 8192])
def test_fht_large_vs_float64_and_involution(oracle, n):
    x = rng.standard_normal((3, n)).astype(np.float32)
    H = scipy.linalg.hadamard(n).astype(np.float64)
    scale = np.float32(np.sqrt(n))
    y = oracle.fht(x, scale)
    np.testing.assert_allclose(y, x.astype(np.float64) @ H.T / np.float64(scale), rtol=0, atol=2e-5)
    np.testing.assert_allclose(oracle.fht(y, scale), x, atol=1e-5)              # H(Hx)/n = x
    np.testing.assert_allclose((y.astype(np.float64) ** 2).sum(1), (x.astype(np.float64) ** 2).sum(1), rtol=1e-5)


def test_fht_stage_order_is_bits_1_to_m_minus_1_then_0(oracle):
    """The omega network equals an in-place butterfly network whose stage s pairs indices that
    differ in bit (s+1) mod m, bit-clear element first; same float result bit for bit."""
    n, m = 256, 8
    x = (rng.standard_normal((4, n)) * 1e3).astype(np.float32)
    d = x.copy()
    idx = np.arange(n)
    for s in range(m):
        bit = 1 << ((s + 1) % m)
        lo = idx[(idx & bit) == 0]
        u, v = d[:, lo].copy(), d[:, lo | bit].copy()
        d[:, lo] = u + v
        d[:, lo | bit] = u - v
    assert np.array_equal(oracle.fht(x), d)


# ------------------------------------------------------------------ norms / activations
def test_rmsnorm_vs_float64(oracle):
    x = rng.standard_normal((16, 2048)).astype(np.float32) * 3
    g = rng.uniform(0.5, 1.5, 2048).astype(np.float32)
    x64 = x.astype(np.float64)
    ref = x64 / np.sqrt((x64 ** 2).mean(1, keepdims=True) + 1e-5) * g
    np.testing.assert_allclose(oracle.rmsnorm_pref(x, g), ref, rtol=2e-6)
    for bp in (4, 8, 16):
        np.testing.assert_allclose(oracle.rmsnorm_dec(x[0], g, bp), ref[0], rtol=2e-6)
    # unit-gamma output has unit mean square
    y = oracle.rmsnorm_pref(x, np.ones(2048, np.float32))
    np.testing.assert_allclose((y.astype(np.float64) ** 2).mean(1), 1.0, rtol=1e-4)


def test_swish_gate_residual(oracle):
    x = rng.standard_normal(4096).astype(np.float32) * 4
    np.testing.assert_allclose(oracle.swish(x), x.astype(np.float64) * scipy.special.expit(x.astype(np.float64)), rtol=1e-6, atol=1e-9)
    assert oracle.swish(np.zeros(1, np.float32))[0] == 0
    a = rng.standard_normal(64).astype(np.float32); b = rng.standard_normal(64).astype(np.float32)
    assert np.array_equal(oracle.gate(a, b), a * b) and np.array_equal(oracle.residual(a, b), a + b)


def test_softmax_vs_scipy_and_ragged(oracle):
    for dim in (1, 3, 5, 64, 1023, 4096):
        x = (rng.standard_normal((3, dim)) * 5).astype(np.float32)
        y = oracle.softmax(x)
        np.testing.assert_allclose(y, scipy.special.softmax(x.astype(np.float64), axis=1), rtol=3e-6, atol=1e-12)
        np.testing.assert_allclose(y.astype(np.float64).sum(1), 1.0, rtol=1e-5)
    # masked entries (-1e32) become exact zeros and do not disturb the rest
    x = (rng.standard_normal((1, 64))).astype(np.float32)
    xm = x.copy(); xm[0, 40:] = np.float32(-1e32)
    ym = oracle.softmax(xm)
    assert not ym[0, 40:].any()
    assert np.array_equal(ym[0, :40], oracle.softmax(x[:, :40])[0])


def test_causal_mask(oracle):
    x = rng.standard_normal((8, 2, 8)).astype(np.float32)
    y = oracle.causal_mask(x)
    for r in range(8):
        assert np.array_equal(y[r, :, :r + 1], x[r, :, :r + 1])
        assert np.all(y[r, :, r + 1:] == np.float32(-1e32))


# ------------------------------------------------------------------ RoPE
def _hf_llama3_inv_freq(head_dim=64, theta=500000.0, factor=32.0, low=1.0, high=4.0, orig=8192):
    """Llama-3 rope scaling as published with the model (float64)."""
    inv_freq = 1.0 / theta ** (np.arange(0, head_dim, 2, dtype=np.float64) / head_dim)
    low_wl, high_wl = orig / low, orig / high
    wl = 2 * np.pi / inv_freq
    out = np.where(wl > low_wl, inv_freq / factor, inv_freq)
    smooth = (orig / wl - low) / (high - low)
    mid = (1 - smooth) * inv_freq / factor + smooth * inv_freq
    is_mid = (wl >= high_wl) & (wl <= low_wl)
    return np.where(is_mid, mid, out)


def test_rope_table_vs_published_llama3_scaling(oracle):
    s, c = oracle.rope_table(2048)
    inv = _hf_llama3_inv_freq()
    pos = np.arange(2048, dtype=np.float64)[:, None]
    # float32 angle pos*freq carries ~1e-7 relative error -> absolute error grows with the angle
    np.testing.assert_allclose(s, np.sin(pos * inv), atol=3e-4)
    np.testing.assert_allclose(c, np.cos(pos * inv), atol=3e-4)
    np.testing.assert_allclose(s[:64], np.sin(pos[:64] * inv), atol=1e-5)
    assert np.all(s[0] == 0) and np.all(c[0] == 1)


def test_rope_rotation_properties(oracle):
    s, c = oracle.rope_table(128)
    x = rng.standard_normal((100, 4, 64)).astype(np.float32)
    y = oracle.rope(x, s, c, pos0=7)
    # pairs (k, k+32) are rotated: norms preserved
    np.testing.assert_allclose(y[..., :32] ** 2 + y[..., 32:] ** 2, x[..., :32] ** 2 + x[..., 32:] ** 2, rtol=1e-5, atol=1e-6)
    z = (x[..., :32] + 1j * x[..., 32:]) * (c[7:107, None, :] + 1j * s[7:107, None, :])
    np.testing.assert_allclose(y[..., :32], z.real, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(y[..., 32:], z.imag, rtol=1e-5, atol=1e-6)
    assert np.array_equal(oracle.rope(x[:1], s, c, pos0=0), x[:1])       # position 0 is the identity


# ------------------------------------------------------------------ attention
def _scales(qh=8, kvh=2):
    q_s = (0.02 + 0.002 * np.arange(qh)).astype(np.float32)
    k_s = (0.03 + 0.003 * np.arange(kvh)).astype(np.float32)
    v_s = (0.025 + 0.002 * np.arange(kvh)).astype(np.float32)
    a_s = np.full(qh, 1.0 / 255, np.float32)
    return q_s, k_s, v_s, a_s


def test_mha_prefill_vs_testbench_style_fake_quant_golden(oracle):
    """Golden built the way SpinQuant_Llama_32_1B/MHA_i8xi8_prefilling_tb.cpp:26-218 builds it:
    fake-quant q/k/v, float matmuls, masked softmax, fake-quant P, float PV; 5e-3 relative (tb :251)."""
    S, qh, kvh, hd = 64, 8, 2, 64
    q = rng.uniform(-2.8, 2.8, (S, qh, hd)).astype(np.float32)
    k = rng.uniform(-2.8, 2.8, (S, kvh, hd)).astype(np.float32)
    v = rng.uniform(-2.8, 2.8, (S, kvh, hd)).astype(np.float32)
    q_s, k_s, v_s, a_s = _scales(qh, kvh)
    out = oracle.mha_prefill(q, k, v, q_s, k_s, v_s, a_s, want_p=True)
    rnd = lambda t: np.sign(t) * np.floor(np.abs(t) + 0.5)
    qf = np.clip(rnd(q.astype(np.float64) / 8 / q_s[None, :, None]), -128, 127)
    kf = np.clip(rnd(k.astype(np.float64) / k_s[None, :, None]), -128, 127)
    vf = np.clip(rnd(v.astype(np.float64) / v_s[None, :, None]), -128, 127)
    assert np.array_equal(out["q8"], qf) and np.array_equal(out["k8"], kf) and np.array_equal(out["v8"], vf)
    o_ref = np.zeros((S, qh, hd))
    for h in range(qh):
        kh = h // (qh // kvh)
        a = (qf[:, h] * q_s[h]) @ (kf[:, kh] * k_s[kh]).T
        a[np.triu_indices(S, 1)] = -np.inf
        p = scipy.special.softmax(a, axis=1)
        pq = np.minimum(255, rnd(p / a_s[h]))
        # P may differ by one step where p/a_s sits on a rounding tie in float32 vs float64
        assert np.abs(out["p8"][h].astype(np.int64) - pq).max() <= 1
        assert (out["p8"][h] != pq).mean() < 2e-3
        assert not np.triu(out["p8"][h], 1).any()
        o_ref[:, h] = (out["p8"][h].astype(np.float64) * a_s[h]) @ (vf[:, kh] * v_s[kh])
    np.testing.assert_allclose(out["o"], o_ref, rtol=5e-3, atol=1e-5)
    np.testing.assert_allclose(out["o"], o_ref, rtol=1e-5, atol=1e-6)


def test_mha_decode_equals_prefill_rows_bit_for_bit(oracle):
    """Decode of query i over i+1 cached keys must reproduce prefill row i exactly: masked scores
    contribute exact zeros to the same four partial sums."""
    S, qh, kvh, hd = 37 + 3, 8, 2, 64
    q = rng.uniform(-3, 3, (S, qh, hd)).astype(np.float32)
    k = rng.uniform(-3, 3, (S, kvh, hd)).astype(np.float32)
    v = rng.uniform(-3, 3, (S, kvh, hd)).astype(np.float32)
    sc = _scales(qh, kvh)
    out = oracle.mha_prefill(q, k, v, *sc, want_p=True)
    for i in (0, 1, 2, 3, 4, 17, S - 1):
        o, p = oracle.mha_decode(out["q8"][i], out["k8"][:i + 1], out["v8"][:i + 1], *sc, want_p=True)
        assert np.array_equal(o, out["o"][i])
        assert np.array_equal(p, out["p8"][:, i, :i + 1])


def test_mha_dyn_vs_float64_fake_quant_golden_with_per_token_scales(oracle):
    """Attention with dynamic per-(token, head) scales: golden built the testbench way (fake-quant tensors, float
    matmuls, scipy softmax) in float64 with every scale taken per token and head; the three facts the variant adds
    (1/sqrt(d) folded into Q's scale, K's scale indexed by KEY, V's scale folded into the probabilities) are each
    switched off once and must be noticed."""
    S, qh, kvh, hd = 48, 8, 2, 64
    r = np.random.default_rng(77)
    q = (r.standard_normal((S, qh, hd)) * r.uniform(0.2, 3, (S, qh, 1))).astype(np.float32)      # scales differ a lot per token
    k = (r.standard_normal((S, kvh, hd)) * r.uniform(0.2, 3, (S, kvh, 1))).astype(np.float32)
    v = (r.standard_normal((S, kvh, hd)) * r.uniform(0.2, 3, (S, kvh, 1))).astype(np.float32)
    out = oracle.mha_prefill_dyn(q, k, v, want_p=True)
    rnd = lambda t: np.sign(t) * np.floor(np.abs(t) + 0.5)
    sq = np.abs(q).max(-1) / np.float32(127); sk = np.abs(k).max(-1) / np.float32(127); sv = np.abs(v).max(-1) / np.float32(127)
    assert np.array_equal(out["q_s"], (sq / np.float32(8)).astype(np.float32)) and np.array_equal(out["k_s"], sk) and np.array_equal(out["v_s"], sv)
    qf, kf, vf = rnd(q / sq[..., None]), rnd(k / sk[..., None]), rnd(v / sv[..., None])
    assert np.array_equal(out["q8"], qf) and np.array_equal(out["k8"], kf) and np.array_equal(out["v8"], vf)
    assert np.abs(out["q8"]).max(-1).min() == 127                       # every (token, head) uses its full range

    def golden(mut=None):
        o = np.zeros((S, qh, hd)); P = np.zeros((qh, S, S)); ps = np.zeros((S, qh))
        for h in range(qh):
            kh = h // (qh // kvh)
            q_deq = qf[:, h] * (sq[:, h, None].astype(np.float64) / (1.0 if mut == "no_sqrt_d" else 8.0))
            k_scale = sk[:, kh].astype(np.float64)
            a = (q_deq @ kf[:, kh].T) * (k_scale[:, None] if mut == "k_scale_by_query" else k_scale[None, :])
            a[np.triu_indices(S, 1)] = -np.inf
            p = scipy.special.softmax(a, axis=1)
            pp = p * (1.0 if mut == "v_scale_not_folded" else sv[None, :, kh].astype(np.float64))
            ps[:, h] = pp.max(1) / 127.0
            P[h] = rnd(pp / ps[:, h, None])
            o[:, h] = (P[h] * ps[:, h, None]) @ vf[:, kh]
        return o, P, ps

    o_ref, P_ref, ps_ref = golden()
    np.testing.assert_allclose(out["p_s"], ps_ref, rtol=2e-6)
    d = np.abs(out["p8"].astype(np.int64) - P_ref)
    assert d.max() <= 1 and (d != 0).mean() < 2e-3 and out["p8"].min() == 0 and out["p8"].max() == 127
    assert not np.triu(out["p8"][0], 1).any()
    np.testing.assert_allclose(out["o"], o_ref, rtol=0, atol=3e-3 * np.abs(o_ref).max())       # P steps of 1/127
    o_exact = np.stack([(out["p8"][h].astype(np.float64) * out["p_s"][:, h, None].astype(np.float64)) @ vf[:, h // (qh // kvh)]
                        for h in range(qh)], axis=1)
    np.testing.assert_allclose(out["o"], o_exact, rtol=1e-5, atol=1e-6)
    for mut in ("no_sqrt_d", "k_scale_by_query", "v_scale_not_folded"):
        assert np.abs(golden(mut)[0] - out["o"]).max() > 3e-2 * np.abs(o_ref).max(), mut
    # per-channel V scale (the reference library's own form, MHA.h:713-738): one more factor per output channel
    vch = r.uniform(0.5, 2.0, (kvh, hd)).astype(np.float32)
    o2 = oracle.mha_prefill_dyn(q, k, v, v_ch_s=vch)["o"]
    assert np.array_equal(o2, (out["o"] * np.repeat(vch, qh // kvh, axis=0)[None]).astype(np.float32))


def test_mha_decode_dyn_equals_prefill_dyn_rows_bit_for_bit(oracle):
    S, qh, kvh, hd = 37, 8, 2, 64
    r = np.random.default_rng(78)
    q = r.standard_normal((S, qh, hd)).astype(np.float32); k = r.standard_normal((S, kvh, hd)).astype(np.float32)
    v = r.standard_normal((S, kvh, hd)).astype(np.float32)
    out = oracle.mha_prefill_dyn(q, k, v, want_p=True)
    for i in (0, 1, 5, 20, S - 1):
        o, p8, p_s = oracle.mha_decode_dyn(out["q8"][i], out["q_s"][i], out["k8"][:i + 1], out["k_s"][:i + 1],
                                           out["v8"][:i + 1], out["v_s"][:i + 1], want_p=True)
        assert np.array_equal(o, out["o"][i]) and np.array_equal(p_s, out["p_s"][i])
        assert np.array_equal(p8, out["p8"][:, i, :i + 1])


# ------------------------------------------------------------------ layouts
def test_prefill_and_decode_stream_layouts_roundtrip_and_index_formula(oracle):
    tokens, dim, tp = 16, 24, 8
    x = rng.standard_normal((tokens, dim)).astype(np.float32)
    p = oracle.pack_pref(x, tp)
    # MHA_i8xi8_prefilling_tb.cpp:38-40: idx = (i/TP)*dim + j ; sub = i%TP
    for i in (0, 7, 8, 15):
        for j in (0, 5, 23):
            assert p.reshape(-1, tp)[(i // tp) * dim + j, i % tp] == x[i, j]
    assert np.array_equal(oracle.unpack_pref(p, tp), x)
    bp, d = 8, 64
    t = rng.standard_normal(d).astype(np.float32)
    pd = oracle.pack_dec(t, bp)
    # Linear_Layer_Decoding_tb.cpp:148: [j % (dim/BP)][j / (dim/BP)]
    for j in (0, 7, 8, 63):
        assert pd[j % (d // bp), j // (d // bp)] == t[j]
    assert np.array_equal(oracle.unpack_dec(pd, bp), t)


def test_half_to_float_and_lm_head(oracle):
    vals = np.array([0.0, -0.0, 1.0, -2.5, 65504.0, 6.1e-5, 5.96e-8, 3e-6, 0.333], np.float16)
    for h in vals:
        assert np.float32(oracle.half_to_float(h.view(np.uint16))) == np.float32(h)
    E = rng.standard_normal((50, 128)).astype(np.float16)
    n = rng.standard_normal(128).astype(np.float32)
    np.testing.assert_allclose(oracle.lm_head(E.view(np.uint16), n), E.astype(np.float64) @ n, rtol=1e-4, atol=1e-4)


# ------------------------------------------------------------------ Logits.h top-k sampling
def test_sample_topk_against_sorting_and_closed_forms(oracle):
    """Pins fxo_sample_topk (Logits.h:145-279) with facts outside its own loops: the candidates are the k largest
    logits (numpy sort, no ties in random data) for any lane count; the probabilities are the softmax of the k values
    (float64); the token is the first candidate whose cumulative probability exceeds rand, the last one otherwise."""
    r = np.random.default_rng(5)
    for n, k, lanes in [(128256, 5, 8), (4096, 1, 4), (1024, 8, 16), (64, 16, 1), (131072, 5, 32)]:
        x = (r.standard_normal(n) * 4).astype(np.float32)
        order = np.argsort(-x.astype(np.float64), kind="stable")[:k]
        p64 = np.exp(x[order].astype(np.float64) - float(x[order][0])); p64 /= p64.sum()
        cdf32 = np.cumsum(p64)
        for rand in (0.0, 0.13, 0.5, 0.77, 0.999999):
            tok, idx, val, prob = oracle.sample_topk(x, k, rand, lanes)
            assert np.array_equal(idx, order) and np.array_equal(val, x[order])
            np.testing.assert_allclose(prob, p64, rtol=2e-6)
            margins = np.abs(cdf32 - rand)
            if margins.min() > 1e-5:                       # away from a boundary the choice is unambiguous
                sel = int(np.argmax(cdf32 > rand)) if (cdf32 > rand).any() else k - 1
                assert tok == order[sel]
    # rand beyond the last cumulative value (rounding): the last candidate
    x = np.zeros(64, np.float32); x[[3, 9, 20]] = [2.0, 1.0, 0.5]
    assert oracle.sample_topk(x, 3, 1.5, 8)[0] == 20
    # enable_sub_max=False: plain exp of the logits, same normalised probabilities here
    a = oracle.sample_topk(x, 3, 0.2, 8, enable_sub_max=False)[3]
    b = oracle.sample_topk(x, 3, 0.2, 8, enable_sub_max=True)[3]
    np.testing.assert_allclose(a, b, rtol=1e-6)


def test_sample_topk_tie_order_is_the_insertion_order(oracle):
    """sort_top_k inserts with a strict '>' (Logits.h:15): of equal logits the one inserted first ranks higher.
    Within a lane that is the smaller index; across lanes the merge is rank-major (Logits.h:224-232), so a lane's
    second equal value ranks behind another lane's first one even if its index is smaller."""
    x = np.full(32, -5.0, np.float32)
    x[[1, 2]] = 7.0          # lane 0 (indices 0..7) holds two equal maxima
    x[9] = 7.0               # lane 1 holds one
    tok, idx, val, prob = oracle.sample_topk(x, 3, 0.0, 4)
    assert list(idx) == [1, 9, 2] and np.all(val == 7.0)
    np.testing.assert_allclose(prob, [1 / 3] * 3, rtol=1e-6)


# ------------------------------------------------------------------ HMT plug-in (Modules/HMT.h)
def test_linear_f32_and_scaled_softmax_against_float64(oracle):
    x = rng.standard_normal(2048).astype(np.float32)
    w = rng.standard_normal((96, 2048)).astype(np.float32)
    y = oracle.linear_f32(x, w)
    ref = w.astype(np.float64) @ x.astype(np.float64)
    np.testing.assert_allclose(y, ref, rtol=0, atol=2e-4)                  # ~45 * 2048 * 2^-24 worst-case growth
    assert np.array_equal(oracle.linear_f32(np.ones(8, np.float32), np.arange(16, dtype=np.float32).reshape(2, 8)),
                          np.array([28, 92], np.float32))                  # exact in any order
    a = (rng.standard_normal(64) * 30).astype(np.float32)
    p = oracle.softmax_dec(a, 4, scale=45.2548339959)
    ref = scipy.special.softmax(a.astype(np.float64) / 45.2548339959)      # the scale divides the exponent
    np.testing.assert_allclose(p, ref, rtol=2e-6)
    assert abs(float(p.sum()) - 1.0) < 1e-6
    p1 = oracle.softmax_dec(a, 4)                                          # without scale: plain softmax
    np.testing.assert_allclose(p1, scipy.special.softmax(a.astype(np.float64)), rtol=2e-6, atol=1e-30)


def test_hmt_retrieve_counts_empty_slots_and_is_a_convex_combination(oracle):
    hidden, mem_num = 256, 8
    mmem = np.zeros((mem_num, hidden), np.float32); kmem = np.zeros((mem_num, hidden), np.float32)
    mmem[:3] = rng.standard_normal((3, hidden)); kmem[:3] = rng.standard_normal((3, hidden))
    q = rng.standard_normal(hidden).astype(np.float32)
    scale = 16.0
    a, p = oracle.hmt_retrieve(q, kmem, mmem, scale)
    s = kmem.astype(np.float64) @ q.astype(np.float64)                     # empty slots score exactly 0 and take part
    ref_a = scipy.special.softmax(s / scale)
    np.testing.assert_allclose(a, ref_a, rtol=1e-5)
    np.testing.assert_allclose(p, ref_a @ mmem.astype(np.float64), rtol=0, atol=1e-5)
    assert a[3:].min() > 0 and np.allclose(a[3:], a[3])                    # five empty slots share equal, non-zero weight
    # a zero query weighs all slots equally: P is the mean over ALL slots, empty ones included
    a0, p0 = oracle.hmt_retrieve(np.zeros(hidden, np.float32), kmem, mmem, scale)
    assert np.allclose(a0, 1.0 / mem_num)
    np.testing.assert_allclose(p0, mmem.sum(0) / mem_num, rtol=0, atol=1e-6)


def test_hmt_stage_lengths_match_the_reference_comments(oracle):
    # Modules/HMT.h:47 "1 + 495 + 1 = 497" and :125 "1 + 32 + 990 + 1 = 1024" for a full segment, before padding to
    # the token-parallel factor (8): 497 -> 504, 1024 -> 1024
    cur, l0, l1 = oracle.hmt_stage_lengths(3000, 1, 4, 990, 495, 32, 8)
    assert (cur, l0, l1) == (990, 504, 1024)
    cur, l0, l1 = oracle.hmt_stage_lengths(3000, 3, 4, 990, 495, 32, 8)    # last segment: 3000 - 3*990 = 30 tokens
    assert (cur, l0, l1) == (30, 32, 64)


def test_hmt_segment_flow_with_a_transparent_backbone(oracle):
    """With the reference's own stand-in backbone (hmt_dummy_prefilling, Modules/HMT.h:494-521: x + 1) every quantity
    of the segment loop has a closed form: S_n = T + 1, M_n = P_n + 1, slot = n % mem_num."""
    hidden, seg_len, sum_len, rec, mem_num = 64, 10, 5, 3, 2
    emb = rng.standard_normal((34, hidden)).astype(np.float32)             # 4 segments: 10, 10, 10, 4
    t_embed = rng.standard_normal(hidden).astype(np.float32)
    wq = (rng.standard_normal((hidden, hidden)) / 8).astype(np.float32)
    wk = (rng.standard_normal((hidden, hidden)) / 8).astype(np.float32)
    seen = []

    def backbone(x):
        seen.append(x.copy())
        return x + np.float32(1.0)

    outs, mmem, kmem, ps = oracle.hmt_run(backbone, emb, t_embed, wq, wk, seg_len, sum_len, rec, mem_num, 8.0, pad=4, block_parallel=2)
    assert [o.shape[0] for o in outs] == [10, 10, 10, 4] and len(ps) == 3 and len(seen) == 7
    for n, o in enumerate(outs):                                           # stage-1 rows of the segment's own tokens
        assert np.array_equal(o, emb[n * seg_len:n * seg_len + o.shape[0]] + np.float32(1.0))
    # stage-1 input of segment 0: zero P, zero recurrent rows (nothing precedes the text), tokens, zero P, zero padding
    x1 = seen[0]
    assert x1.shape[0] == 16 and not x1[0].any() and not x1[1:4].any() and np.array_equal(x1[4:14], emb[:10]) and not x1[14:].any()
    # stage-0 input of segment 1: [T, first 5 tokens of the segment, T] padded to 8
    x0 = seen[1]
    assert x0.shape[0] == 8 and np.array_equal(x0[0], t_embed) and np.array_equal(x0[1:6], emb[10:15]) and np.array_equal(x0[6], t_embed) and not x0[7].any()
    # stage-1 input of segment 1: P_1, the 3 tokens before the segment, the segment, P_1
    x1 = seen[2]
    assert np.array_equal(x1[0], ps[0]) and np.array_equal(x1[1:4], emb[7:10]) and np.array_equal(x1[4:14], emb[10:20]) and np.array_equal(x1[14], ps[0])
    # last segment: no trailing P row
    assert not seen[6][1 + rec + 4:].any()
    # memories: M_0 = 0 + 1 went to slot 0, M_1 = P_1 + 1 to slot 1, M_2 = P_2 + 1 overwrote slot 0 (ring of 2)
    assert np.array_equal(mmem[1], ps[0] + np.float32(1.0)) and np.array_equal(mmem[0], ps[1] + np.float32(1.0))
    np.testing.assert_allclose(kmem[0], wk.astype(np.float64) @ mmem[0].astype(np.float64), rtol=0, atol=1e-5)
    # P_1 from first principles in float64: only slot 0 is filled (ones), slot 1 empty
    q1 = wq.astype(np.float64) @ (t_embed.astype(np.float64) + 1.0)
    k0 = wk.astype(np.float64) @ np.ones(hidden)
    wts = scipy.special.softmax(np.array([q1 @ k0, 0.0]) / 8.0)
    np.testing.assert_allclose(ps[0], wts[0] * np.ones(hidden), rtol=0, atol=1e-5)
