"""Pins the oracle's graph-level functions (fxo_llama_decode_token, fxo_llama_prefill, oracle.w4a4_layer) and its
remaining one-liners against an independent restatement of the reference's task graphs
(SpinQuant_Llama_32_1B/SpinQuant_Prefilling.h:940-1049, SpinQuant_Decoding_mem_opt.h:1050-1126) written here in
float64 numpy the way the reference's testbenches build their goldens: "fake quant" (round to the integer grid, keep
the value as a float), float matmuls of dequantised operands, scipy softmax, the explicit Sylvester matrix for the
Hadamard rotation and the published Llama-3 rotary formula.  Nothing in this file calls an oracle function to build
the expected values.

Every wiring fact the graphs depend on is switched off once (`mut=`): the restatement with that fact broken must
DISAGREE with the oracle, which shows that the agreement of the unbroken one pins it.
"""
import numpy as np
import pytest
import scipy.linalg
import scipy.special

CFG = dict(layers=2, hidden=256, kv_hidden=128, inter=512, q_heads=4, kv_heads=2, head_dim=64, vocab=96, max_pos=16,
           eps=1e-5, fht_scale=float(np.sqrt(512.0)))


def rnd(t):
    """round half away from zero (std::round)"""
    return np.sign(t) * np.floor(np.abs(t) + 0.5)


def llama3_rope_tables(max_pos, head_dim=64, theta=500000.0, factor=32.0, low=1.0, high=4.0, orig=8192):
    """sin/cos tables from the rotary scaling published with Llama 3 (float64)."""
    inv_freq = 1.0 / theta ** (np.arange(0, head_dim, 2, dtype=np.float64) / head_dim)
    wl = 2 * np.pi / inv_freq
    scaled = np.where(wl > orig / low, inv_freq / factor, inv_freq)
    smooth = (orig / wl - low) / (high - low)
    mid = (1 - smooth) * inv_freq / factor + smooth * inv_freq
    inv = np.where((wl >= orig / high) & (wl <= orig / low), mid, scaled)
    ang = np.arange(max_pos, dtype=np.float64)[:, None] * inv[None, :]
    return np.sin(ang), np.cos(ang)


def make_weights(cfg, seed, bits=8):
    """bits=8: W8A8 symmetric weights; bits=4: int4 weights in [-8,7] with the row sums of the dequantised rows."""
    r = np.random.default_rng(seed)
    L, H, KV, I = cfg["layers"], cfg["hidden"], cfg["kv_hidden"], cfg["inter"]
    dims = dict(q=(H, H), k=(KV, H), v=(KV, H), o=(H, H), g=(I, H), u=(I, H), d=(H, I))
    w = {}
    lo, hi, amp = (-127, 128, 73.0) if bits == 8 else (-8, 8, 4.6)
    for p, (n, k) in dims.items():
        w["w" + p] = [r.integers(lo, hi, (n, k)).astype(np.int8) for _ in range(L)]
        w["s" + p] = [(r.uniform(0.5, 1.5, n) / (amp * np.sqrt(k))).astype(np.float32) for _ in range(L)]
        w["sum" + p] = [(w["w" + p][l].sum(1, dtype=np.int64).astype(np.float64) * w["s" + p][l]).astype(np.float32)
                        for l in range(L)]
    w["gamma"] = r.uniform(0.5, 1.5, (2 * L + 1, H)).astype(np.float32)
    w["q_s"] = (r.uniform(0.8, 1.2, (L, cfg["q_heads"])) * 0.004).astype(np.float32)
    w["k_s"] = (r.uniform(0.8, 1.2, (L, cfg["kv_heads"])) * 0.03).astype(np.float32)
    w["v_s"] = (r.uniform(0.8, 1.2, (L, cfg["kv_heads"])) * 0.03).astype(np.float32)
    w["a_s"] = (r.uniform(0.9, 1.1, (L, cfg["q_heads"])) / 255).astype(np.float32)
    w["embed"] = r.uniform(-0.5, 0.5, (cfg["vocab"], H)).astype(np.float16).view(np.uint16)
    return w


# ------------------------------------------------------------------ the float64 restatement
def lin_w8a8(x, wq, ws):
    """per-token symmetric int8 fake quant, float matmul of the dequantised operands"""
    s = np.abs(x).max(1, keepdims=True) / 127.0
    s[s == 0] = 1.0
    return (rnd(x / s) * s) @ (wq.astype(np.float64) * ws.astype(np.float64)[:, None]).T


def lin_w4a4(x, wq, ws):
    """per-token asymmetric uint4 fake quant (scale + zero point = row minimum), as Linear_Layer_Decoding_tb.cpp:137-152"""
    mn = x.min(1, keepdims=True)
    s = (x.max(1, keepdims=True) - mn) / 15.0
    s[s == 0] = 1.0
    return (rnd((x - mn) / s) * s + mn) @ (wq.astype(np.float64) * ws.astype(np.float64)[:, None]).T


def ref_layer(cfg, w, l, x, pos0, kc, vc, sin_t, cos_t, lin=lin_w8a8, mut=None):
    """One decoder layer on S tokens at positions pos0.. with the layer's token-major int8 caches kc, vc
    ([max_pos][kv_hidden], float64 holding integers), updated in place.  Token i attends to positions 0..pos0+i."""
    S, H = x.shape
    qh, kvh, hd = cfg["q_heads"], cfg["kv_heads"], cfg["head_dim"]
    half = hd // 2
    g_row0, g_row1 = 2 * l, 2 * l + 1
    if mut == "gamma_swapped":
        g_row0, g_row1 = g_row1, g_row0
    if mut == "gamma_by_layer":
        g_row0, g_row1 = l, l + 1

    def rms(t, row):
        return t / np.sqrt((t * t).mean(1, keepdims=True) + cfg["eps"]) * w["gamma"][row].astype(np.float64)

    def rope(t, heads):
        t = t.reshape(S, heads, hd)
        sn = sin_t[pos0:pos0 + S, None, :]; cs = cos_t[pos0:pos0 + S, None, :]
        if mut == "rope_position_0":
            sn = sin_t[0:S, None, :]; cs = cos_t[0:S, None, :]
        if mut == "rope_interleaved":
            a, b = t[..., 0::2], t[..., 1::2]
            out = np.empty_like(t)
            out[..., 0::2] = a * cs - b * sn; out[..., 1::2] = a * sn + b * cs
            return out
        a, b = t[..., :half], t[..., half:]
        return np.concatenate([a * cs - b * sn, a * sn + b * cs], axis=-1)

    n0 = rms(x, g_row0)
    q = rope(lin(n0, w["wq"][l], w["sq"][l]), qh)
    k = rope(lin(n0, w["wk"][l], w["sk"][l]), kvh)
    v = lin(n0, w["wv"][l], w["sv"][l]).reshape(S, kvh, hd)
    if mut == "v_roped":
        v = rope(v.reshape(S, -1), kvh)
    q_s, k_s, v_s, a_s = [w[n][l].astype(np.float64) for n in ("q_s", "k_s", "v_s", "a_s")]
    q_div = q_s if mut == "q_without_sqrt_d" else np.sqrt(hd) * q_s
    q8 = np.clip(rnd(q / q_div[None, :, None]), -128, 127)
    kc[pos0:pos0 + S] = np.clip(rnd(k / k_s[None, :, None]), -128, 127).reshape(S, -1)
    vc[pos0:pos0 + S] = np.clip(rnd(v / v_s[None, :, None]), -128, 127).reshape(S, -1)
    att = np.zeros((S, qh, hd))
    for h in range(qh):
        kh = h // (qh // kvh)
        if mut == "gqa_modulo":
            kh = h % kvh
        for i in range(S):
            n_keys = pos0 + i + 1
            if mut == "no_causal_mask":
                n_keys = pos0 + S
            keys = kc[:n_keys].reshape(n_keys, kvh, hd)[:, kh]
            vals = vc[:n_keys].reshape(n_keys, kvh, hd)[:, kh]
            p = scipy.special.softmax((q8[i, h] * q_s[h]) @ (keys * k_s[kh]).T)
            p8 = np.minimum(127 if mut == "p_signed" else 255, rnd(p / a_s[h]))
            att[i, h] = (p8 * a_s[h]) @ (vals * v_s[kh])
    ao = lin(att.reshape(S, H), w["wo"][l], w["so"][l])
    res0 = ao if mut == "no_residual_0" else ao + x
    n1 = rms(res0, g_row1)
    g = lin(n1, w["wg"][l], w["sg"][l])
    u = lin(n1, w["wu"][l], w["su"][l])
    if mut == "gate_up_swapped":
        g, u = u, g
    hmid = g * scipy.special.expit(g) * u
    if mut != "no_hadamard":
        hmid = hmid @ scipy.linalg.hadamard(cfg["inter"]).astype(np.float64).T
        if mut != "hadamard_unscaled":
            hmid = hmid / cfg["fht_scale"]
    d = lin(hmid, w["wd"][l], w["sd"][l])
    return d if mut == "no_residual_1" else d + res0


def ref_model(cfg, w, x, pos0, kcs, vcs, sin_t, cos_t, lin=lin_w8a8, mut=None, want_logits=False):
    x = np.asarray(x, np.float64)
    for l in range(cfg["layers"]):
        kc, vc = (kcs[0], vcs[0]) if mut == "cache_layer_0_only" else (kcs[l], vcs[l])
        x = ref_layer(cfg, w, l, x, pos0, kc, vc, sin_t, cos_t, lin, mut)
    if not want_logits:
        return x
    row = 2 * cfg["layers"] - 1 if mut == "final_gamma_row" else 2 * cfg["layers"]
    n = x / np.sqrt((x * x).mean(1, keepdims=True) + cfg["eps"]) * w["gamma"][row].astype(np.float64)
    return x, n @ w["embed"].view(np.float16).astype(np.float64).T


MUTANTS = ["gamma_swapped", "gamma_by_layer", "rope_interleaved", "v_roped", "q_without_sqrt_d", "gqa_modulo",
           "p_signed", "no_residual_0", "no_residual_1", "gate_up_swapped", "no_hadamard", "hadamard_unscaled",
           "cache_layer_0_only"]


def rel(a, b):
    return np.abs(a - b).max() / np.abs(b).max()


@pytest.fixture(scope="module")
def setup(oracle):
    cfg = CFG
    w = make_weights(cfg, 7)
    sin64, cos64 = llama3_rope_tables(cfg["max_pos"], cfg["head_dim"])
    sin32, cos32 = oracle.rope_table(cfg["max_pos"], cfg["head_dim"])
    ow = dict(w); ow["rope_sin"], ow["rope_cos"] = sin32, cos32
    return cfg, w, oracle.OracleModel(cfg, ow), sin64, cos64


def test_decode_token_graph_against_float64_restatement(oracle, setup):
    """fxo_llama_decode_token, 2 layers, positions 0..5: hidden state, logits and both layers' cache rows."""
    cfg, w, om, sin64, cos64 = setup
    L, P, KV = cfg["layers"], cfg["max_pos"], cfg["kv_hidden"]
    r = np.random.default_rng(11)
    xs = r.standard_normal((6, cfg["hidden"])).astype(np.float32)
    kc, vc = om.new_caches()
    kr = np.zeros((L, P, KV)); vr = np.zeros((L, P, KV))
    km = {m: (np.zeros((L, P, KV)), np.zeros((L, P, KV))) for m in MUTANTS + ["rope_position_0", "final_gamma_row"]}
    for pos in range(6):
        hid, logits = om.decode_token(xs[pos], pos, kc, vc)
        ref_h, ref_l = ref_model(cfg, w, xs[pos:pos + 1], pos, kr, vr, sin64, cos64, want_logits=True)
        assert rel(hid, ref_h[0]) < 1e-3 and rel(logits, ref_l[0]) < 1e-3, pos
        assert np.array_equal(kc[:, :pos + 1], kr[:, :pos + 1]) and np.array_equal(vc[:, :pos + 1], vr[:, :pos + 1])
        assert not kc[:, pos + 1:].any()                         # nothing written beyond the current position
        if pos == 5:
            for m, (a, b) in km.items():
                for p in range(5):                               # the mutant shares the true history ...
                    a[:, p] = kr[:, p]; b[:, p] = vr[:, p]
                mh, ml = ref_model(cfg, w, xs[pos:pos + 1], pos, a, b, sin64, cos64, mut=m, want_logits=True)
                assert max(rel(hid, mh[0]), rel(logits, ml[0])) > 1e-2, "mutant %s is not detected" % m


def test_prefill_graph_against_float64_restatement(oracle, setup):
    """fxo_llama_prefill, 2 layers, 8 tokens, then a decode token on the caches the prefill left."""
    cfg, w, om, sin64, cos64 = setup
    L, P, KV = cfg["layers"], cfg["max_pos"], cfg["kv_hidden"]
    S = 8
    r = np.random.default_rng(12)
    x = r.standard_normal((S + 1, cfg["hidden"])).astype(np.float32)
    kc, vc = om.new_caches()
    hid = om.prefill(x[:S], kc, vc)
    kr = np.zeros((L, P, KV)); vr = np.zeros((L, P, KV))
    ref = ref_model(cfg, w, x[:S], 0, kr, vr, sin64, cos64)
    assert rel(hid, ref) < 1e-3
    assert np.array_equal(kc, kr) and np.array_equal(vc, vr)
    # (a prefill rewrites every cache row it reads, so the per-layer cache offset shows in the cache bytes above and in
    # the decode test, not in the prefill's hidden state)
    for m in [m for m in MUTANTS if m != "cache_layer_0_only"] + ["no_causal_mask"]:
        a = np.zeros((L, P, KV)); b = np.zeros((L, P, KV))
        assert rel(hid, ref_model(cfg, w, x[:S], 0, a, b, sin64, cos64, mut=m)) > 1e-2, "mutant %s is not detected" % m
    hid1, _ = om.decode_token(x[S], S, kc, vc, want_logits=False)
    ref1 = ref_model(cfg, w, x[S:S + 1], S, kr, vr, sin64, cos64)
    assert rel(hid1, ref1[0]) < 1e-3
    assert np.array_equal(kc, kr) and np.array_equal(vc, vr)


def test_w4a4_layer_against_float64_restatement(oracle):
    """oracle.w4a4_linear / oracle.w4a4_layer (the shipped uint4 x int4 configuration): prefill of 8 tokens and a
    decode token per layer, against the same restatement with the asymmetric 4-bit fake quant in the linears."""
    cfg = dict(CFG)
    w = make_weights(cfg, 9, bits=4)
    sin64, cos64 = llama3_rope_tables(cfg["max_pos"], cfg["head_dim"])
    ow = dict(w); ow["rope_sin"], ow["rope_cos"] = oracle.rope_table(cfg["max_pos"], cfg["head_dim"])
    r = np.random.default_rng(13)
    S = 8
    x = r.standard_normal((S + 1, cfg["hidden"])).astype(np.float32)
    # one linear on its own, zero point x row sum included
    y = oracle.w4a4_linear(x[:3], w["wq"][0], w["sq"][0], w["sumq"][0])
    assert rel(y, lin_w4a4(x[:3].astype(np.float64), w["wq"][0], w["sq"][0])) < 1e-5
    for l in range(cfg["layers"]):
        kc = np.zeros((cfg["max_pos"], cfg["kv_hidden"]), np.int8); vc = np.zeros_like(kc)
        kr = np.zeros(kc.shape); vr = np.zeros(kc.shape)
        out = oracle.w4a4_layer(cfg, ow, l, x[:S], 0, kc, vc)
        ref = ref_layer(cfg, w, l, x[:S].astype(np.float64), 0, kr, vr, sin64, cos64, lin=lin_w4a4)
        assert rel(out, ref) < 1e-3
        assert np.array_equal(kc, kr) and np.array_equal(vc, vr)
        for m in ["gamma_swapped", "rope_interleaved", "q_without_sqrt_d", "gqa_modulo", "no_residual_0",
                  "no_residual_1", "gate_up_swapped", "no_hadamard"]:
            a = np.zeros(kc.shape); b = np.zeros(kc.shape)
            mo = ref_layer(cfg, w, l, x[:S].astype(np.float64), 0, a, b, sin64, cos64, lin=lin_w4a4, mut=m)
            assert rel(out, mo) > 1e-2, "mutant %s is not detected" % m
        out1 = oracle.w4a4_layer(cfg, ow, l, x[S:S + 1], S, kc, vc)
        ref1 = ref_layer(cfg, w, l, x[S:S + 1].astype(np.float64), S, kr, vr, sin64, cos64, lin=lin_w4a4)
        assert rel(out1, ref1) < 1e-3
        assert np.array_equal(kc, kr) and np.array_equal(vc, vr)


# ------------------------------------------------------------------ the remaining one-liners
def test_static_dequant_maps_query_head_to_kv_head_by_integer_division(oracle):
    """fxo_static_dequant (quant.h:296-326, :758-805): y = acc * a_s[h] * w_s[h // (act_heads / w_heads)]."""
    r = np.random.default_rng(21)
    rows, ah, wh, dim = 3, 8, 2, 5
    acc = r.integers(-2**20, 2**20, (rows, ah, dim)).astype(np.int32)
    a_s = r.uniform(1e-3, 1e-2, ah).astype(np.float32)
    w_s = np.array([0.5, 3.0], np.float32)                       # very different, so a wrong head map cannot hide
    y = oracle.static_dequant(acc, a_s, w_s)
    for h in range(ah):
        exp = (acc[:, h].astype(np.float32) * a_s[h]).astype(np.float32) * w_s[h // 4]
        assert np.array_equal(y[:, h], exp.astype(np.float32)), h
    assert not np.array_equal(y[:, 1], (acc[:, 1].astype(np.float32) * a_s[1]).astype(np.float32) * w_s[1 % 2])
    # equal head counts: one scale per head
    w8 = r.uniform(1e-3, 1e-2, ah).astype(np.float32)
    y8 = oracle.static_dequant(acc, a_s, w8)
    assert np.array_equal(y8, ((acc.astype(np.float32) * a_s[None, :, None]).astype(np.float32) * w8[None, :, None]).astype(np.float32))


def test_head_quant_is_the_symmetric_quantiser_per_token_and_head(oracle):
    """fxo_head_quant_sym (quant.h:527-617): absmax over the 64 values of one (token, head), scale absmax/127, zero
    head -> scale 1, values rounded half away from zero."""
    r = np.random.default_rng(22)
    x = r.standard_normal((5, 4, 64)).astype(np.float32)
    x[2, 1] = 0.0
    x[3, 0, 7] = 40.0                                            # an outlier must only touch its own head's scale
    q, s = oracle.head_quant_sym(x)
    s_np = (np.abs(x).max(-1) / np.float32(127)).astype(np.float32)
    s_np[2, 1] = 1.0
    t = (x / s_np[..., None]).astype(np.float32)
    assert np.array_equal(s, s_np)
    assert np.array_equal(q, (np.sign(t) * np.floor(np.abs(t) + np.float32(0.5))).astype(np.int8))
    assert q[3, 0, 7] == 127 and np.abs(q[3, 1]).max() == 127 and not q[2, 1].any()


def test_argmax_takes_the_first_of_equal_maxima(oracle):
    import ctypes as C
    for x in ([1.0, 5.0, 5.0, 2.0], [-3.0, -3.0, -3.0], [0.0, -1.0, 7.0, 7.0, 7.0], [9.0]):
        a = np.array(x, np.float32)
        got = oracle.lib().fxo_argmax(a.ctypes.data_as(C.c_void_p), a.size)
        assert got == int(np.argmax(a))                          # numpy returns the first maximum
    r = np.random.default_rng(23)
    a = r.standard_normal(128256).astype(np.float32)
    assert oracle.lib().fxo_argmax(a.ctypes.data_as(C.c_void_p), a.size) == int(np.argmax(a))


def test_embed_is_the_fp16_row_widened(oracle):
    r = np.random.default_rng(24)
    table = r.standard_normal((40, 64)).astype(np.float16)
    table[3, :4] = [np.float16(6e-8), np.float16(-0.0), np.float16(65504), np.float16(1e-5)]   # subnormal, -0, max
    for tok in (0, 3, 39):
        assert np.array_equal(oracle.embed(table.view(np.uint16), tok), table[tok].astype(np.float32))
