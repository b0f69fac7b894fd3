"""Prefill side: int8 MFMA GEMM (exact), causal int8 attention and the whole prefill graph against the oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

rng = np.random.default_rng(77)


@pytest.fixture(scope="module")
def fx():
    import flexllm_amd as fx
    fx.lib()
    return fx


@pytest.mark.parametrize("m,k,n", [(128, 64, 128), (64, 128, 64), (256, 2048, 512), (1024, 2048, 512), (96, 192, 160),
                                   (1, 64, 1), (33, 64, 257), (512, 8192, 256)])
def test_gemm_int32_exact(fx, m, k, n):
    a = rng.integers(-128, 128, (m, k)).astype(np.int8)
    w = rng.integers(-128, 128, (n, k)).astype(np.int8)
    acc = fx.ops.linear_i8_gemm(fx.to_device(a), fx.to_device(w)).numpy()
    ref = a.astype(np.int32) @ w.astype(np.int32).T         # exact: |sum| < 2^31
    assert np.array_equal(acc, ref)


def test_gemm_down_projection_shape(fx, oracle):
    """1024 x 8192 -> 2048, the shape that takes 64x128 tiles with two k-groups per workgroup: raw int32 and the
    dequantised + residual epilogue.  float64 BLAS is exact here (|sum| < 2^31)."""
    m, k, n = 1024, 8192, 2048
    a = rng.integers(-128, 128, (m, k)).astype(np.int8)
    w = rng.integers(-128, 128, (n, k)).astype(np.int8)
    ref = (a.astype(np.float64) @ w.astype(np.float64).T).astype(np.int64).astype(np.int32)
    da, dw = fx.to_device(a), fx.to_device(w)
    assert np.array_equal(fx.ops.linear_i8_gemm(da, dw).numpy(), ref)
    s_x = rng.uniform(0.01, 0.02, m).astype(np.float32)
    w_s = rng.uniform(1e-3, 1e-2, n).astype(np.float32)
    res = rng.standard_normal((m, n)).astype(np.float32)
    y = fx.ops.linear_i8_gemm_dequant(da, fx.to_device(s_x), dw, fx.to_device(w_s), residual=fx.to_device(res)).numpy()
    assert np.array_equal(y, oracle.residual(oracle.dequant(ref, s_x, w_s), res))


def test_gemm_all_tile_shapes_and_extremes(fx):
    # 128x128 tiles (>= 512 workgroups), 64x128 and 64x64 paths; saturated operands
    for m, k, n in [(1024, 128, 8192), (512, 128, 4096), (256, 128, 256)]:
        a = rng.integers(-128, 128, (m, k)).astype(np.int8)
        w = rng.integers(-128, 128, (n, k)).astype(np.int8)
        assert np.array_equal(fx.ops.linear_i8_gemm(fx.to_device(a), fx.to_device(w)).numpy(),
                              a.astype(np.int32) @ w.astype(np.int32).T)
    a = np.full((64, 8192), -128, np.int8); w = np.full((64, 8192), -128, np.int8)
    assert np.all(fx.ops.linear_i8_gemm(fx.to_device(a), fx.to_device(w)).numpy() == 8192 * 128 * 128)


@pytest.mark.parametrize("m,k,n", [(4096, 2048, 2048), (2048, 128, 4096), (2000, 384, 4100), (3072, 256, 2048), (1024, 2048, 2048)])
def test_gemm_long_prefill_shapes(fx, oracle, m, k, n):
    """Shapes with 384..767 tiles of 128x128 (the o projection of a 4096-token prefill, shallow ones, a ragged one):
    the 128x128 variant with two stages of 128-byte rows; and the o projection of a 1024-token prefill (1024 x 2048 ->
    2048, the narrow-tile instance the layer graph runs at that length).  Raw int32 and dequantised + residual, float64 BLAS as the
    exact reference (|sum| < 2^31)."""
    a = rng.integers(-128, 128, (m, k)).astype(np.int8)
    w = rng.integers(-128, 128, (n, k)).astype(np.int8)
    ref = (a.astype(np.float64) @ w.astype(np.float64).T).astype(np.int64).astype(np.int32)
    da, dw = fx.to_device(a), fx.to_device(w)
    assert np.array_equal(fx.ops.linear_i8_gemm(da, dw).numpy(), ref)
    s_x = rng.uniform(0.01, 0.02, m).astype(np.float32); w_s = rng.uniform(1e-3, 1e-2, n).astype(np.float32)
    res = rng.standard_normal((m, n)).astype(np.float32)
    y = fx.ops.linear_i8_gemm_dequant(da, fx.to_device(s_x), dw, fx.to_device(w_s), residual=fx.to_device(res)).numpy()
    assert np.array_equal(y, oracle.residual(oracle.dequant(ref, s_x, w_s), res))


def test_gemm_dequant_residual_bit_exact(fx, oracle):
    m, k, n = 160, 2048, 384
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = rng.integers(-127, 128, (n, k)).astype(np.int8)
    w_s = rng.uniform(1e-3, 1e-2, n).astype(np.float32)
    res = rng.standard_normal((m, n)).astype(np.float32)
    q, s = fx.ops.quant_sym_i8(fx.to_device(x))
    y = fx.ops.linear_i8_gemm_dequant(q, s, fx.to_device(w), fx.to_device(w_s)).numpy()
    y_res = fx.ops.linear_i8_gemm_dequant(q, s, fx.to_device(w), fx.to_device(w_s), residual=fx.to_device(res)).numpy()
    q_ref, s_ref = oracle.quant_sym(x)
    ref = oracle.dequant(oracle.linear_i8(q_ref, w), s_ref, w_s)
    assert np.array_equal(y, ref)
    assert np.array_equal(y_res, oracle.residual(ref, res))
    # prefill GEMM row == decode GEMV of that row
    yv = fx.ops.linear_i8_gemv_dequant(fx.to_device(q_ref[5]), fx.to_device(s_ref[5:6]), fx.to_device(w), fx.to_device(w_s)).numpy()
    assert np.array_equal(yv, y[5])


@pytest.mark.parametrize("m,k,n", [(160, 2048, 384), (64, 128, 32), (1024, 2048, 8192), (33, 64, 6)])
def test_gemm_swiglu(fx, oracle, m, k, n):
    """Gate/up GEMM with SiLU(gate)*up in the epilogue: == dequant GEMM + gate layer on the device bit for bit, == the
    decode GEMV entry point row by row, and == the oracle up to the device's expf (<= 2 ulp -> 2e-6 relative)."""
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = rng.integers(-127, 128, (2 * n, k)).astype(np.int8)           # rows interleaved: 2i gate, 2i+1 up
    w_s = rng.uniform(1e-3, 1e-2, 2 * n).astype(np.float32)
    q, s = fx.ops.quant_sym_i8(fx.to_device(x))
    dw, dws = fx.to_device(w), fx.to_device(w_s)
    h = fx.ops.linear_i8_gemm_swiglu(q, s, dw, dws).numpy()
    assert h.shape == (m, n)
    gu = fx.ops.linear_i8_gemm_dequant(q, s, dw, dws).numpy()
    gate, up = np.ascontiguousarray(gu[:, 0::2]), np.ascontiguousarray(gu[:, 1::2])
    assert np.array_equal(h, fx.ops.swiglu_f32(fx.to_device(gate), fx.to_device(up)).numpy())
    q_ref, s_ref = oracle.quant_sym(x)
    gu_ref = oracle.dequant(oracle.linear_i8(q_ref, w), s_ref, w_s)
    np.testing.assert_allclose(h, oracle.gate(gu_ref[:, 1::2], oracle.swish(gu_ref[:, 0::2])), rtol=2e-6, atol=1e-30)
    for row in (0, m - 1):
        hv = fx.ops.linear_i8_gemv_swiglu(fx.to_device(q_ref[row]), fx.to_device(s_ref[row:row + 1]), dw, dws).numpy()
        assert np.array_equal(hv, h[row])


@pytest.mark.parametrize("m,qh,kvh,pos0", [(128, 32, 8, 0), (96, 8, 2, 64), (32, 4, 4, 0), (1024, 32, 8, 0)])
def test_gemm_qkv_rope_cache_fused(fx, oracle, m, qh, kvh, pos0):
    """q/k/v GEMM with RoPE + static quantisation + cache stores in the epilogue: int8 outputs bit-exact against the
    oracle's chain (linear -> dequant -> RoPE -> static quant) and against the unfused device entry points."""
    k, max_pos = 2048, 1280
    n = (qh + 2 * kvh) * 64
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = rng.integers(-127, 128, (n, k)).astype(np.int8)
    w_s = rng.uniform(1e-3, 3e-3, n).astype(np.float32)
    r = np.random.default_rng(11)
    q_s = r.uniform(0.02, 0.05, qh).astype(np.float32); k_s = r.uniform(0.1, 0.3, kvh).astype(np.float32)
    v_s = r.uniform(0.05, 0.2, kvh).astype(np.float32); a_s = np.full(qh, 1.0 / 255, np.float32)
    sin_t, cos_t = oracle.rope_table(max_pos)
    sc = fx.ops.Scales(q_s, k_s, v_s, a_s)
    q, s = fx.ops.quant_sym_i8(fx.to_device(x))
    dw, dws, dsin, dcos = fx.to_device(w), fx.to_device(w_s), fx.to_device(sin_t), fx.to_device(cos_t)
    kc, vc = fx.ops.kv_cache(kvh, max_pos)
    q8 = fx.ops.linear_i8_gemm_qkv_rope_cache(q, s, dw, dws, dsin, dcos, sc, kc, vc, qh, pos0=pos0).numpy()
    # oracle chain
    q_ref, s_ref = oracle.quant_sym(x)
    y = oracle.dequant(oracle.linear_i8(q_ref, w), s_ref, w_s)
    qf = oracle.rope(y[:, :qh * 64].reshape(m, qh, 64), sin_t, cos_t, pos0)
    kf = oracle.rope(y[:, qh * 64:(qh + kvh) * 64].reshape(m, kvh, 64), sin_t, cos_t, pos0)
    vf = np.ascontiguousarray(y[:, (qh + kvh) * 64:].reshape(m, kvh, 64))
    assert np.array_equal(q8, oracle.static_quant(qf, q_s, 8.0))
    k8_ref, v8_ref = oracle.static_quant(kf, k_s, 1.0), oracle.static_quant(vf, v_s, 1.0)
    kc_h, vc_h = kc.numpy(), vc.numpy()                       # [kvh][pos][64], [kvh][pos/64][64 ch][64 pos]
    assert np.array_equal(kc_h[:, pos0:pos0 + m, :], k8_ref.transpose(1, 0, 2))
    v_lin = vc_h.transpose(0, 1, 3, 2).reshape(kvh, max_pos, 64)
    assert np.array_equal(v_lin[:, pos0:pos0 + m, :], v8_ref.transpose(1, 0, 2))
    assert not kc_h[:, pos0 + m:, :].any() and not v_lin[:, pos0 + m:, :].any() and not kc_h[:, :pos0, :].any()
    # unfused device path
    yd = fx.ops.linear_i8_gemm_dequant(q, s, dw, dws).numpy()
    qd = fx.ops.rope_f32(fx.to_device(np.ascontiguousarray(yd[:, :qh * 64]).reshape(m, qh, 64)), dsin, dcos, pos0=pos0)
    assert np.array_equal(q8, fx.ops.static_quant_i8(qd, fx.to_device(q_s), 8.0).numpy())
    kd = fx.ops.rope_f32(fx.to_device(np.ascontiguousarray(yd[:, qh * 64:(qh + kvh) * 64]).reshape(m, kvh, 64)), dsin, dcos, pos0=pos0)
    kc2, vc2 = fx.ops.kv_cache(kvh, max_pos)
    fx.ops.kv_append_i8(kd, fx.to_device(np.ascontiguousarray(yd[:, (qh + kvh) * 64:]).reshape(m, kvh, 64)), kc2, vc2, sc, pos0)
    assert np.array_equal(kc_h, kc2.numpy()) and np.array_equal(vc_h, vc2.numpy())


def mha_scales(qh=32, kvh=8, seed=3):
    r = np.random.default_rng(seed)
    return (r.uniform(0.003, 0.005, qh).astype(np.float32), r.uniform(0.02, 0.04, kvh).astype(np.float32),
            r.uniform(0.02, 0.04, kvh).astype(np.float32), np.full(qh, 1.0 / 255, np.float32))


@pytest.mark.parametrize("s,qh,kvh", [(32, 4, 1), (64, 8, 2), (160, 32, 8), (256, 32, 8), (1024, 32, 8), (1088, 4, 1), (2048, 4, 1)])
def test_mha_prefill_vs_oracle(fx, oracle, s, qh, kvh):
    """Probability bytes and outputs against the oracle, up to the benchmark's 1024 tokens x 32/8 heads (every row kept
    in registers, `pf_attention_cached_kernel`) and, with fewer heads, rows of more than 1024 keys, which take the kernel
    that recomputes the scores in its second pass (`pf_attention_kernel`)."""
    hd = 64
    q_s, k_s, v_s, a_s = mha_scales(qh, kvh)
    q = rng.standard_normal((s, qh, hd)).astype(np.float32)
    k = rng.standard_normal((s, kvh, hd)).astype(np.float32)
    v = rng.standard_normal((s, kvh, hd)).astype(np.float32)
    ref = oracle.mha_prefill(q, k, v, q_s, k_s, v_s, a_s, want_p=True)
    sc = fx.ops.Scales(q_s, k_s, v_s, a_s)
    max_pos = ((s + 63) // 64) * 64
    kc, vc = fx.ops.kv_cache(kvh, max_pos)
    fx.ops.kv_append_i8(fx.to_device(k), fx.to_device(v), kc, vc, sc, 0)
    q8 = fx.ops.static_quant_i8(fx.to_device(q), fx.to_device(q_s), factor=8.0)
    assert np.array_equal(q8.numpy(), ref["q8"])
    assert np.array_equal(kc.numpy()[:, :s], ref["k8"].transpose(1, 0, 2))
    o, p8 = fx.ops.mha_i8_prefill(q8, kc, vc, sc, want_p=True)
    p = p8.numpy()
    d = np.abs(p.astype(np.int32) - ref["p8"].astype(np.int32))
    # rounding ties of p/A_s may fall either way (device exp, association of the row sum): one step, rare
    assert d.max() <= 1 and (d != 0).mean() < 2e-3
    assert not np.triu(p, 1).any()                                   # causal: nothing above the diagonal
    # the integer P.V stage is exact given the kernel's own probability bytes
    group = qh // kvh
    # (float64 matrix products of integers below 2^53: exact)
    acc = np.stack([p[h].astype(np.float64) @ ref["v8"][:, h // group].astype(np.float64) for h in range(qh)], axis=1)
    o_from_p = (acc.astype(np.float32) * a_s[None, :, None]) * np.repeat(v_s, group)[None, :, None]
    assert np.array_equal(o.numpy(), o_from_p.astype(np.float32))
    flips = d.sum(-1).T[:, :, None]                                   # [s][qh][1]
    tol = (a_s * np.repeat(v_s, group) * 128)[None, :, None]
    assert np.all(np.abs(o.numpy().astype(np.float64) - ref["o"]) <= 1e-6 * np.abs(ref["o"]) + flips * tol + 1e-9)


@pytest.mark.parametrize("s", [1024, 4096])
def test_mha_prefill_rows_equal_decode(fx, s):
    """Size-independent property at full size (1024 tokens and the maximum context 4096, 32/8 heads): prefill row i
    equals decode of query i against the first i+1 cache positions, in the probability bytes and hence bit for bit in
    the output, except where the two kernels' row sums differ in the last bit (a one-step probability flip)."""
    qh, kvh, hd = 32, 8, 64
    q_s, k_s, v_s, a_s = mha_scales(qh, kvh)
    sc = fx.ops.Scales(q_s, k_s, v_s, a_s)
    q8 = rng.integers(-128, 128, (s, qh, hd)).astype(np.int8)
    k8 = rng.integers(-40, 40, (s, kvh, hd)).astype(np.int8)
    v8 = rng.integers(-128, 128, (s, kvh, hd)).astype(np.int8)
    kc, vc = fx.ops.kv_cache(kvh, s)
    fx.ops.kv_store_i8(fx.to_device(k8), fx.to_device(v8), kc, vc, 0)
    o, _ = fx.ops.mha_i8_prefill(fx.to_device(q8), kc, vc, sc)
    oh = o.numpy()
    for i in (0, 31, 32, 500, s - 1):
        od, _ = fx.ops.mha_i8_decode(fx.to_device(q8[i]), kc, vc, sc, i + 1)
        tol = (a_s * np.repeat(v_s, qh // kvh) * 128 * 2)[:, None]
        assert np.all(np.abs(od.numpy() - oh[i]) <= 1e-6 * np.abs(oh[i]) + tol)
        assert (od.numpy() == oh[i]).mean() > 0.9


def token_errors(a, ref):
    """max |a-ref| per token, relative to the tensor's own scale."""
    return np.abs(a - ref).max(axis=-1) / np.abs(ref).max()


def test_prefill_single_layer_is_exact_except_for_rounding_ties(fx):
    """One layer, 64 tokens.  Every integer stage is exact and the fp32 stages follow the reference's order
    except the row reductions (sum of squares, sum of exponentials) and exp itself; a token's result
    therefore equals the oracle's to fp32 rounding unless one of its ~14k roundings to int8/uint8 sat on a
    tie, in which case one quantised value moves by one step (a probability byte: 1/255 of a V row)."""
    from flexllm_amd import llama, synth
    from oracle import oracle
    cfg = llama.make_config(layers=1, vocab=1024, max_pos=128)
    host_w = llama.synth_weights(cfg, seed=9, device=False)
    model = llama.Llama(cfg, llama.synth_weights(cfg, seed=9, device=True))
    om = oracle.OracleModel(cfg, host_w)
    s = 64
    x = synth.host_normal_f32((s, cfg["hidden"]), 321)
    hid = model.prefill_hidden(fx.to_device(x)).numpy()
    kc, vc = om.new_caches()
    hid_ref = om.prefill(x, kc, vc)
    err = token_errors(hid, hid_ref)
    assert np.median(err) <= 1e-6
    assert (err <= 1e-5).mean() >= 0.8, "tokens that are not exact to fp32 rounding: %s" % np.where(err > 1e-5)[0]
    assert err.max() <= 2e-2
    k_gpu, v_gpu = model.caches_token_major()
    for a, b in ((k_gpu, kc), (v_gpu, vc)):
        d = np.abs(a[:, :s].astype(np.int32) - b[:, :s].astype(np.int32))
        assert d.max() <= 1 and (d != 0).mean() < 1e-3
    model.close()


def test_prefill_graph_matches_oracle_and_feeds_decode(fx):
    """Two layers: a tie flipped in layer 0 perturbs layer 1's K/V for every later token, so the bound is the
    quantisation step's size, not fp32 rounding."""
    from flexllm_amd import llama, synth
    from oracle import oracle
    cfg = llama.make_config(layers=2, vocab=1024, max_pos=128)
    host_w = llama.synth_weights(cfg, seed=9, device=False)
    dev_w = llama.synth_weights(cfg, seed=9, device=True)
    model = llama.Llama(cfg, dev_w)
    om = oracle.OracleModel(cfg, host_w)
    s = 64
    x = synth.host_normal_f32((s, cfg["hidden"]), 321)
    hid = model.prefill_hidden(fx.to_device(x)).numpy()
    kc, vc = om.new_caches()
    hid_ref = om.prefill(x, kc, vc)
    err = token_errors(hid, hid_ref)
    assert err.max() <= 3e-2 and np.median(err) <= 1e-2
    k_gpu, v_gpu = model.caches_token_major()
    for a, b in ((k_gpu, kc), (v_gpu, vc)):
        d = np.abs(a[:, :s].astype(np.int32) - b[:, :s].astype(np.int32))
        assert d.max() <= 6 and (d != 0).mean() < 5e-2
        assert (d[0] != 0).mean() < 1e-3 and d[0].max() <= 1           # layer 0's cache: ties only
    # decode continues from the prefilled cache (teacher-forced with the GPU's own cache to isolate the step)
    k_tm, v_tm = model.caches_token_major()
    xt = synth.host_normal_f32((cfg["hidden"],), 322)
    h1, _ = model.decode_hidden(fx.to_device(xt), s)
    h1_ref, _ = om.decode_token(xt, s, k_tm.copy(), v_tm.copy(), want_logits=False)
    assert np.abs(h1.numpy() - h1_ref).max() <= 2e-2 * np.abs(h1_ref).max()
    model.close()


def test_full_size_prefill_prefix_invariance_and_decode_equivalence(fx):
    """The benchmark's model size (16 layers, hidden 2048, 32/8 heads, intermediate 8192), no oracle in the loop.
    (1) Causality: prefilling the first 128 tokens gives bit for bit the first 128 rows (residual stream and caches of
    all 16 layers) of prefilling 256 - a row never depends on later rows, whatever tile shapes the longer run picks.
    (2) Prefill against token-by-token decode of the same embeddings: token 0 (a one-key context has no rounding
    ties) agrees through all 16 layers to fp32 rounding, layer 0's caches agree for every token, layer 1's up to
    the ties of layer 0.  Deeper layers are not compared: with random weights a flipped quantisation step grows by
    two orders of magnitude per layer (0.4 % of layer 1's cache bytes differ by one step, 37 % of layer 2's)."""
    from flexllm_amd import llama, synth
    cfg = llama.make_config(vocab=4096, max_pos=512)                  # the table size does not enter the layer stack
    assert cfg["layers"] == 16 and cfg["hidden"] == 2048 and cfg["inter"] == 8192
    dev_w = llama.synth_weights(cfg, seed=41, device=True)
    pre, dec = llama.Llama(cfg, dev_w), llama.Llama(cfg, dev_w)
    s, H = 256, cfg["hidden"]
    x = synth.device_uniform_f32((s, H), 4100, -1.7, 1.7)
    hid_half = pre.prefill_hidden(x.view(0, (s // 2, H), np.float32)).numpy()
    k_half, v_half = pre.caches_token_major()
    pre.k_cache.zero_(); pre.v_cache.zero_()
    hid_p = pre.prefill_hidden(x).numpy()
    kp, vp = pre.caches_token_major()
    assert np.array_equal(hid_p[:s // 2], hid_half)
    assert np.array_equal(kp[:, :s // 2], k_half[:, :s // 2]) and np.array_equal(vp[:, :s // 2], v_half[:, :s // 2])
    assert not k_half[:, s // 2:].any() and not kp[:, s:].any() and not vp[:, s:].any()      # nothing past the sequence
    hid_d = np.empty_like(hid_p)
    for i in range(s):
        h, _ = dec.decode_hidden(x.view(i * H * 4, (H,), np.float32), i)
        hid_d[i] = h.numpy()
    dec.check()
    kd, vd = dec.caches_token_major()
    assert np.abs(hid_p[0] - hid_d[0]).max() <= 1e-5 * np.abs(hid_d[0]).max()                 # token 0, all 16 layers
    assert np.array_equal(kp[:, 0], kd[:, 0]) and np.array_equal(vp[:, 0], vd[:, 0])
    for a, b in ((kp, kd), (vp, vd)):
        d = np.abs(a[:, :s].astype(np.int32) - b[:, :s].astype(np.int32))
        assert (d[0] != 0).mean() < 1e-3 and d[0].max() <= 1          # layer 0: ties only
        assert (d[1] != 0).mean() < 2e-2 and d[1].max() <= 3          # layer 1 inherits layer 0's flipped steps
    pre.close(); dec.close()


@pytest.mark.parametrize("s,qh,kvh,spread,a_div", [(288, 6, 2, 3.0, 255.0), (544, 2, 2, 1.0, 255.0), (800, 6, 2, 2.0, 100.0),
                                                   (1056, 2, 2, 3.0, 255.0), (1536, 4, 1, 2.0, 100.0)])
def test_mha_prefill_other_shapes(fx, oracle, s, qh, kvh, spread, a_div):
    """Lengths that are not multiples of 64 or of the eight-tile deal (row blocks with idle waves, a last cache block
    half full), head groupings of 3 and 1 query heads per KV head, a probability scale other than 1/255 and wider
    scores, on both attention kernels: probability bytes against the oracle, the output as the exact product of the
    reported bytes with V, and the instance that does not report the bytes against the one that does."""
    r = np.random.default_rng(4000 + s)
    q = (r.standard_normal((s, qh, 64)) * spread).astype(np.float32)
    k = r.standard_normal((s, kvh, 64)).astype(np.float32)
    v = r.standard_normal((s, kvh, 64)).astype(np.float32)
    q_s, k_s, v_s, _ = mha_scales(qh, kvh, seed=s)
    q_s = (q_s * spread).astype(np.float32)
    a_s = np.full(qh, 1.0 / a_div, np.float32)
    ref = oracle.mha_prefill(q, k, v, q_s, k_s, v_s, a_s, want_p=True)
    sc = fx.ops.Scales(q_s, k_s, v_s, a_s)
    kc, vc = fx.ops.kv_cache(kvh, (s + 63) // 64 * 64)
    fx.ops.kv_append_i8(fx.to_device(k), fx.to_device(v), kc, vc, sc, 0)
    q8 = fx.ops.static_quant_i8(fx.to_device(q), fx.to_device(q_s), factor=8.0)
    assert np.array_equal(q8.numpy(), ref["q8"])
    o, p8 = fx.ops.mha_i8_prefill(q8, kc, vc, sc, want_p=True)
    o2, _ = fx.ops.mha_i8_prefill(q8, kc, vc, sc, want_p=False)
    p = p8.numpy()
    d = np.abs(p.astype(np.int32) - ref["p8"].astype(np.int32))
    assert d.max() <= 1 and (d != 0).mean() < 1e-4
    group = qh // kvh
    acc = np.stack([p[h].astype(np.float64) @ ref["v8"][:, h // group].astype(np.float64) for h in range(qh)], axis=1)
    o_from_p = (acc.astype(np.float32) * a_s[None, :, None]) * np.repeat(v_s, group)[None, :, None]
    assert np.array_equal(o.numpy(), o_from_p.astype(np.float32))
    assert np.array_equal(o2.numpy(), o.numpy())


@pytest.mark.parametrize("s", [1088, 1024], ids=["rows over 1024 keys", "rows up to 1024 keys"])
@pytest.mark.parametrize("case", ["wide scores", "tiny scales", "peaky rows"])
def test_mha_prefill_long_rows_fast_and_exact_paths(fx, oracle, case, s):
    """Rows of more than 1024 keys (`pf_attention_kernel`) and of up to 1024 keys (`pf_attention_cached_kernel`, whose
    row blocks of more than 256 keys take the fast probabilities) where the fast path is under strain or
    switched off: scores spread over +-25 (large |max|: the widest window), scales so small that the kernel takes the
    reference's expression for every probability (Q_s K_s log2 e < 2e-5), and rows dominated by one key (the factor
    255/sum at its largest).  Same criteria as test_mha_prefill_vs_oracle; the output must be the product of the
    probability bytes the kernel reports with V, bit for bit (this is what ties the groups that are put right after
    the main loop to the accumulators), and the instance that does not report the bytes must give the same output."""
    qh, kvh, hd = 4, 1, 64
    r = np.random.default_rng({"wide scores": 31, "tiny scales": 32, "peaky rows": 33}[case])
    q = r.standard_normal((s, qh, hd)).astype(np.float32)
    k = r.standard_normal((s, kvh, hd)).astype(np.float32)
    v = r.standard_normal((s, kvh, hd)).astype(np.float32)
    q_s, k_s, v_s, a_s = mha_scales(qh, kvh)
    if case == "wide scores":
        q *= 6.0
        q_s = (q_s * 6.0).astype(np.float32)
    elif case == "tiny scales":
        q_s = np.full(qh, 2e-5, np.float32); k_s = np.full(kvh, 0.05, np.float32)
        q *= 0.005
    else:
        k[::97] *= 6.0                                            # a few keys that take nearly all of a row
    ref = oracle.mha_prefill(q, k, v, q_s, k_s, v_s, a_s, want_p=True)
    sc = fx.ops.Scales(q_s, k_s, v_s, a_s)
    kc, vc = fx.ops.kv_cache(kvh, s)
    fx.ops.kv_append_i8(fx.to_device(k), fx.to_device(v), kc, vc, sc, 0)
    q8 = fx.ops.static_quant_i8(fx.to_device(q), fx.to_device(q_s), factor=8.0)
    assert np.array_equal(q8.numpy(), ref["q8"])
    o, p8 = fx.ops.mha_i8_prefill(q8, kc, vc, sc, want_p=True)
    p = p8.numpy()
    d = np.abs(p.astype(np.int32) - ref["p8"].astype(np.int32))
    print(case, "probability bytes off by one:", int((d != 0).sum()), "of", int(s * (s + 1) // 2 * qh), "largest byte", int(ref["p8"].max()), flush=True)
    assert d.max() <= 1 and (d != 0).mean() < 1e-4
    group = qh // kvh
    acc = np.stack([p[h].astype(np.float64) @ ref["v8"][:, h // group].astype(np.float64) for h in range(qh)], axis=1)
    o_from_p = (acc.astype(np.float32) * a_s[None, :, None]) * np.repeat(v_s, group)[None, :, None]
    assert np.array_equal(o.numpy(), o_from_p.astype(np.float32))
    o2, _ = fx.ops.mha_i8_prefill(q8, kc, vc, sc, want_p=False)
    assert np.array_equal(o2.numpy(), o.numpy())
