"""W4A4 linear layers (asymmetric uint4 activations x symmetric int4 weights, two values per byte): the decode GEMV
and the prefill GEMM against the oracle, built the way the reference's Linear_Layer_*_tb.cpp builds its inputs."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

rng = np.random.default_rng(404)


@pytest.fixture(scope="module")
def fx():
    import flexllm_amd as fx
    fx.lib()
    return fx


def pack(values):
    v = np.asarray(values).astype(np.uint8) & 0xF
    return (v[..., 0::2] | (v[..., 1::2] << 4)).astype(np.uint8)


def quantise_weights_int4(w):
    """As Linear_Layer_Decoding_tb.cpp:160-190: per output channel scale = max|w|/7 (0 -> 1), q = clamp(round(w/s)),
    w_sum = running float32 sum of the dequantised weights."""
    scale = (np.abs(w).max(axis=1) / np.float32(7.0)).astype(np.float32)
    scale[scale == 0] = 1.0
    q = np.clip(np.round(w / scale[:, None]), -8, 7).astype(np.int8)
    deq = (q.astype(np.float32) * scale[:, None]).astype(np.float32)
    w_sum = np.zeros(w.shape[0], np.float32)
    for j in range(w.shape[1]):
        w_sum = (w_sum + deq[:, j]).astype(np.float32)
    return q, scale, w_sum, deq


def test_pack_nibbles(fx):
    v = rng.integers(-8, 8, (7, 64)).astype(np.int8)
    assert np.array_equal(fx.ops.pack_nibbles(fx.to_device(v)).numpy(), pack(v))
    u = rng.integers(0, 16, (3, 4096)).astype(np.uint8)
    assert np.array_equal(fx.ops.pack_nibbles(fx.to_device(u)).numpy(), pack(u))


@pytest.mark.parametrize("k,n", [(2048, 2048), (8192, 2048), (2048, 16384), (32, 1), (64, 33), (4096, 500)])
def test_gemv_u4i4_exact(fx, k, n):
    x = rng.integers(0, 16, k).astype(np.uint8)
    w = rng.integers(-8, 8, (n, k)).astype(np.int8)
    acc = fx.ops.linear_u4i4_gemv(fx.to_device(pack(x)), fx.to_device(pack(w))).numpy()
    assert np.array_equal(acc, w.astype(np.int32) @ x.astype(np.int32))
    # extremes: all 15 x all -8
    xe = np.full(k, 15, np.uint8); we = np.full((n, k), -8, np.int8)
    assert np.all(fx.ops.linear_u4i4_gemv(fx.to_device(pack(xe)), fx.to_device(pack(we))).numpy() == -120 * k)


@pytest.mark.parametrize("m,k,n", [(128, 64, 128), (160, 2048, 384), (1024, 2048, 2048), (33, 128, 257), (1, 64, 1)])
def test_gemm_u4i4_exact(fx, m, k, n):
    a = rng.integers(0, 16, (m, k)).astype(np.uint8)
    w = rng.integers(-8, 8, (n, k)).astype(np.int8)
    acc = fx.ops.linear_u4i4_gemm(fx.to_device(pack(a)), fx.to_device(pack(w))).numpy()
    assert np.array_equal(acc, a.astype(np.int32) @ w.astype(np.int32).T)


@pytest.mark.parametrize("m,k,n", [(1024, 2048, 8192), (1024, 8192, 2048), (1024, 2048, 2048), (160, 2048, 384), (96, 64, 132),
                                   (33, 128, 260), (1, 64, 4)])
def test_gemm_on_byte_held_operands_equals_the_packed_path(fx, oracle, m, k, n):
    """W4A4 values held one per byte on the direct-load kernel (every tile variant its launcher picks, ragged edges):
    bit for bit the oracle's dequantised product, hence the nibble-packed entry point's result too."""
    a = rng.integers(0, 16, (m, k)).astype(np.uint8)
    w = rng.integers(-8, 8, (n, k)).astype(np.int8)
    s_x = rng.uniform(0.05, 0.2, m).astype(np.float32); b_x = rng.uniform(-2, 0, m).astype(np.float32)
    w_s = rng.uniform(0.01, 0.05, n).astype(np.float32)
    w_sum = (w.sum(1, dtype=np.int64).astype(np.float32) * w_s).astype(np.float32)
    res = rng.standard_normal((m, n)).astype(np.float32)
    da, dw = fx.to_device(a), fx.to_device(w)
    dev = [fx.to_device(v) for v in (s_x, b_x, w_s, w_sum)]
    y = fx.ops.linear_i8_gemm_dequant_asym(da, dev[0], dev[1], dw, dev[2], dev[3]).numpy()
    y_res = fx.ops.linear_i8_gemm_dequant_asym(da, dev[0], dev[1], dw, dev[2], dev[3], residual=fx.to_device(res)).numpy()
    acc = a.astype(np.int32) @ w.astype(np.int32).T
    ref = oracle.dequant(acc, s_x, w_s, b_x=b_x, w_sum=w_sum)
    assert np.array_equal(y, ref)
    assert np.array_equal(y_res, oracle.residual(ref, res))
    if m * n <= 1024 * 2048:
        y_packed = fx.ops.linear_u4i4_gemm_dequant(fx.to_device(pack(a)), dev[0], dev[1], fx.to_device(pack(w)), dev[2], dev[3]).numpy()
        assert np.array_equal(y, y_packed)
    # the largest byte value the container admits, against the most negative weight
    a2 = np.full((m, k), 127, np.uint8); w2 = np.full((n, k), -128, np.int8)
    y2 = fx.ops.linear_i8_gemm_dequant_asym(fx.to_device(a2), dev[0], dev[1], fx.to_device(w2), dev[2], dev[3]).numpy()
    assert np.array_equal(y2, oracle.dequant(np.full((m, n), -127 * 128 * k, np.int32), s_x, w_s, b_x=b_x, w_sum=w_sum))


@pytest.mark.parametrize("m,k,n", [(1024, 2048, 8192), (512, 2048, 8192), (160, 2048, 192), (96, 64, 66), (32, 128, 2)])
def test_gate_up_with_swiglu_in_the_epilogue_equals_the_two_step_route(fx, oracle, m, k, n):
    """Gate/up projection of the W4A4 precision with SiLU(gate)*up in the GEMM epilogue (every tile variant its launcher
    picks: 256x256 at the prefill shape, 128x128, 64x64, ragged edges) against the dequantising GEMM on the same
    interleaved rows followed by the SwiGLU kernel: bit for bit; and the dequantised pairs against the oracle."""
    a = rng.integers(0, 16, (m, k)).astype(np.uint8)
    w = rng.integers(-8, 8, (2 * n, k)).astype(np.int8)                      # row 2i gate, row 2i+1 up
    s_x = rng.uniform(0.01, 0.04, m).astype(np.float32); b_x = rng.uniform(-0.3, 0, m).astype(np.float32)
    w_s = rng.uniform(0.01, 0.05, 2 * n).astype(np.float32)
    w_sum = (w.sum(1, dtype=np.int64).astype(np.float32) * w_s).astype(np.float32)
    da, dw = fx.to_device(a), fx.to_device(w)
    dev = [fx.to_device(v) for v in (s_x, b_x, w_s, w_sum)]
    h = fx.ops.linear_i8_gemm_swiglu_asym(da, dev[0], dev[1], dw, dev[2], dev[3]).numpy()
    y = fx.ops.linear_i8_gemm_dequant_asym(da, dev[0], dev[1], dw, dev[2], dev[3]).numpy()
    acc = a.astype(np.int32) @ w.astype(np.int32).T
    assert np.array_equal(y, oracle.dequant(acc, s_x, w_s, b_x=b_x, w_sum=w_sum))
    gate = np.ascontiguousarray(y[:, 0::2]); up = np.ascontiguousarray(y[:, 1::2])
    h2 = fx.ops.swiglu_f32(fx.to_device(gate), fx.to_device(up)).numpy()
    assert np.array_equal(h, h2)
    ref = up.astype(np.float64) * (gate.astype(np.float64) / (1.0 + np.exp(-gate.astype(np.float64))))
    assert np.abs(h - ref).max() <= 1e-6 * max(1.0, np.abs(ref).max())


@pytest.mark.parametrize("n,rows", [(8192, 96), (2048, 33), (1024, 5)])
def test_fht_with_asymmetric_quantisation_equals_the_two_step_route(fx, n, rows):
    """Hadamard transform + asymmetric uint4 (and uint8) quantisation in one kernel against the transform followed by
    the quantisation kernel: bytes, scales and minima bit for bit (the quotients by the transform's scale are correctly
    rounded in both, and the rounding of (v - min) / s through the reciprocal gives the division's integers)."""
    x = fx.to_device((rng.standard_normal((rows, n)) * rng.uniform(0.1, 3.0, (rows, 1))).astype(np.float32))
    scale = float(np.sqrt(n))
    y = fx.ops.fht_f32(x, scale)
    for bits in (4, 8):
        q2, s2, b2 = fx.ops.quant_asym_u8(y, bits=bits)
        q1, s1, b1 = fx.ops.fht_quant_asym_u8(x, scale, bits=bits)
        assert np.array_equal(s1.numpy(), s2.numpy()) and np.array_equal(b1.numpy(), b2.numpy())
        assert np.array_equal(q1.numpy(), q2.numpy())
        assert int(q1.numpy().max()) == (1 << bits) - 1 and int(q1.numpy().min()) == 0


def test_rmsnorm_with_asymmetric_quantisation(fx, oracle):
    """RMSNorm + asymmetric uint4 quantisation, one wave per row of 2048 values, against the oracle's norm and
    quantiser: scale and minimum to fp32 rounding (the kernel sums the squares in the model graphs' order), bytes equal
    but for single steps at rounding ties; and against the device's two-kernel route on the values that route produces."""
    rows, dim = 200, 2048
    x = (rng.standard_normal((rows, dim)) * rng.uniform(0.2, 4.0, (rows, 1))).astype(np.float32)
    gamma = rng.uniform(0.5, 1.5, dim).astype(np.float32)
    q, s, b = fx.ops.rmsnorm_quant_asym_u8(fx.to_device(x), fx.to_device(gamma))
    q, s, b = q.numpy(), s.numpy(), b.numpy()
    yn = oracle.rmsnorm_pref(x, gamma)
    qr, sr, br = oracle.quant_asym(yn, 4)
    assert np.abs(s - sr).max() <= 2e-6 * np.abs(sr).max() and np.abs(b - br).max() <= 2e-6 * np.abs(br).max()
    d = np.abs(q.astype(np.int32) - qr.astype(np.int32))
    assert d.max() <= 1 and (d != 0).mean() < 2e-3
    q2, s2, b2 = fx.ops.quant_asym_u8(fx.ops.rmsnorm_f32(fx.to_device(x), fx.to_device(gamma)), bits=4)
    d2 = np.abs(q.astype(np.int32) - q2.numpy().astype(np.int32))
    assert d2.max() <= 1 and (d2 != 0).mean() < 2e-3
    assert int(q.max()) == 15 and int(q.min()) == 0


def test_w4a4_layer_like_the_reference_testbench(fx, oracle):
    """quant (asym uint4) -> linear -> dequant with zero point, decode and prefill shapes: bit-exact against the oracle
    chain, and within the testbench's own 1e-2 criterion of the fake-quant golden (…_tb.cpp:215-236)."""
    m, k, n = 96, 2048, 2048
    x = rng.standard_normal((m, k)).astype(np.float32)
    wf = rng.standard_normal((n, k)).astype(np.float32)
    q_w, w_s, w_sum, w_deq = quantise_weights_int4(wf)
    res = rng.standard_normal((m, n)).astype(np.float32)
    # device: quantise, pack, multiply
    dq, ds, db = fx.ops.quant_asym_u8(fx.to_device(x), bits=4)
    a4 = fx.ops.pack_nibbles(dq)
    w4 = fx.to_device(pack(q_w))
    dws, dwsum = fx.to_device(w_s), fx.to_device(w_sum)
    y = fx.ops.linear_u4i4_gemm_dequant(a4, ds, db, w4, dws, dwsum).numpy()
    y_res = fx.ops.linear_u4i4_gemm_dequant(a4, ds, db, w4, dws, dwsum, residual=fx.to_device(res)).numpy()
    # oracle chain
    q_ref, s_ref, b_ref = oracle.quant_asym(x, bits=4)
    assert np.array_equal(dq.numpy(), q_ref)
    acc_ref = q_ref.astype(np.int32) @ q_w.astype(np.int32).T
    ref = oracle.dequant(acc_ref, s_ref, w_s, b_x=b_ref, w_sum=w_sum)
    assert np.array_equal(y, ref)
    assert np.array_equal(y_res, oracle.residual(ref, res))
    # decode path row by row
    a4_h, s_h, b_h = a4.numpy(), ds.numpy().reshape(-1), db.numpy().reshape(-1)
    for row in (0, 17, m - 1):
        yv = fx.ops.linear_u4i4_gemv_dequant(fx.to_device(a4_h[row]), fx.to_device(s_h[row:row + 1]), fx.to_device(b_h[row:row + 1]),
                                             w4, dws, dwsum).numpy()
        assert np.array_equal(yv, ref[row])
    # the testbench's criterion against the fake-quant golden (float matmul of the dequantised operands).  The
    # golden needs the fake-quantised input: x_fq = q*s + b
    x_fq = (q_ref.astype(np.float32) * s_ref[:, None] + b_ref[:, None]).astype(np.float32)
    gold = x_fq.astype(np.float64) @ w_deq.astype(np.float64).T
    big = np.abs(gold) > 1.0
    assert np.max(np.abs(y[big] - gold[big]) / np.abs(gold[big])) < 1e-2


def test_int4_lm_head_at_the_padded_vocabulary(fx, oracle):
    """The reference's output head: 131072 x 2048 int4 weights (vocabulary padded), asymmetric uint4 activation.
    Logits bit-exact against the oracle chain (quant -> exact integer product -> dequant with zero point x row sum),
    and the sampler on those logits picks the oracle's token."""
    vocab_pad, hidden = 131072, 2048
    r = np.random.default_rng(99)
    n_vec = r.standard_normal(hidden).astype(np.float32)
    q_w = r.integers(-8, 8, (vocab_pad, hidden)).astype(np.int8)
    w_s = r.uniform(1e-3, 1e-2, vocab_pad).astype(np.float32)
    w_sum = (q_w.sum(1, dtype=np.int64).astype(np.float32) * w_s).astype(np.float32)
    w4 = fx.to_device(pack(q_w))
    logits = fx.ops.lm_head_u4i4(fx.to_device(n_vec), w4, fx.to_device(w_s), fx.to_device(w_sum)).numpy()
    q_ref, s_ref, b_ref = oracle.quant_asym(n_vec[None, :], bits=4)
    acc = np.empty(vocab_pad, np.int32)
    xq = q_ref[0].astype(np.float32)
    for i in range(0, vocab_pad, 16384):                                  # fp32 BLAS is exact here (|sum| < 2^24)
        acc[i:i + 16384] = (q_w[i:i + 16384].astype(np.float32) @ xq).astype(np.int32)
    ref = oracle.dequant(acc[None, :], s_ref, w_s, b_x=b_ref, w_sum=w_sum)[0]
    assert np.array_equal(logits, ref)
    tok, idx, val, prob = fx.ops.sample_topk_f32(fx.to_device(logits), top_k=5, rand=0.37)
    tok_ref, idx_ref, val_ref, prob_ref = oracle.sample_topk(ref, top_k=5, rand=0.37)
    assert tok == tok_ref and np.array_equal(idx, idx_ref)


def test_generation_loop_with_int4_head(fx, oracle):
    """Host-sequenced generation (embedding -> layers -> final norm -> int4 head -> top-k sampling): first step against
    the oracle chain to the layer-graph tolerance, the whole loop deterministic and in range."""
    from flexllm_amd import llama
    cfg = llama.make_config(layers=2, vocab=4096, max_pos=256)
    host_w = llama.synth_weights(cfg, seed=21, device=False)
    model = llama.Llama(cfg, llama.synth_weights(cfg, seed=21, device=True))
    hidden, vocab_pad = cfg["hidden"], cfg["vocab"]          # every id the head can produce has an embedding row
    r = np.random.default_rng(5)
    q_w = r.integers(-8, 8, (vocab_pad, hidden)).astype(np.int8)
    w_s = r.uniform(1e-3, 1e-2, vocab_pad).astype(np.float32)
    w_sum = (q_w.sum(1, dtype=np.int64).astype(np.float32) * w_s).astype(np.float32)
    head = (fx.to_device(pack(q_w)), fx.to_device(w_s), fx.to_device(w_sum))
    rands = [0.11, 0.52, 0.93, 0.30, 0.76, 0.05]
    toks = model.generate_int4_head(77, 0, len(rands), rands, 5, head)
    model.check()
    assert len(toks) == len(rands) and all(0 <= t < vocab_pad for t in toks)
    # oracle chain for the first step
    om = oracle.OracleModel(cfg, host_w)
    kc, vc = om.new_caches()
    x = oracle.embed(host_w["embed"], 77)
    hid_ref, _ = om.decode_token(x, 0, kc, vc, want_logits=False)
    n_ref = oracle.rmsnorm_dec(hid_ref, host_w["gamma"][2 * cfg["layers"]])
    q_ref, s_ref, b_ref = oracle.quant_asym(n_ref[None, :], bits=4)
    acc = (q_w.astype(np.float32) @ q_ref[0].astype(np.float32)).astype(np.int32)
    logits_ref = oracle.dequant(acc[None, :], s_ref, w_s, b_x=b_ref, w_sum=w_sum)[0]
    tok_ref, idx_ref, _, prob_ref = oracle.sample_topk(logits_ref, top_k=5, rand=rands[0])
    assert toks[0] in idx_ref.tolist()                                    # a 4-bit rounding tie may reorder near-equal candidates
    # the loop is deterministic: a second model run from the same state gives the same ids
    model2 = llama.Llama(cfg, llama.synth_weights(cfg, seed=21, device=True))
    assert model2.generate_int4_head(77, 0, len(rands), rands, 5, head) == toks
    # an id without an embedding row (a head may carry padding rows beyond the vocabulary) is refused, not looked up
    with pytest.raises(ValueError, match="outside the embedding table"):
        model2.generate_int4_head(cfg["vocab"] + 3, 6, 1, [0.0], 1, head)
    model.close(); model2.close()
