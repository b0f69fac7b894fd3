"""Parity of the HIP operators (through the C ABI) against the CPU oracle on identical seeded inputs.
Integer/byte results must match bit for bit; fp32 tolerances are written at each check."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

rng = np.random.default_rng(20251125)


@pytest.fixture(scope="module")
def fx():
    import flexllm_amd as fx
    fx.lib()
    print("device:", fx.device.device_name(), flush=True)
    return fx


def outliers(x, frac=0.01, mult=20.0, seed=7):
    """1% of the channels (fixed, seeded) scaled x20, as in the SpinQuant rotation workload."""
    r = np.random.default_rng(seed)
    ch = r.choice(x.shape[-1], max(1, int(frac * x.shape[-1])), replace=False)
    x = x.copy()
    x[..., ch] *= mult
    return x


# ------------------------------------------------------------------ synthetic fills
def test_device_fill_equals_host_fill(fx):
    from flexllm_amd import synth
    n = 100003
    assert np.array_equal(synth.device_i8((n,), 42).numpy(), synth.host_i8((n,), 42))
    assert np.array_equal(synth.device_i8((n,), 43, -8, 7).numpy(), synth.host_i8((n,), 43, -8, 7))
    assert np.array_equal(synth.device_uniform_f32((n,), 44, 1e-3, 1e-2).numpy(), synth.host_uniform_f32((n,), 44, 1e-3, 1e-2))
    assert np.array_equal(synth.device_uniform_f16((n,), 45, -0.05, 0.05).numpy().view(np.uint16),
                          synth.host_uniform_f16((n,), 45, -0.05, 0.05).view(np.uint16))


# ------------------------------------------------------------------ quant.h
@pytest.mark.parametrize("rows,dim", [(1, 2048), (1, 8192), (64, 2048), (33, 8192), (5, 64), (3, 1028), (2, 16384), (0, 2048)])
def test_quant_sym_bit_exact(fx, oracle, rows, dim):
    x = outliers(rng.standard_normal((rows, dim)).astype(np.float32)) if rows else np.zeros((0, dim), np.float32)
    if rows > 2:
        x[1] = 0.0                       # all-zero row -> scale 1
        x[2, 5:] = 0.0                   # nearly empty row
    q, s = fx.ops.quant_sym_i8(fx.to_device(x))
    q_ref, s_ref = oracle.quant_sym(x)
    assert np.array_equal(s.numpy().reshape(-1)[:rows], s_ref.reshape(-1))
    assert np.array_equal(q.numpy(), q_ref)


def test_quant_sym_ties_and_near_ties(fx, oracle):
    """The kernels quantise with x * (1/s) and fall back to the exact x / s near a tie: rows built so that most
    values sit on, or a few ulps beside, a rounding tie (k + 0.5) * s, for power-of-two and arbitrary scales."""
    r = np.random.default_rng(123)
    rows = []
    for s in [1.0, 0.5, 3.0 / 127, 1e-3, 7.77e-2, 123.456, float(np.float32(1.0) / np.float32(255.0))] + list(r.uniform(1e-4, 10, 9)):
        s = np.float32(s)
        k = np.arange(-126, 127, dtype=np.float32)
        base = ((k + np.float32(0.5)) * s).astype(np.float32)
        vals = [base]
        for step in (1, 2, 3, 8, 40):
            up, dn = base.copy(), base.copy()
            for _ in range(step):
                up = np.nextafter(up, np.float32(np.inf)); dn = np.nextafter(dn, np.float32(-np.inf))
            vals += [up, dn]
        row = np.concatenate(vals + [r.uniform(-126, 126, 2048).astype(np.float32) * s])
        row = np.concatenate([row, [np.float32(127.0) * s]])            # pins absmax, hence the scale, to 127*s/127
        rows.append(row.astype(np.float32))
    dim = max(len(x) for x in rows)
    dim += (-dim) % 4
    x = np.zeros((len(rows), dim), np.float32)
    for i, row in enumerate(rows):
        x[i, :len(row)] = row
    q, s_out = fx.ops.quant_sym_i8(fx.to_device(x))
    q_ref, s_ref = oracle.quant_sym(x)
    assert np.array_equal(s_out.numpy().reshape(-1), s_ref.reshape(-1))
    assert np.array_equal(q.numpy(), q_ref)
    # and a bulk check: 4M values over 256 scales
    xb = (r.standard_normal((256, 16384)) * r.uniform(1e-3, 50, (256, 1))).astype(np.float32)
    qb, _ = fx.ops.quant_sym_i8(fx.to_device(xb))
    assert np.array_equal(qb.numpy(), oracle.quant_sym(xb)[0])


@pytest.mark.parametrize("bits", [4, 8])
def test_quant_asym_bit_exact(fx, oracle, bits):
    x = rng.uniform(-1, 1, (17, 2048)).astype(np.float32)
    x[3] = 0.25                          # constant row -> scale 1
    q, s, b = fx.ops.quant_asym_u8(fx.to_device(x), bits)
    q_ref, s_ref, b_ref = oracle.quant_asym(x, bits)
    assert np.array_equal(s.numpy(), s_ref) and np.array_equal(b.numpy(), b_ref)
    assert np.array_equal(q.numpy(), q_ref)


def test_dequant_bit_exact(fx, oracle):
    acc = rng.integers(-2**27, 2**27, (9, 2048)).astype(np.int32)
    s_x = rng.uniform(1e-3, 1e-1, 9).astype(np.float32)
    w_s = rng.uniform(1e-3, 1e-2, 2048).astype(np.float32)
    y = fx.ops.dequant_i32_f32(fx.to_device(acc), fx.to_device(s_x), fx.to_device(w_s))
    assert np.array_equal(y.numpy(), oracle.dequant(acc, s_x, w_s))
    b_x = rng.uniform(-1, 1, 9).astype(np.float32)
    w_sum = rng.uniform(-3, 3, 2048).astype(np.float32)
    y = fx.ops.dequant_i32_f32(fx.to_device(acc), fx.to_device(s_x), fx.to_device(w_s), fx.to_device(b_x), fx.to_device(w_sum))
    assert np.array_equal(y.numpy(), oracle.dequant(acc, s_x, w_s, b_x, w_sum))


def test_static_quant_and_dequant_bit_exact(fx, oracle):
    x = (rng.standard_normal((40, 32, 64)) * 3).astype(np.float32)
    sc = rng.uniform(0.01, 0.05, 32).astype(np.float32)
    q = fx.ops.static_quant_i8(fx.to_device(x), fx.to_device(sc), factor=8.0)
    assert np.array_equal(q.numpy(), oracle.static_quant(x, sc, 8.0))
    q = fx.ops.static_quant_i8(fx.to_device(x), fx.to_device(sc), factor=1.0)      # saturates both ways
    ref = oracle.static_quant(x, sc, 1.0)
    assert ref.max() == 127 and ref.min() == -128 and np.array_equal(q.numpy(), ref)
    p = rng.uniform(0, 1.2, (7, 32, 128)).astype(np.float32)
    a_s = np.full(32, 1.0 / 255, np.float32)
    u = fx.ops.static_quant_i8(fx.to_device(p), fx.to_device(a_s), signed=False)
    assert np.array_equal(u.numpy(), oracle.static_quant(p, a_s, signed=False))
    acc = rng.integers(-2**20, 2**20, (7, 32, 64)).astype(np.int32)
    w_s = rng.uniform(0.01, 0.05, 8).astype(np.float32)
    y = fx.ops.static_dequant_i32_f32(fx.to_device(acc), fx.to_device(sc), fx.to_device(w_s))
    assert np.array_equal(y.numpy(), oracle.static_dequant(acc, sc, w_s))


def test_head_quant_bit_exact(fx, oracle):
    x = (rng.standard_normal((50, 8, 64)) * 2).astype(np.float32)
    x[3, 2] = 0
    q, s = fx.ops.head_quant_sym_i8(fx.to_device(x))
    q_ref, s_ref = oracle.head_quant_sym(x)
    assert np.array_equal(q.numpy(), q_ref) and np.array_equal(s.numpy(), s_ref)


# ------------------------------------------------------------------ Linear_Layer.h (decode)
@pytest.mark.parametrize("k,n", [(2048, 2048), (2048, 512), (2048, 8192), (8192, 2048), (256, 7), (16, 1), (4096, 33), (16384, 16)])
def test_gemv_int32_exact(fx, oracle, k, n):
    x = rng.integers(-128, 128, k).astype(np.int8)
    w = rng.integers(-128, 128, (n, k)).astype(np.int8)
    acc = fx.ops.linear_i8_gemv(fx.to_device(x), fx.to_device(w))
    assert np.array_equal(acc.numpy(), oracle.linear_i8(x[None, :], w)[0])


@pytest.mark.parametrize("m,k,n", [(1, 16, 1), (7, 48, 5), (100, 1024, 64), (33, 4096, 64), (1024, 1024, 64)])
def test_u8i8_gemm_int32_exact(fx, m, k, n):
    """MHA_i8xi8.h:286-345 (probabilities x V as a module of its own): unsigned 8-bit rows times signed 8-bit rows."""
    a = rng.integers(0, 256, (m, k)).astype(np.uint8)
    w = rng.integers(-128, 128, (n, k)).astype(np.int8)
    a[0, :] = 255; w[0, :] = -128                       # the extreme product, k * 255 * -128, in acc[0][0]
    acc = fx.ops.linear_u8i8_gemm(fx.to_device(a), fx.to_device(w)).numpy()
    ref = a.astype(np.int64) @ w.astype(np.int64).T
    assert np.array_equal(acc, ref.astype(np.int32)) and acc[0, 0] == -k * 255 * 128


def test_u8i8_gemm_rejects_a_ragged_inner_size(fx):
    a = fx.to_device(np.zeros((2, 24), np.uint8)); w = fx.to_device(np.zeros((3, 24), np.int8))
    from flexllm_amd._lib import FlexLLMError
    with pytest.raises(FlexLLMError, match="multiple of 16"):
        fx.ops.linear_u8i8_gemm(a, w)


def test_gemv_extreme_values_exact(fx):
    k, n = 8192, 64
    x = np.full(k, -128, np.int8); w = np.full((n, k), -128, np.int8)
    assert np.all(fx.ops.linear_i8_gemv(fx.to_device(x), fx.to_device(w)).numpy() == k * 128 * 128)


def test_config1_quant_gemv_dequant_bit_exact(fx, oracle):
    """x 1x2048 ~N(0,1) -> per-token int8; W 2048x2048 U[-127,127]; s_w U[1e-3,1e-2]; dequant to fp32."""
    from flexllm_amd import synth
    x = synth.host_normal_f32((1, 2048), 11)
    w = synth.host_i8((2048, 2048), 12)
    w_s = synth.host_uniform_f32((2048,), 13, 1e-3, 1e-2)
    q, s = fx.ops.quant_sym_i8(fx.to_device(x))
    res = rng.standard_normal(2048).astype(np.float32)
    y = fx.ops.linear_i8_gemv_dequant(q, s, fx.to_device(w), fx.to_device(w_s))
    y_res = fx.ops.linear_i8_gemv_dequant(q, s, fx.to_device(w), fx.to_device(w_s), residual=fx.to_device(res))
    q_ref, s_ref = oracle.quant_sym(x)
    ref = oracle.dequant(oracle.linear_i8(q_ref, w), s_ref, w_s)
    assert np.array_equal(y.numpy(), ref[0])
    assert np.array_equal(y_res.numpy(), oracle.residual(ref[0], res))
    # the reference testbench's own criterion: 1e-2 relative against the fake-quant float golden
    fq = (q_ref.astype(np.float64) * s_ref[:, None]) @ (w.astype(np.float64) * w_s[:, None]).T
    np.testing.assert_allclose(y.numpy(), fq[0], rtol=1e-2, atol=1e-4)


# ------------------------------------------------------------------ FHT.h
@pytest.mark.parametrize("n", [1024, 2048, 4096, 8192])
def test_fht_bit_exact(fx, oracle, n):
    x = outliers(rng.standard_normal((19, n)).astype(np.float32))
    scale = np.float32(90.50966799) if n == 8192 else np.float32(np.sqrt(n))
    y = fx.ops.fht_f32(fx.to_device(x), scale)
    assert np.array_equal(y.numpy(), oracle.fht(x, scale))
    q, s = fx.ops.fht_quant_i8(fx.to_device(x), scale)
    q_ref, s_ref = oracle.quant_sym(oracle.fht(x, scale))
    assert np.array_equal(s.numpy(), s_ref) and np.array_equal(q.numpy(), q_ref)


@pytest.mark.parametrize("n", [2048, 8192])
def test_fht_quant_division_paths(fx, oracle, n):
    """The fused transform + quantisation divides by the scale through a reciprocal with an exact residual step and
    falls back to the plain division outside the safe magnitude range: rows of ordinary, huge, tiny and mixed
    magnitude (and a zero row) must all give the oracle's bytes and scales."""
    base = rng.standard_normal((12, n)).astype(np.float32)
    mags = np.array([1.0, 1e-3, 1e3, 1e28, 3e32, 1e-15, 1e-22, 1e-30, 1.0, 1.0, 0.0, 1e10], np.float32)
    x = base * mags[:, None]
    x[8, ::3] *= np.float32(1e-26)            # a normal row with elements far below the safe range
    x[9, : n // 2] = 0.0
    scale = np.float32(90.50966799) if n == 8192 else np.float32(np.sqrt(n))
    q, s = fx.ops.fht_quant_i8(fx.to_device(x), scale)
    q_ref, s_ref = oracle.quant_sym(oracle.fht(x, scale))
    assert np.array_equal(s.numpy(), s_ref)
    assert np.array_equal(q.numpy(), q_ref)


def test_fht_config2_full_size_properties(fx, oracle):
    """1024 x 2048 and 1024 x 8192 with 1% outlier channels x20: spot rows against the oracle, all rows
    through size-independent properties (involution H(Hx)/n = x, Parseval, dequantised error bound)."""
    for n in (2048, 8192):
        x = outliers(rng.standard_normal((1024, n)).astype(np.float32))
        scale = np.float32(np.sqrt(n))
        dx = fx.to_device(x)
        y = fx.ops.fht_f32(dx, scale)
        yh = y.numpy()
        rows = [0, 1, 511, 1023]
        assert np.array_equal(yh[rows], oracle.fht(x[rows], scale))
        back = fx.ops.fht_f32(y, scale).numpy()
        np.testing.assert_allclose(back, x, atol=2e-4)
        np.testing.assert_allclose((yh.astype(np.float64) ** 2).sum(1), (x.astype(np.float64) ** 2).sum(1), rtol=1e-5)
        q, s = fx.ops.fht_quant_i8(dx, scale)
        qh, sh = q.numpy(), s.numpy()
        assert np.array_equal(sh, np.abs(yh).max(1) / np.float32(127))
        assert np.abs(qh).max(1).min() == 127
        assert np.all(np.abs(qh * sh[:, None] - yh) <= sh[:, None] * 0.50001)
        assert np.array_equal(qh[rows], oracle.quant_sym(yh[rows])[0])


# ------------------------------------------------------------------ LayerNorm.h
def test_rmsnorm_and_fused_quant(fx, oracle):
    x = (rng.standard_normal((48, 2048)) * 2).astype(np.float32)
    g = rng.uniform(0.5, 1.5, 2048).astype(np.float32)
    y = fx.ops.rmsnorm_f32(fx.to_device(x), fx.to_device(g)).numpy()
    # row sum of squares is associated differently from the reference's four running partial sums:
    # fp32 outputs agree to 1e-5 relative (bound stated for the path: 1e-3)
    np.testing.assert_allclose(y, oracle.rmsnorm_pref(x, g), rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(y[0], oracle.rmsnorm_dec(x[0], g, 8), rtol=1e-5, atol=1e-7)
    # the fused quantisation is exact with respect to the kernel's own fp32 normalised row
    q, s = fx.ops.rmsnorm_quant_i8(fx.to_device(x), fx.to_device(g))
    q_ref, s_ref = oracle.quant_sym(y)
    assert np.array_equal(q.numpy(), q_ref) and np.array_equal(s.numpy(), s_ref)


# ------------------------------------------------------------------ RoPE.h
def test_rope_table_and_rotation_bit_exact(fx, oracle):
    s, c = fx.ops.rope_table(4096)
    s_ref, c_ref = oracle.rope_table(4096)
    # host libm on both sides: identical
    assert np.array_equal(s, s_ref) and np.array_equal(c, c_ref)
    x = rng.standard_normal((37, 32, 64)).astype(np.float32)
    y = fx.ops.rope_f32(fx.to_device(x), fx.to_device(s), fx.to_device(c), pos0=1000)
    assert np.array_equal(y.numpy(), oracle.rope(x, s, c, 1000))
    y0 = fx.ops.rope_f32(fx.to_device(x[:1]), fx.to_device(s), fx.to_device(c), pos0=0)
    assert np.array_equal(y0.numpy(), x[:1])


# ------------------------------------------------------------------ Swish / gate / residual / softmax
def test_swish_swiglu_residual(fx, oracle):
    g = (rng.standard_normal((3, 8192)) * 4).astype(np.float32)
    u = rng.standard_normal((3, 8192)).astype(np.float32)
    # device expf vs glibc expf: <= 2 ulp on exp -> 1e-6 relative on the result
    np.testing.assert_allclose(fx.ops.swish_f32(fx.to_device(g)).numpy(), oracle.swish(g), rtol=2e-6, atol=1e-30)
    np.testing.assert_allclose(fx.ops.swiglu_f32(fx.to_device(g), fx.to_device(u)).numpy(),
                               oracle.gate(u, oracle.swish(g)), rtol=2e-6, atol=1e-30)
    assert np.array_equal(fx.ops.residual_add_f32(fx.to_device(g), fx.to_device(u)).numpy(), oracle.residual(g, u))


@pytest.mark.parametrize("dim", [1, 5, 64, 1023, 4096])
def test_softmax(fx, oracle, dim):
    x = (rng.standard_normal((6, dim)) * 4).astype(np.float32)
    if dim > 8:
        x[2, dim // 2:] = np.float32(-1e32)       # masked tail -> exact zeros
    y = fx.ops.softmax_f32(fx.to_device(x)).numpy()
    np.testing.assert_allclose(y, oracle.softmax(x), rtol=1e-5, atol=1e-12)
    if dim > 8:
        assert not y[2, dim // 2:].any()


# ------------------------------------------------------------------ MHA_i8xi8 decode
def mha_scales(qh=32, kvh=8, seed=3):
    r = np.random.default_rng(seed)
    return (r.uniform(0.02, 0.04, qh).astype(np.float32), r.uniform(0.02, 0.04, kvh).astype(np.float32),
            r.uniform(0.02, 0.04, kvh).astype(np.float32), np.full(qh, 1.0 / 255, np.float32))


def check_attention_output(o, p8, o_ref, p_ref, v8_abs_max, a_s, v_s, group):
    """P is compared exactly except on rounding ties of p/A_s (device expf and the association of the row
    sum differ in the last bits): |dP| <= 1 and rare.  O is then bounded by the P mismatches it inherits."""
    d = np.abs(p8.astype(np.int32) - p_ref.astype(np.int32))
    assert d.max() <= 1, "probability bytes differ by more than one step"
    assert (d != 0).mean() < 2e-3, "too many probability bytes differ: %g" % (d != 0).mean()
    heads = o_ref.shape[-2]
    flips = d.reshape(heads, -1).sum(1) if d.ndim == 2 else d.sum(-1)       # per head (decode) / per (head,row)
    tol_h = np.array([a_s[h] * v_s[h // group] * v8_abs_max for h in range(heads)], np.float64)
    return flips, tol_h


@pytest.mark.parametrize("length", [1, 5, 64, 127, 128, 129, 1000, 4096])
def test_mha_decode_vs_oracle(fx, oracle, length):
    qh, kvh, hd = 32, 8, 64
    max_pos = ((length + 63) // 64) * 64 + 64
    q_s, k_s, v_s, a_s = mha_scales()
    q8 = rng.integers(-128, 128, (qh, hd)).astype(np.int8)
    k8 = rng.integers(-60, 60, (length, kvh, hd)).astype(np.int8)
    v8 = rng.integers(-128, 128, (length, kvh, hd)).astype(np.int8)
    sc = fx.ops.Scales(q_s, k_s, v_s, a_s)
    kc, vc = fx.ops.kv_cache(kvh, max_pos)
    # poison the cache beyond `length`: positions past the end must not influence the result
    kc.copy_from(rng.integers(-128, 128, kc.shape).astype(np.int8))
    vc.copy_from(rng.integers(-128, 128, vc.shape).astype(np.int8))
    fx.ops.kv_store_i8(fx.to_device(k8), fx.to_device(v8), kc, vc, 0)
    o, p8 = fx.ops.mha_i8_decode(fx.to_device(q8), kc, vc, sc, length, want_p=True)
    o_ref, p_ref = oracle.mha_decode(q8, k8, v8, q_s, k_s, v_s, a_s, want_p=True)
    flips, tol_h = check_attention_output(o.numpy(), p8.numpy(), o_ref, p_ref, 128, a_s, v_s, qh // kvh)
    err = np.abs(o.numpy().astype(np.float64) - o_ref)
    assert np.all(err <= 1e-6 * np.abs(o_ref) + (flips * tol_h)[:, None] + 1e-9)
    # integer stage alone, from the oracle's own probability bytes: exact
    acc_ref = np.einsum("ht,thd->hd", p8.numpy().astype(np.int64), np.repeat(v8, qh // kvh, axis=1).astype(np.int64))
    o_from_p = (acc_ref.astype(np.float32) * a_s[:, None]) * np.repeat(v_s, qh // kvh)[:, None]
    assert np.array_equal(o.numpy(), o_from_p.astype(np.float32))


def test_kv_append_quantises_and_lays_out(fx, oracle):
    kvh, hd, max_pos = 8, 64, 256
    q_s, k_s, v_s, a_s = mha_scales()
    sc = fx.ops.Scales(q_s, k_s, v_s, a_s)
    k = (rng.standard_normal((70, kvh, hd)) * 2).astype(np.float32)
    v = (rng.standard_normal((70, kvh, hd)) * 2).astype(np.float32)
    kc, vc = fx.ops.kv_cache(kvh, max_pos)
    fx.ops.kv_append_i8(fx.to_device(k), fx.to_device(v), kc, vc, sc, pos0=100)
    k_ref = oracle.static_quant(k, k_s); v_ref = oracle.static_quant(v, v_s)
    kh = kc.numpy(); vh = vc.numpy()
    assert np.array_equal(kh[:, 100:170], k_ref.transpose(1, 0, 2))
    v_flat = vh.transpose(0, 1, 3, 2).reshape(kvh, max_pos, hd)     # [h][blk][d][p] -> [h][pos][d]
    assert np.array_equal(v_flat[:, 100:170], v_ref.transpose(1, 0, 2))
    assert not kh[:, :100].any() and not kh[:, 170:].any() and not v_flat[:, :100].any() and not v_flat[:, 170:].any()


# ------------------------------------------------------------------ greedy head
def test_embed_lm_head_argmax(fx, oracle):
    from flexllm_amd import synth
    vocab, hidden = 5000, 2048
    table = synth.host_uniform_f16((vocab, hidden), 5, -0.05, 0.05)
    n = rng.standard_normal(hidden).astype(np.float32)
    dt = fx.to_device(table)
    logits = fx.ops.lm_head_f16(dt, fx.to_device(n)).numpy()
    ref = oracle.lm_head(table.view(np.uint16), n)
    # fp32 accumulation order differs (lane-strided partial sums vs sequential): 1e-3 relative of the row scale
    np.testing.assert_allclose(logits, ref, rtol=1e-3, atol=1e-4)
    am = fx.ops.argmax_f32(fx.to_device(ref)).numpy()[0]
    assert am == int(np.argmax(ref))
    tie = np.zeros(70000, np.float32); tie[[69999, 123, 4567]] = 3.0
    assert fx.ops.argmax_f32(fx.to_device(tie)).numpy()[0] == 123
    tok = fx.to_device(np.array([4321], np.int32))
    e = fx.ops.embed_f16(dt, tok).numpy()
    assert np.array_equal(e, table[4321].astype(np.float32))


# ------------------------------------------------------------------ error behaviour
def test_bad_arguments_are_rejected_with_a_message(fx):
    from flexllm_amd._lib import FlexLLMError
    x = fx.to_device(np.zeros((2, 6), np.float32))
    with pytest.raises(FlexLLMError, match="multiple of 4"):
        fx.ops.quant_sym_i8(x)
    with pytest.raises(FlexLLMError, match="power of two"):
        fx.ops.fht_f32(fx.to_device(np.zeros((1, 3000), np.float32)))
    with pytest.raises(FlexLLMError, match="multiple of 16"):
        fx.ops.linear_i8_gemv(fx.to_device(np.zeros(8, np.int8)), fx.to_device(np.zeros((4, 8), np.int8)))


# ------------------------------------------------------------------ Logits.h top-k sampling
@pytest.mark.parametrize("n,k", [(128256, 5), (131072, 5), (4096, 1), (1000, 8), (64, 16)])
def test_sample_topk(fx, oracle, n, k):
    r = np.random.default_rng(n + k)
    x = (r.standard_normal(n) * 4).astype(np.float32)
    dx = fx.to_device(x)
    lanes = 8 if n % 8 == 0 else 1
    for rand in (0.0, 0.07, 0.31, 0.5, 0.83, 0.9999):
        tok, idx, val, prob = fx.ops.sample_topk_f32(dx, k, rand)
        tok_r, idx_r, val_r, prob_r = oracle.sample_topk(x, k, rand, lanes)
        assert np.array_equal(idx, idx_r) and np.array_equal(val, val_r)           # candidates: exact
        np.testing.assert_allclose(prob, prob_r, rtol=2e-6)                        # device expf vs glibc expf
        if np.abs(np.cumsum(prob_r.astype(np.float64)) - rand).min() > 1e-5:
            assert tok == tok_r
    # equal logits: same values and probabilities as the reference order, candidates ranked by index
    y = np.full(n, -3.0, np.float32); y[[n - 1, 5, n // 2]] = 9.0
    tok, idx, val, prob = fx.ops.sample_topk_f32(fx.to_device(y), min(k, 3) if k >= 3 else 1, 0.0)
    assert list(idx) == sorted([n - 1, 5, n // 2])[:len(idx)] and np.all(val == 9.0) and tok == 5


def test_stand_alone_scratch_is_per_stream(fx, oracle):
    """flexllm_mha_i8_decode, flexllm_argmax_f32 and flexllm_sample_topk_f32 keep their scratch per (device, stream):
    calls issued back to back on two streams with no synchronisation between them (so that they may overlap on the
    device) give what each gives alone, also after a stream's scratch had to grow."""
    rng = np.random.default_rng(314)
    qh, kvh, max_pos = 32, 8, 4096
    sc = fx.ops.Scales(rng.uniform(0.003, 0.005, qh).astype(np.float32), rng.uniform(0.02, 0.04, kvh).astype(np.float32),
                       rng.uniform(0.02, 0.04, kvh).astype(np.float32), np.full(qh, 1.0 / 255, np.float32))
    cases = []
    for length in (4096, 3000):
        q8 = fx.to_device(rng.integers(-128, 128, (qh, 64)).astype(np.int8))
        kc, vc = fx.ops.kv_cache(kvh, max_pos)
        fx.ops.kv_store_i8(fx.to_device(rng.integers(-60, 60, (length, kvh, 64)).astype(np.int8)),
                           fx.to_device(rng.integers(-128, 128, (length, kvh, 64)).astype(np.int8)), kc, vc, 0)
        o_ref, _ = fx.ops.mha_i8_decode(q8, kc, vc, sc, length)
        logits = fx.to_device(rng.standard_normal(128256).astype(np.float32))
        cases.append((q8, kc, vc, length, o_ref.numpy(), logits, int(np.argmax(logits.numpy()))))
    streams = [fx.Stream(), fx.Stream()]
    fx.ops.mha_i8_decode(cases[0][0], cases[0][1], cases[0][2], sc, 64, stream=streams[0])    # a small scratch first: the long call must grow it
    for rep in range(20):
        outs = []
        for (q8, kc, vc, length, o_ref, logits, am), st in zip(cases, streams):
            o, _ = fx.ops.mha_i8_decode(q8, kc, vc, sc, length, stream=st)
            outs.append((o, fx.ops.argmax_f32(logits, stream=st)))
        for st in streams:
            st.sync()
        for (q8, kc, vc, length, o_ref, logits, am), (o, r) in zip(cases, outs):
            assert np.array_equal(o.numpy(), o_ref), "repetition %d" % rep
            assert int(r.numpy()[0]) == am
    tok_a = fx.ops.sample_topk_f32(cases[0][5], 5, 0.3, stream=streams[0])[0]
    tok_b = fx.ops.sample_topk_f32(cases[1][5], 5, 0.3, stream=streams[1])[0]
    assert tok_a == oracle.sample_topk(cases[0][5].numpy(), 5, 0.3, 8)[0] and tok_b == oracle.sample_topk(cases[1][5].numpy(), 5, 0.3, 8)[0]


@pytest.mark.parametrize("k,n", [(2048, 2048), (4096, 512), (64, 37), (2048, 8192), (1024, 2)])
def test_fused_quant_gemv_dequant_decode_linear(fx, oracle, k, n):
    """flexllm_quant_linear_i8_gemv_dequant - the benchmark's single decode linear (1 x 2048 against 2048 x 2048) in one launch (fp32
    activation ~N(0,1) with outliers -> per-token int8 -> GEMV against uniform int8 weights -> dequantisation with
    per-channel scales): quantised bytes, scale and outputs bit for bit against the oracle's chain and against the
    two-kernel route on the device; a zero activation takes scale 1."""
    r = np.random.default_rng(1000 + k + n)
    x = outliers(r.standard_normal((1, k)).astype(np.float32))[0]
    w = r.integers(-127, 128, (n, k)).astype(np.int8)
    w_s = r.uniform(1e-3, 1e-2, n).astype(np.float32)
    res = r.standard_normal(n).astype(np.float32)
    dw, dws = fx.to_device(w), fx.to_device(w_s)
    for xv in (x, np.zeros(k, np.float32)):
        dx = fx.to_device(xv)
        y, q, s = fx.ops.quant_linear_i8_gemv_dequant(dx, dw, dws, want_q=True)
        q_ref, s_ref = oracle.quant_sym(xv[None, :])
        assert np.array_equal(q.numpy(), q_ref[0]) and np.array_equal(s.numpy(), s_ref.reshape(1))
        y_ref = oracle.dequant(oracle.linear_i8(q_ref, w), s_ref, w_s)[0]
        assert np.array_equal(y.numpy(), y_ref)
        y_res = fx.ops.quant_linear_i8_gemv_dequant(dx, dw, dws, residual=fx.to_device(res))
        assert np.array_equal(y_res.numpy(), oracle.residual(y_ref, res))
        q2, s2 = fx.ops.quant_sym_i8(fx.to_device(xv[None, :]))
        y2 = fx.ops.linear_i8_gemv_dequant(q2.view(0, (k,)), s2, dw, dws)
        assert np.array_equal(y.numpy(), y2.numpy())
    assert float(s.numpy()[0]) == 1.0 and not y.numpy().any()
