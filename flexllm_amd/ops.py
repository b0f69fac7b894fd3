"""Python wrappers over the C ABI operators.  Arguments are DeviceArrays; outputs are allocated here
unless passed in.  Names follow the reference's module names (quant, Linear_Layer, FHT, LayerNorm, RoPE,
Swish, Residual_Layer, Softmax, MHA_i8xi8)."""
import ctypes as C

import numpy as np

from ._lib import lib, check, MhaScales, MhaDynScales
from .device import DeviceArray, _s, to_device


def _p(a):
    return C.c_void_p(a.ptr) if a is not None else None


def _rows(a):
    return int(np.prod(a.shape[:-1], dtype=np.int64))


# ---------------------------------------------------------------- quant.h
def quant_sym_i8(x, stream=None):
    q = DeviceArray(x.shape, np.int8)
    s = DeviceArray(x.shape[:-1] or (1,), np.float32)
    check(lib().flexllm_quant_sym_i8(_p(x), _p(q), _p(s), _rows(x), x.shape[-1], _s(stream)))
    return q, s


def quant_asym_u8(x, bits=4, stream=None):
    q = DeviceArray(x.shape, np.uint8)
    s = DeviceArray(x.shape[:-1] or (1,), np.float32)
    b = DeviceArray(x.shape[:-1] or (1,), np.float32)
    check(lib().flexllm_quant_asym_u8(_p(x), _p(q), _p(s), _p(b), bits, _rows(x), x.shape[-1], _s(stream)))
    return q, s, b


def dequant_i32_f32(acc, s_x, w_s, b_x=None, w_sum=None, stream=None):
    y = DeviceArray(acc.shape, np.float32)
    check(lib().flexllm_dequant_i32_f32(_p(acc), _p(s_x), _p(b_x), _p(w_s), _p(w_sum), _p(y), _rows(acc),
                                        acc.shape[-1], _s(stream)))
    return y


def static_quant_i8(x, scale, factor=1.0, signed=True, stream=None):
    rows, heads, dim = x.shape
    q = DeviceArray(x.shape, np.int8 if signed else np.uint8)
    check(lib().flexllm_static_quant_i8(_p(x), _p(q), _p(scale), C.c_float(factor), int(signed), rows, heads, dim,
                                        _s(stream)))
    return q


def static_dequant_i32_f32(acc, a_s, w_s, stream=None):
    rows, ah, dim = acc.shape
    y = DeviceArray(acc.shape, np.float32)
    check(lib().flexllm_static_dequant_i32_f32(_p(acc), _p(y), _p(a_s), _p(w_s), rows, ah, w_s.shape[0], dim, _s(stream)))
    return y


def head_quant_sym_i8(x, stream=None):
    rows, heads, dim = x.shape
    q = DeviceArray(x.shape, np.int8)
    s = DeviceArray((rows, heads), np.float32)
    check(lib().flexllm_head_quant_sym_i8(_p(x), _p(q), _p(s), rows, heads, dim, _s(stream)))
    return q, s


# ---------------------------------------------------------------- Linear_Layer.h
def linear_i8_gemv(x, w, stream=None, out=None):
    n, k = w.shape
    acc = out if out is not None else DeviceArray((n,), np.int32)
    check(lib().flexllm_linear_i8_gemv(_p(x), _p(w), _p(acc), k, n, _s(stream)))
    return acc


def linear_u8i8_gemm(a, w, stream=None, out=None):
    """acc[m][n] = sum_k a[m][k] (uint8) * w[n][k] (int8): the probabilities x V product as a stand-alone module."""
    m, k = a.shape
    n = w.shape[0]
    acc = out if out is not None else DeviceArray((m, n), np.int32)
    check(lib().flexllm_linear_u8i8_gemm(_p(a), _p(w), _p(acc), m, k, n, _s(stream)))
    return acc


def linear_i8_gemv_dequant(x, s_x, w, w_s, residual=None, stream=None, out=None):
    n, k = w.shape
    y = out if out is not None else DeviceArray((n,), np.float32)
    check(lib().flexllm_linear_i8_gemv_dequant(_p(x), _p(s_x), _p(w), _p(w_s), _p(residual), _p(y), k, n, _s(stream)))
    return y


def quant_linear_i8_gemv_dequant(x, w, w_s, residual=None, want_q=False, stream=None, out=None):
    """One token's whole decode linear in one launch: quantise x fp32 [k] per token (symmetric int8), GEMV, dequantise
    (+ residual).  Returns y, or (y, q int8 [k], s_x [1]) with want_q."""
    n, k = w.shape
    y = out if out is not None else DeviceArray((n,), np.float32)
    q = DeviceArray((k,), np.int8) if want_q else None
    s = DeviceArray((1,), np.float32) if want_q else None
    check(lib().flexllm_quant_linear_i8_gemv_dequant(_p(x), _p(w), _p(w_s), _p(residual), _p(y), _p(s), _p(q), k, n, _s(stream)))
    return (y, q, s) if want_q else y


def linear_i8_gemv_swiglu(x, s_x, w_gu, w_s_gu, stream=None, out=None):
    """x int8 [k], w_gu int8 [2n][k] (rows interleaved gate, up) -> y fp32 [n] = up * silu(gate)."""
    k = x.shape[-1]
    n = w_gu.shape[0] // 2
    y = out if out is not None else DeviceArray((n,), np.float32)
    check(lib().flexllm_linear_i8_gemv_swiglu(_p(x), _p(s_x), _p(w_gu), _p(w_s_gu), _p(y), k, n, _s(stream)))
    return y


def linear_i8_gemm(a, w, stream=None, out=None):
    m, k = a.shape
    n = w.shape[0]
    acc = out if out is not None else DeviceArray((m, n), np.int32)
    check(lib().flexllm_linear_i8_gemm(_p(a), _p(w), _p(acc), m, k, n, _s(stream)))
    return acc


def linear_i8_gemm_dequant(a, s_x, w, w_s, residual=None, stream=None, out=None):
    m, k = a.shape
    n = w.shape[0]
    y = out if out is not None else DeviceArray((m, n), np.float32)
    check(lib().flexllm_linear_i8_gemm_dequant(_p(a), _p(s_x), _p(w), _p(w_s), _p(residual), _p(y), m, k, n, _s(stream)))
    return y


def linear_i8_gemm_swiglu(a, s_x, w_gu, w_s_gu, stream=None, out=None):
    """a int8 [m][k], w_gu int8 [2n][k] (rows interleaved gate, up) -> h fp32 [m][n] = up * silu(gate)."""
    m, k = a.shape
    n = w_gu.shape[0] // 2
    h = out if out is not None else DeviceArray((m, n), np.float32)
    check(lib().flexllm_linear_i8_gemm_swiglu(_p(a), _p(s_x), _p(w_gu), _p(w_s_gu), _p(h), m, k, n, _s(stream)))
    return h


# ---------------------------------------------------------------- W4A4 (Linear_Layer.h i4 PEs)
def pack_nibbles(values, stream=None):
    """uint8/int8 [..., k] one value per byte -> uint8 [..., k/2], low nibble = even index."""
    out = DeviceArray(values.shape[:-1] + (values.shape[-1] // 2,), np.uint8)
    check(lib().flexllm_pack_nibbles(_p(values), _p(out), C.c_size_t(values.size), _s(stream)))
    return out


def linear_u4i4_gemv(x4, w4, stream=None):
    n, k = w4.shape[0], w4.shape[1] * 2
    acc = DeviceArray((n,), np.int32)
    check(lib().flexllm_linear_u4i4_gemv(_p(x4), _p(w4), _p(acc), k, n, _s(stream)))
    return acc


def linear_u4i4_gemv_dequant(x4, s_x, b_x, w4, w_s, w_sum, residual=None, stream=None):
    n, k = w4.shape[0], w4.shape[1] * 2
    y = DeviceArray((n,), np.float32)
    check(lib().flexllm_linear_u4i4_gemv_dequant(_p(x4), _p(s_x), _p(b_x), _p(w4), _p(w_s), _p(w_sum), _p(residual), _p(y),
                                                 k, n, _s(stream)))
    return y


def linear_u4i4_gemm(a4, w4, stream=None):
    m, n, k = a4.shape[0], w4.shape[0], w4.shape[1] * 2
    acc = DeviceArray((m, n), np.int32)
    check(lib().flexllm_linear_u4i4_gemm(_p(a4), _p(w4), _p(acc), m, k, n, _s(stream)))
    return acc


def linear_u4i4_gemm_dequant(a4, s_x, b_x, w4, w_s, w_sum, residual=None, stream=None):
    m, n, k = a4.shape[0], w4.shape[0], w4.shape[1] * 2
    y = DeviceArray((m, n), np.float32)
    check(lib().flexllm_linear_u4i4_gemm_dequant(_p(a4), _p(s_x), _p(b_x), _p(w4), _p(w_s), _p(w_sum), _p(residual), _p(y),
                                                 m, k, n, _s(stream)))
    return y


# ---------------------------------------------------------------- FHT.h
def linear_i8_gemm_dequant_asym(a, s_x, b_x, w, w_s, w_sum, residual=None, stream=None):
    """W4A4-style product on operands held one value per byte: a [m][k] unsigned values (0..127) in int8/uint8
    containers, w [n][k] int8; y = (float(acc) * s_x) * w_s + b_x * w_sum (+ residual)."""
    m, k = a.shape
    n = w.shape[0]
    y = DeviceArray((m, n), np.float32)
    check(lib().flexllm_linear_i8_gemm_dequant_asym(_p(a), _p(s_x), _p(b_x), _p(w), _p(w_s), _p(w_sum), _p(residual), _p(y),
                                                    m, k, n, _s(stream)))
    return y


def linear_i8_gemm_swiglu_asym(a, s_x, b_x, w_gu, w_s_gu, w_sum_gu, stream=None):
    """Gate/up projection of the W4A4 precision (operands one value per byte, interleaved gate/up rows) with
    SiLU(gate) * up in the epilogue: h [m][n], n = w_gu.shape[0] // 2."""
    m, k = a.shape
    n = w_gu.shape[0] // 2
    h = DeviceArray((m, n), np.float32)
    check(lib().flexllm_linear_i8_gemm_swiglu_asym(_p(a), _p(s_x), _p(b_x), _p(w_gu), _p(w_s_gu), _p(w_sum_gu), _p(h), m, k, n,
                                                   _s(stream)))
    return h


def lm_head_u4i4(n_vec, w4, w_s, w_sum, stream=None):
    """The reference's output head (SpinQuant_Decoding_mem_opt.h:363-365, config D6): the normalised hidden vector is
    quantised to asymmetric uint4, multiplied with the int4 head weights (nibble-packed [vocab_pad][hidden/2]) and
    dequantised with zero point x row sum.  Returns fp32 logits [vocab_pad]."""
    hidden = n_vec.shape[-1]
    q, s, b = quant_asym_u8(n_vec.view(0, (1, hidden)), bits=4, stream=stream)
    a4 = pack_nibbles(q, stream=stream)
    return linear_u4i4_gemv_dequant(a4.view(0, (hidden // 2,)), s, b, w4, w_s, w_sum, stream=stream)


def fht_f32(x, scale=1.0, stream=None, out=None):
    y = out if out is not None else DeviceArray(x.shape, np.float32)
    check(lib().flexllm_fht_f32(_p(x), _p(y), _rows(x), x.shape[-1], C.c_float(scale), _s(stream)))
    return y


def fht_quant_i8(x, scale=1.0, stream=None):
    q = DeviceArray(x.shape, np.int8)
    s = DeviceArray(x.shape[:-1] or (1,), np.float32)
    check(lib().flexllm_fht_quant_i8(_p(x), _p(q), _p(s), _rows(x), x.shape[-1], C.c_float(scale), _s(stream)))
    return q, s


def fht_quant_asym_u8(x, scale=1.0, bits=4, stream=None):
    q = DeviceArray(x.shape, np.uint8)
    s = DeviceArray(x.shape[:-1] or (1,), np.float32)
    b = DeviceArray(x.shape[:-1] or (1,), np.float32)
    check(lib().flexllm_fht_quant_asym_u8(_p(x), _p(q), _p(s), _p(b), bits, _rows(x), x.shape[-1], C.c_float(scale), _s(stream)))
    return q, s, b


# ---------------------------------------------------------------- LayerNorm.h
def rmsnorm_quant_asym_u8(x, gamma, eps=1e-5, bits=4, stream=None):
    q = DeviceArray(x.shape, np.uint8)
    s = DeviceArray(x.shape[:-1] or (1,), np.float32)
    b = DeviceArray(x.shape[:-1] or (1,), np.float32)
    check(lib().flexllm_rmsnorm_quant_asym_u8(_p(x), _p(gamma), _p(q), _p(s), _p(b), bits, _rows(x), x.shape[-1], C.c_float(eps),
                                              _s(stream)))
    return q, s, b


def rmsnorm_f32(x, gamma, eps=1e-5, stream=None):
    y = DeviceArray(x.shape, np.float32)
    check(lib().flexllm_rmsnorm_f32(_p(x), _p(gamma), _p(y), _rows(x), x.shape[-1], C.c_float(eps), _s(stream)))
    return y


def rmsnorm_quant_i8(x, gamma, eps=1e-5, stream=None):
    q = DeviceArray(x.shape, np.int8)
    s = DeviceArray(x.shape[:-1] or (1,), np.float32)
    check(lib().flexllm_rmsnorm_quant_i8(_p(x), _p(gamma), _p(q), _p(s), _rows(x), x.shape[-1], C.c_float(eps), _s(stream)))
    return q, s


# ---------------------------------------------------------------- RoPE.h
def rope_table(max_pos, head_dim=64, theta=500000.0, factor=32, low=1, high=4, orig=8192):
    s = np.empty((max_pos, head_dim // 2), np.float32)
    c = np.empty((max_pos, head_dim // 2), np.float32)
    check(lib().flexllm_rope_table_host(s.ctypes.data_as(C.c_void_p), c.ctypes.data_as(C.c_void_p), max_pos, head_dim,
                                        C.c_float(theta), factor, low, high, orig))
    return s, c


def rope_f32(x, sin_t, cos_t, pos0=0, stream=None):
    tokens, heads, hd = x.shape
    y = DeviceArray(x.shape, np.float32)
    check(lib().flexllm_rope_f32(_p(x), _p(y), _p(sin_t), _p(cos_t), tokens, heads, hd, pos0, _s(stream)))
    return y


# ---------------------------------------------------------------- Swish.h / gate / Residual_Layer.h
def swish_f32(x, stream=None):
    y = DeviceArray(x.shape, np.float32)
    check(lib().flexllm_swish_f32(_p(x), _p(y), C.c_size_t(x.size), _s(stream)))
    return y


def swiglu_f32(gate, up, stream=None):
    y = DeviceArray(gate.shape, np.float32)
    check(lib().flexllm_swiglu_f32(_p(gate), _p(up), _p(y), C.c_size_t(gate.size), _s(stream)))
    return y


def residual_add_f32(a, b, stream=None):
    y = DeviceArray(a.shape, np.float32)
    check(lib().flexllm_residual_add_f32(_p(a), _p(b), _p(y), C.c_size_t(a.size), _s(stream)))
    return y


def softmax_f32(x, stream=None):
    y = DeviceArray(x.shape, np.float32)
    check(lib().flexllm_softmax_f32(_p(x), _p(y), _rows(x), x.shape[-1], _s(stream)))
    return y


# ---------------------------------------------------------------- MHA_i8xi8.h
class Scales:
    """Device copies of one layer's static attention scales."""

    def __init__(self, q_s, k_s, v_s, a_s):
        self.arrays = [to_device(np.asarray(a, np.float32)) for a in (q_s, k_s, v_s, a_s)]
        self.struct = MhaScales(*[a.ptr for a in self.arrays])

    def ref(self):
        return C.byref(self.struct)


def kv_cache(kv_heads, max_pos, head_dim=64):
    assert max_pos % 64 == 0
    k = DeviceArray((kv_heads, max_pos, head_dim), np.int8).zero_()
    v = DeviceArray((kv_heads, max_pos // 64, head_dim, 64), np.int8).zero_()
    return k, v


def kv_append_i8(k, v, k_cache, v_cache, scales, pos0, stream=None):
    tokens, kvh, hd = k.shape
    max_pos = k_cache.shape[1]
    check(lib().flexllm_kv_append_i8(_p(k), _p(v), _p(k_cache), _p(v_cache), scales.ref(), tokens, kvh, hd, max_pos, pos0,
                                     _s(stream)))


def linear_i8_gemm_qkv_rope_cache(a, s_x, w_qkv, w_s, sin_t, cos_t, scales, k_cache, v_cache, q_heads, pos0=0, stream=None):
    """Fused q/k/v projection + RoPE + static quantisation + cache stores; returns q8 [m][q_heads][64]."""
    m, k = a.shape
    kv_heads, max_pos = k_cache.shape[0], k_cache.shape[1]
    q8 = DeviceArray((m, q_heads, 64), np.int8)
    check(lib().flexllm_linear_i8_gemm_qkv_rope_cache(_p(a), _p(s_x), _p(w_qkv), _p(w_s), _p(sin_t), _p(cos_t), scales.ref(),
                                                      _p(q8), _p(k_cache), _p(v_cache), m, k, q_heads, kv_heads, max_pos,
                                                      pos0, _s(stream)))
    return q8


def kv_store_i8(k8, v8, k_cache, v_cache, pos0, stream=None):
    tokens, kvh, hd = k8.shape
    max_pos = k_cache.shape[1]
    check(lib().flexllm_kv_store_i8(_p(k8), _p(v8), _p(k_cache), _p(v_cache), tokens, kvh, hd, max_pos, pos0, _s(stream)))


def mha_i8_decode(q8, k_cache, v_cache, scales, length, want_p=False, stream=None):
    qh, hd = q8.shape
    kvh, max_pos, _ = k_cache.shape
    o = DeviceArray((qh, hd), np.float32)
    p8 = DeviceArray((qh, length), np.uint8) if want_p else None
    check(lib().flexllm_mha_i8_decode(_p(q8), _p(k_cache), _p(v_cache), scales.ref(), _p(o), _p(p8), length, qh, kvh, hd,
                                      max_pos, _s(stream)))
    return o, p8


def mha_i8_decode_noalloc(q8, k_cache, v_cache, scales, length, o, p8=None, stream=None):
    """flexllm_mha_i8_decode on the library's built-in scratch: the caller passes the outputs, nothing is allocated."""
    qh, hd = q8.shape
    kvh, max_pos, _ = k_cache.shape
    check(lib().flexllm_mha_i8_decode_noalloc(_p(q8), _p(k_cache), _p(v_cache), scales.ref(), _p(o), _p(p8), length, qh, kvh,
                                              hd, max_pos, _s(stream)))
    return o, p8


def mha_i8_prefill(q8, k_cache, v_cache, scales, want_p=False, stream=None):
    s, qh, hd = q8.shape
    kvh, max_pos, _ = k_cache.shape
    o = DeviceArray((s, qh, hd), np.float32)
    p8 = DeviceArray((qh, s, s), np.uint8).zero_() if want_p else None
    check(lib().flexllm_mha_i8_prefill(_p(q8), _p(k_cache), _p(v_cache), scales.ref(), _p(o), _p(p8), s, qh, kvh, hd,
                                       max_pos, _s(stream)))
    return o, p8


def _dyn_scales(q_s, k_s, v_s, v_ch_s, q_scale_div):
    return MhaDynScales(q_s.ptr, k_s.ptr, v_s.ptr, v_ch_s.ptr if v_ch_s is not None else None, float(q_scale_div))


def mha_i8_prefill_dyn(q8, q_s, k_cache, k_s, v_cache, v_s, v_ch_s=None, q_scale_div=8.0, want_p=False, stream=None):
    """Attention with dynamic per-(token, head) scales: q_s [s][qh], k_s / v_s [max_pos][kvh] device arrays of the
    quantiser's scales.  Returns (o, p8 int8 [qh][s][s] or None, p_s [s][qh])."""
    s, qh, hd = q8.shape
    kvh, max_pos, _ = k_cache.shape
    o = DeviceArray((s, qh, hd), np.float32)
    p8 = DeviceArray((qh, s, s), np.int8).zero_() if want_p else None
    p_s = DeviceArray((s, qh), np.float32)
    sc = _dyn_scales(q_s, k_s, v_s, v_ch_s, q_scale_div)
    check(lib().flexllm_mha_i8_prefill_dyn(_p(q8), _p(k_cache), _p(v_cache), C.byref(sc), _p(o), _p(p8), _p(p_s), s, qh, kvh, hd,
                                           max_pos, _s(stream)))
    return o, p8, p_s


def mha_i8_decode_dyn(q8, q_s, k_cache, k_s, v_cache, v_s, length, v_ch_s=None, q_scale_div=8.0, want_p=False, stream=None):
    qh, hd = q8.shape
    kvh, max_pos, _ = k_cache.shape
    o = DeviceArray((qh, hd), np.float32)
    p8 = DeviceArray((qh, length), np.int8) if want_p else None
    p_s = DeviceArray((qh,), np.float32)
    sc = _dyn_scales(q_s, k_s, v_s, v_ch_s, q_scale_div)
    check(lib().flexllm_mha_i8_decode_dyn(_p(q8), _p(k_cache), _p(v_cache), C.byref(sc), _p(o), _p(p8), _p(p_s), length, qh, kvh,
                                          hd, max_pos, _s(stream)))
    return o, p8, p_s


# ---------------------------------------------------------------- Logits.h (greedy)
def embed_f16(table, token, stream=None):
    y = DeviceArray((table.shape[1],), np.float32)
    check(lib().flexllm_embed_f16(_p(table), _p(token), _p(y), table.shape[1], _s(stream)))
    return y


def lm_head_f16(table, n, stream=None):
    vocab, hidden = table.shape
    logits = DeviceArray((vocab,), np.float32)
    check(lib().flexllm_lm_head_f16(_p(table), _p(n), _p(logits), vocab, hidden, _s(stream)))
    return logits


def argmax_f32(x, stream=None):
    r = DeviceArray((1,), np.int32)
    check(lib().flexllm_argmax_f32(_p(x), x.size, _p(r), _s(stream)))
    return r


def sample_topk_f32(logits, top_k=5, rand=0.5, enable_sub_max=True, stream=None):
    """Top-k sampling (Logits.h): returns (token, top_idx, top_val, top_prob) as host values."""
    n = logits.size
    r = to_device(np.array([rand], np.float32))
    tok = DeviceArray((1,), np.int32)
    idx = DeviceArray((top_k,), np.int32); val = DeviceArray((top_k,), np.float32); prob = DeviceArray((top_k,), np.float32)
    check(lib().flexllm_sample_topk_f32(_p(logits), n, top_k, _p(r), int(enable_sub_max), _p(tok), _p(idx), _p(val), _p(prob),
                                        _s(stream)))
    return int(tok.numpy()[0]), idx.numpy(), val.numpy(), prob.numpy()
