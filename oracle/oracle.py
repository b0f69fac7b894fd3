"""ctypes loader for the CPU oracle (oracle/flexllm_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke run and by the
benchmark's cpu_baseline leg, never by the shipped package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libflexllm_oracle.so")


def build(force=False):
    """Compile the oracle with gcc (no GPU toolchain involved)."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-B", "-C", _HERE, "libflexllm_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_SO)
        _lib.fxo_half_to_float.restype = C.c_float
        _lib.fxo_half_to_float.argtypes = [C.c_uint16]
        _lib.fxo_argmax.restype = C.c_int
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _f(v):
    return C.c_float(float(v))


def quant_sym(x, bits=8):
    x = _f32(x)
    rows, dim = x.reshape(-1, x.shape[-1]).shape
    q = np.empty(x.shape, np.int8)
    s = np.empty(rows, np.float32)
    lib().fxo_quant_sym(_p(x), rows, dim, bits, _p(q), _p(s))
    return q, s.reshape(x.shape[:-1])


def quant_asym(x, bits=4):
    x = _f32(x)
    rows, dim = x.reshape(-1, x.shape[-1]).shape
    q = np.empty(x.shape, np.uint8)
    s = np.empty(rows, np.float32)
    b = np.empty(rows, np.float32)
    lib().fxo_quant_asym(_p(x), rows, dim, bits, _p(q), _p(s), _p(b))
    return q, s, b


def dequant(acc, s_x, w_s, b_x=None, w_sum=None):
    acc = np.ascontiguousarray(acc, np.int32)
    rows, n = acc.shape
    s_x = _f32(np.reshape(s_x, -1)); w_s = _f32(w_s)
    b_x = _f32(np.reshape(b_x, -1)) if b_x is not None else None
    w_sum = _f32(w_sum) if w_sum is not None else None
    y = np.empty((rows, n), np.float32)
    lib().fxo_dequant(_p(acc), rows, n, _p(s_x), _p(b_x), _p(w_s), _p(w_sum), _p(y))
    return y


def static_quant(x, scale, factor=1.0, signed=True, bits=8):
    """x [rows][heads][dim] -> int8 (signed) / uint8 (unsigned)."""
    x = _f32(x)
    rows, heads, dim = x.shape
    scale = _f32(scale)
    assert scale.shape == (heads,)
    q = np.empty(x.shape, np.int8)
    lib().fxo_static_quant(_p(x), rows, heads, dim, _p(scale), _f(factor), int(signed), bits, _p(q))
    return q if signed else q.view(np.uint8)


def static_dequant(acc, a_s, w_s):
    acc = np.ascontiguousarray(acc, np.int32)
    rows, ah, dim = acc.shape
    a_s = _f32(a_s); w_s = _f32(w_s)
    y = np.empty(acc.shape, np.float32)
    lib().fxo_static_dequant(_p(acc), rows, ah, w_s.shape[0], dim, _p(a_s), _p(w_s), _p(y))
    return y


def head_quant_sym(x, bits=8):
    x = _f32(x)
    rows, heads, dim = x.shape
    q = np.empty(x.shape, np.int8)
    s = np.empty((rows, heads), np.float32)
    lib().fxo_head_quant_sym(_p(x), rows, heads, dim, bits, _p(q), _p(s))
    return q, s


def linear_i8(a, w):
    a = np.ascontiguousarray(a); w = np.ascontiguousarray(w, np.int8)
    m, k = a.shape
    n = w.shape[0]
    assert w.shape[1] == k
    c = np.empty((m, n), np.int32)
    if a.dtype == np.uint8:
        lib().fxo_linear_u8i8(_p(a), _p(w), m, k, n, _p(c))
    else:
        assert a.dtype == np.int8
        lib().fxo_linear_i8(_p(a), _p(w), m, k, n, _p(c))
    return c


def fht(x, scale=1.0):
    x = _f32(x)
    rows, n = x.reshape(-1, x.shape[-1]).shape
    y = np.empty(x.shape, np.float32)
    lib().fxo_fht(_p(x), rows, n, _f(scale), _p(y))
    return y


def rmsnorm_pref(x, gamma, eps=1e-5):
    x = _f32(x); gamma = _f32(gamma)
    rows, dim = x.shape
    y = np.empty(x.shape, np.float32)
    lib().fxo_rmsnorm_pref(_p(x), _p(gamma), rows, dim, _f(eps), _p(y))
    return y


def rmsnorm_dec(x, gamma, block_parallel=8, eps=1e-5):
    x = _f32(x); gamma = _f32(gamma)
    y = np.empty(x.shape, np.float32)
    lib().fxo_rmsnorm_dec(_p(x), _p(gamma), x.shape[-1], block_parallel, _f(eps), _p(y))
    return y


def rope_table(max_pos, head_dim=64, theta=500000.0, factor=32, low=1, high=4, orig=8192):
    s = np.empty((max_pos, head_dim // 2), np.float32)
    c = np.empty((max_pos, head_dim // 2), np.float32)
    lib().fxo_rope_table(max_pos, head_dim, _f(theta), factor, low, high, orig, _p(s), _p(c))
    return s, c


def rope(x, sin_t, cos_t, pos0=0):
    x = _f32(x)
    tokens, heads, hd = x.shape
    y = np.empty(x.shape, np.float32)
    lib().fxo_rope(_p(x), tokens, heads, hd, _p(_f32(sin_t)), _p(_f32(cos_t)), pos0, _p(y))
    return y


def swish(x):
    x = _f32(x); y = np.empty(x.shape, np.float32)
    lib().fxo_swish(_p(x), x.size, _p(y)); return y


def gate(a, b):
    a = _f32(a); b = _f32(b); y = np.empty(a.shape, np.float32)
    lib().fxo_gate(_p(a), _p(b), a.size, _p(y)); return y


def residual(a, b):
    a = _f32(a); b = _f32(b); y = np.empty(a.shape, np.float32)
    lib().fxo_residual(_p(a), _p(b), a.size, _p(y)); return y


def softmax(x):
    x = _f32(x)
    rows, dim = x.reshape(-1, x.shape[-1]).shape
    y = np.empty(x.shape, np.float32)
    lib().fxo_softmax(_p(x), rows, dim, _p(y)); return y


def softmax_dec(x, block_parallel=4, scale=None):
    """dec_Softmax on one block-partitioned vector; `scale` divides the exponent (enable_scale)."""
    x = _f32(x); y = np.empty(x.shape, np.float32)
    lib().fxo_softmax_dec(_p(x), x.size, block_parallel, 0 if scale is None else 1, C.c_float(1.0 if scale is None else scale), _p(y))
    return y


def linear_f32(x, w):
    """fp32 GEMV y = W x with the reference's four partial sums (dec_Linear_Layer_fp32xfp32)."""
    x = _f32(x); w = _f32(w); n, k = w.shape
    y = np.empty(n, np.float32)
    lib().fxo_linear_f32(_p(x), _p(w), k, n, _p(y)); return y


def hmt_retrieve(q, kmem, mmem, scale, block_parallel=4):
    """(softmaxed scores over all memory slots, retrieved memory embedding P) for query q."""
    q = _f32(q); kmem = _f32(kmem); mmem = _f32(mmem)
    mem_num, hidden = mmem.shape
    assert mem_num % block_parallel == 0 and mem_num <= 1024, "memory slots come in whole blocks"
    a = np.empty(mem_num, np.float32); p_out = np.empty(hidden, np.float32)
    lib().fxo_hmt_retrieve(_p(q), _p(kmem), _p(mmem), mem_num, hidden, block_parallel, C.c_float(scale), _p(a), _p(p_out))
    return a, p_out


def w4a4_linear(x, w_q, w_s, w_sum, residual_in=None):
    """One W4A4 linear of the reference: asymmetric uint4 quantisation per token, exact integer product, dequantisation
    with zero point x row sum (quant.h:53-82, Linear_Layer.h i4 PEs, quant.h:147-152), optional residual."""
    q, s, b = quant_asym(x, bits=4)
    y = dequant(linear_i8(q, w_q), s, w_s, b_x=b, w_sum=w_sum)
    return y if residual_in is None else residual(y, residual_in)


def w4a4_layer(cfg, w, l, x, pos0, k_cache, v_cache):
    """One decoder layer of the shipped W4A4 configuration on S tokens starting at pos0 (S > 1: prefill from 0; S == 1:
    decode), stage order of SpinQuant_Prefilling.h:807-1050 / SpinQuant_Decoding_mem_opt.h:947-1128.  k_cache, v_cache:
    int8 [max_pos][kv_hidden] of this layer, updated in place."""
    S, H = x.shape
    qh, kvh, hd = cfg["q_heads"], cfg["kv_heads"], cfg["head_dim"]
    norm = rmsnorm_pref if S > 1 else (lambda t, g, eps: rmsnorm_dec(t[0], g, eps=eps)[None, :])
    n = norm(x, w["gamma"][2 * l], cfg["eps"])
    q = w4a4_linear(n, w["wq"][l], w["sq"][l], w["sumq"][l])
    k = w4a4_linear(n, w["wk"][l], w["sk"][l], w["sumk"][l])
    v = w4a4_linear(n, w["wv"][l], w["sv"][l], w["sumv"][l])
    q = rope(q.reshape(S, qh, hd), w["rope_sin"], w["rope_cos"], pos0)
    k = rope(k.reshape(S, kvh, hd), w["rope_sin"], w["rope_cos"], pos0)
    if S > 1:
        r = mha_prefill(q, k, v.reshape(S, kvh, hd), w["q_s"][l], w["k_s"][l], w["v_s"][l], w["a_s"][l])
        k_cache[:S] = r["k8"].reshape(S, -1); v_cache[:S] = r["v8"].reshape(S, -1)
        o = r["o"]
    else:
        q8 = static_quant(q, w["q_s"][l], factor=8.0)
        k_cache[pos0] = static_quant(k, w["k_s"][l]).reshape(-1)
        v_cache[pos0] = static_quant(v.reshape(1, kvh, hd), w["v_s"][l]).reshape(-1)
        o, _ = mha_decode(q8[0], k_cache[:pos0 + 1].reshape(pos0 + 1, kvh, hd), v_cache[:pos0 + 1].reshape(pos0 + 1, kvh, hd),
                          w["q_s"][l], w["k_s"][l], w["v_s"][l], w["a_s"][l])
    x2 = w4a4_linear(o.reshape(S, H), w["wo"][l], w["so"][l], w["sumo"][l], residual_in=x)
    n2 = norm(x2, w["gamma"][2 * l + 1], cfg["eps"])
    g = w4a4_linear(n2, w["wg"][l], w["sg"][l], w["sumg"][l])
    u = w4a4_linear(n2, w["wu"][l], w["su"][l], w["sumu"][l])
    h = gate(u, swish(g))
    return w4a4_linear(fht(h, cfg["fht_scale"]), w["wd"][l], w["sd"][l], w["sumd"][l], residual_in=x2)


def hmt_stage_lengths(seq_len, seg_id, seg_num, seg_len, sum_seg_len, rec_seg_len, pad):
    """(current segment length, stage-0 length, stage-1 length), lengths padded up to a multiple of `pad`
    (Modules/HMT.h:39-45)."""
    cur = seg_len if seg_id < seg_num - 1 else seq_len - seg_id * seg_len
    cur_sum = min(cur, sum_seg_len)
    up = lambda n: (n + pad - 1) // pad * pad
    return cur, up(1 + cur_sum + 1), up(1 + rec_seg_len + cur + 1)


def hmt_run(backbone, emb, t_embed, wq, wk, seg_len, sum_seg_len, rec_seg_len, mem_num, scale, pad=8, block_parallel=4):
    """The segment loop of the HMT plug-in (Modules/HMT.h:8-195 feeding :198-474) around `backbone`, a function
    [S][hidden] -> [S][hidden] (the layer stack without the final norm).  `emb` holds the token embeddings, `t_embed`
    the summary-prompt embedding stored ahead of them (HMT.h:10).  Returns (list of stage-1 hidden states of each
    segment's own tokens, memory matrix, key matrix, list of retrieved embeddings P_n)."""
    emb = _f32(emb); seq_len, hidden = emb.shape
    seg_num = (seq_len + seg_len - 1) // seg_len
    mmem = np.zeros((mem_num, hidden), np.float32)                 # HMT.h:369-378, :428-437: caches start at zero
    kmem = np.zeros((mem_num, hidden), np.float32)
    p_buf = np.zeros(hidden, np.float32)                           # HMT.h:29-35
    outs, ps = [], []
    for seg in range(seg_num):
        cur, len0, len1 = hmt_stage_lengths(seq_len, seg, seg_num, seg_len, sum_seg_len, rec_seg_len, pad)
        cur_sum = min(cur, sum_seg_len)
        off = seg * seg_len
        if seg > 0:                                                # stage 0: [T, first cur_sum tokens, T] (HMT.h:48-98)
            x0 = np.zeros((len0, hidden), np.float32)
            x0[0] = t_embed
            x0[1:1 + cur_sum] = emb[off:off + cur_sum]
            x0[1 + cur_sum] = t_embed
            s_n = backbone(x0)[1 + cur_sum]                        # HMT.h:101-105
            q_n = linear_f32(s_n, wq)                              # HMT.h:289-292
            _, p_buf = hmt_retrieve(q_n, kmem, mmem, scale, block_parallel)     # HMT.h:294-302
            ps.append(p_buf.copy())
        x1 = np.zeros((len1, hidden), np.float32)                  # stage 1 (HMT.h:125-170)
        x1[0] = p_buf
        for j in range(rec_seg_len):                               # the tokens just before the segment, zeros before the text
            src = off - rec_seg_len + j
            if src >= 0:
                x1[1 + j] = emb[src]
        x1[1 + rec_seg_len:1 + rec_seg_len + cur] = emb[off:off + cur]
        if seg < seg_num - 1:
            x1[1 + rec_seg_len + cur] = p_buf
        h1 = backbone(x1)
        outs.append(h1[1 + rec_seg_len:1 + rec_seg_len + cur].copy())
        if seg < seg_num - 1:                                      # HMT.h:176-190, :397-406, :456-472
            m_n = h1[1 + rec_seg_len + cur]
            mmem[seg % mem_num] = m_n
            kmem[seg % mem_num] = linear_f32(m_n, wk)              # HMT.h:306-311
    return outs, mmem, kmem, ps


def causal_mask(x):
    x = _f32(x)
    rows, heads, dim = x.shape
    y = np.empty(x.shape, np.float32)
    lib().fxo_causal_mask(_p(x), rows, heads, dim, _p(y)); return y


class MhaScales(C.Structure):
    _fields_ = [("q_s", C.c_void_p), ("k_s", C.c_void_p), ("v_s", C.c_void_p), ("a_s", C.c_void_p)]


def _scales(q_s, k_s, v_s, a_s):
    keep = [_f32(q_s), _f32(k_s), _f32(v_s), _f32(a_s)]
    sc = MhaScales(*[a.ctypes.data for a in keep])
    return sc, keep


def mha_prefill(q, k, v, q_s, k_s, v_s, a_s, want_p=False):
    """q [s][qh][hd], k/v [s][kvh][hd] fp32 -> dict(q8,k8,v8,p8,o)."""
    q = _f32(q); k = _f32(k); v = _f32(v)
    s, qh, hd = q.shape
    kvh = k.shape[1]
    sc, keep = _scales(q_s, k_s, v_s, a_s)
    q8 = np.empty(q.shape, np.int8); k8 = np.empty(k.shape, np.int8); v8 = np.empty(v.shape, np.int8)
    p8 = np.empty((qh, s, s), np.uint8) if want_p else None
    o = np.empty(q.shape, np.float32)
    lib().fxo_mha_prefill(_p(q), _p(k), _p(v), s, qh, kvh, hd, C.byref(sc), _p(q8), _p(k8), _p(v8), _p(p8), _p(o))
    return dict(q8=q8, k8=k8, v8=v8, p8=p8, o=o)


def mha_prefill_i8(q8, k8, v8, q_s, k_s, v_s, a_s, p8_in=None, want_p=False):
    """Attention from int8 tensors q8 [s][qh][64], k8/v8 [s][kvh][64]; p8_in [qh][s][s] replaces the computed
    probabilities in P.V."""
    q8 = np.ascontiguousarray(q8, np.int8); k8 = np.ascontiguousarray(k8, np.int8); v8 = np.ascontiguousarray(v8, np.int8)
    s, qh, hd = q8.shape
    kvh = k8.shape[1]
    sc, keep = _scales(q_s, k_s, v_s, a_s)
    p_in = np.ascontiguousarray(p8_in, np.uint8) if p8_in is not None else None
    assert p_in is None or p_in.shape == (qh, s, s)
    p8 = np.empty((qh, s, s), np.uint8) if want_p else None
    o = np.empty((s, qh, hd), np.float32)
    lib().fxo_mha_prefill_i8(_p(q8), _p(k8), _p(v8), s, qh, kvh, hd, C.byref(sc), _p(p_in), _p(p8), _p(o))
    return (o, p8) if want_p else o


def mha_decode(q8, k_cache, v_cache, q_s, k_s, v_s, a_s, want_p=False):
    """q8 [qh][hd] int8, caches [len][kvh][hd] int8 -> (o [qh][hd] fp32, p8 [qh][len])."""
    q8 = np.ascontiguousarray(q8, np.int8)
    k_cache = np.ascontiguousarray(k_cache, np.int8); v_cache = np.ascontiguousarray(v_cache, np.int8)
    qh, hd = q8.shape
    ln, kvh, _ = k_cache.shape
    sc, keep = _scales(q_s, k_s, v_s, a_s)
    p8 = np.empty((qh, ln), np.uint8) if want_p else None
    o = np.empty((qh, hd), np.float32)
    lib().fxo_mha_decode(_p(q8), _p(k_cache), _p(v_cache), ln, qh, kvh, hd, C.byref(sc), _p(p8), _p(o))
    return o, p8


def mha_prefill_dyn(q, k, v, v_ch_s=None, want_p=False):
    """Attention with dynamic per-(token, head) scales.  q [s][qh][hd], k/v [s][kvh][hd] fp32 ->
    dict(q8, q_s, k8, k_s, v8, v_s, p8 (int8 [qh][s][s] or None), p_s [s][qh], o)."""
    q = _f32(q); k = _f32(k); v = _f32(v)
    s, qh, hd = q.shape
    kvh = k.shape[1]
    vch = _f32(v_ch_s) if v_ch_s is not None else None
    r = dict(q8=np.empty(q.shape, np.int8), q_s=np.empty((s, qh), np.float32), k8=np.empty(k.shape, np.int8),
             k_s=np.empty((s, kvh), np.float32), v8=np.empty(v.shape, np.int8), v_s=np.empty((s, kvh), np.float32),
             p8=np.empty((qh, s, s), np.int8) if want_p else None, p_s=np.empty((s, qh), np.float32),
             o=np.empty(q.shape, np.float32))
    lib().fxo_mha_prefill_dyn(_p(q), _p(k), _p(v), s, qh, kvh, hd, _p(vch), _p(r["q8"]), _p(r["q_s"]), _p(r["k8"]), _p(r["k_s"]),
                              _p(r["v8"]), _p(r["v_s"]), _p(r["p8"]), _p(r["p_s"]), _p(r["o"]))
    return r


def mha_decode_dyn(q8, q_s, k_cache, k_s, v_cache, v_s, v_ch_s=None, want_p=False):
    """q8 [qh][hd] int8 with Q_s [qh]; caches [len][kvh][hd] int8 with K_s, V_s [len][kvh] -> (o, p8, p_s)."""
    q8 = np.ascontiguousarray(q8, np.int8); q_s = _f32(q_s)
    k_cache = np.ascontiguousarray(k_cache, np.int8); v_cache = np.ascontiguousarray(v_cache, np.int8)
    k_s = _f32(k_s); v_s = _f32(v_s)
    qh, hd = q8.shape
    ln, kvh, _ = k_cache.shape
    vch = _f32(v_ch_s) if v_ch_s is not None else None
    p8 = np.empty((qh, ln), np.int8) if want_p else None
    p_s = np.empty(qh, np.float32); o = np.empty((qh, hd), np.float32)
    lib().fxo_mha_decode_dyn(_p(q8), _p(q_s), _p(k_cache), _p(k_s), _p(v_cache), _p(v_s), _p(vch), ln, qh, kvh, hd,
                             _p(p8), _p(p_s), _p(o))
    return o, p8, p_s


def half_to_float(h):
    return lib().fxo_half_to_float(int(h))


def embed(table_u16, token):
    table_u16 = np.ascontiguousarray(table_u16, np.uint16)
    y = np.empty(table_u16.shape[1], np.float32)
    lib().fxo_embed(_p(table_u16), table_u16.shape[1], int(token), _p(y))
    return y


def lm_head(table_u16, n):
    table_u16 = np.ascontiguousarray(table_u16, np.uint16)
    vocab, hidden = table_u16.shape
    n = _f32(n)
    logits = np.empty(vocab, np.float32)
    lib().fxo_lm_head(_p(table_u16), vocab, hidden, _p(n), _p(logits))
    return logits


def sample_topk(logits, top_k=5, rand=0.5, lanes=8, enable_sub_max=True):
    """Logits.h:145-279.  Returns (token, top_idx[k], top_val[k], top_prob[k])."""
    logits = _f32(logits).reshape(-1)
    n = logits.shape[0]
    assert n % lanes == 0 and top_k <= 16
    idx = np.empty(top_k, np.int32); val = np.empty(top_k, np.float32); prob = np.empty(top_k, np.float32)
    f = lib().fxo_sample_topk
    f.restype = C.c_int
    tok = f(_p(logits), n, top_k, lanes, _f(rand), int(enable_sub_max), _p(idx), _p(val), _p(prob))
    return int(tok), idx, val, prob


def pack_pref(x, tp):
    x = _f32(x); tokens, dim = x.shape
    out = np.empty((tokens // tp, dim, tp), np.float32)
    lib().fxo_pack_pref(_p(x), tokens, dim, tp, _p(out)); return out


def unpack_pref(packed, tp):
    packed = _f32(packed); blocks, dim, _ = packed.shape
    x = np.empty((blocks * tp, dim), np.float32)
    lib().fxo_unpack_pref(_p(packed), blocks * tp, dim, tp, _p(x)); return x


def pack_dec(x, bp):
    x = _f32(x); dim = x.shape[0]
    out = np.empty((dim // bp, bp), np.float32)
    lib().fxo_pack_dec(_p(x), dim, bp, _p(out)); return out


def unpack_dec(packed, bp):
    packed = _f32(packed); dim = packed.size
    x = np.empty(dim, np.float32)
    lib().fxo_unpack_dec(_p(packed), dim, bp, _p(x)); return x


# ---------------------------------------------------------------- model level

class Model(C.Structure):
    _fields_ = [(n, C.c_int) for n in
                ("layers", "hidden", "kv_hidden", "inter", "q_heads", "kv_heads", "head_dim", "vocab", "max_pos")] + \
               [("eps", C.c_float), ("fht_scale", C.c_float)] + \
               [(n, C.c_void_p) for n in
                ("wq", "wk", "wv", "wo", "wg", "wu", "wd", "sq", "sk", "sv", "so", "sg", "su", "sd",
                 "gamma", "q_s", "k_s", "v_s", "a_s", "rope_sin", "rope_cos", "embed")]


class OracleModel:
    """Wraps numpy weight arrays (see flexllm_amd.llama.synth_weights) for the oracle's model functions."""

    def __init__(self, cfg, w):
        self.cfg = cfg
        self.w = w
        self._keep = []
        L = cfg["layers"]

        def ptr_array(name):
            arrs = [np.ascontiguousarray(w[name][l]) for l in range(L)]
            self._keep.append(arrs)
            pa = (C.c_void_p * L)(*[a.ctypes.data for a in arrs])
            self._keep.append(pa)
            return C.cast(pa, C.c_void_p)

        m = Model()
        for n in ("layers", "hidden", "kv_hidden", "inter", "q_heads", "kv_heads", "head_dim", "vocab", "max_pos"):
            setattr(m, n, int(cfg[n]))
        m.eps = float(cfg["eps"]); m.fht_scale = float(cfg["fht_scale"])
        for n in ("wq", "wk", "wv", "wo", "wg", "wu", "wd", "sq", "sk", "sv", "so", "sg", "su", "sd"):
            setattr(m, n, ptr_array(n))
        for n, dt in (("gamma", np.float32), ("q_s", np.float32), ("k_s", np.float32), ("v_s", np.float32),
                      ("a_s", np.float32), ("rope_sin", np.float32), ("rope_cos", np.float32), ("embed", np.uint16)):
            a = np.ascontiguousarray(w[n], dt)
            self._keep.append(a)
            setattr(m, n, a.ctypes.data)
        self.m = m

    def new_caches(self):
        c = self.cfg
        shape = (c["layers"], c["max_pos"], c["kv_hidden"])
        return np.zeros(shape, np.int8), np.zeros(shape, np.int8)

    def decode_token(self, x_in, pos, k_cache, v_cache, want_logits=True):
        c = self.cfg
        x_in = _f32(x_in)
        hidden = np.empty(c["hidden"], np.float32)
        logits = np.empty(c["vocab"], np.float32) if want_logits else None
        lib().fxo_llama_decode_token(C.byref(self.m), _p(x_in), int(pos), _p(k_cache), _p(v_cache),
                                     _p(hidden), _p(logits))
        return hidden, logits

    def prefill(self, x_in, k_cache, v_cache):
        x_in = _f32(x_in)
        s = x_in.shape[0]
        hidden = np.empty(x_in.shape, np.float32)
        lib().fxo_llama_prefill(C.byref(self.m), _p(x_in), s, _p(k_cache), _p(v_cache), _p(hidden))
        return hidden
