"""Writes tests/golden/modules_small.npz: small seeded inputs and the outputs of the CPU oracle for them.

The reference ships no stored vectors for this path (its testbenches draw random inputs and compute their goldens
in-process), so these are regression vectors of THIS repository's oracle, taken after the oracle was pinned by the
independent checks of tests/test_oracle_pins.py.  They serve two purposes: the CPU suite notices if the oracle ever
changes its answers, and the GPU suite has fixed data to compare the device path with, independent of the oracle build.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

OUT = os.path.join(HERE, "modules_small.npz")


def cases(o):
    """name -> array, in a flat dictionary; `in_` prefixes inputs, `out_` expected outputs."""
    r = np.random.default_rng(20240607)
    g = {}
    # quant.h: per-token symmetric int8 and asymmetric uint4
    x = (r.standard_normal((6, 256)) * 3).astype(np.float32)
    x[1] = 0.0                                                   # an all-zero token (scale falls back to 1)
    g["quant_in_x"] = x
    g["quant_out_q8"], g["quant_out_s8"] = o.quant_sym(x)
    g["quant_out_q4"], g["quant_out_s4"], g["quant_out_b4"] = o.quant_asym(x, 4)
    # Linear_Layer.h: int8 x int8 -> int32, dequantisation
    a = r.integers(-128, 128, (8, 128)).astype(np.int8)
    w = r.integers(-128, 128, (48, 128)).astype(np.int8)
    s_x = r.uniform(0.01, 0.03, 8).astype(np.float32)
    w_s = r.uniform(1e-3, 1e-2, 48).astype(np.float32)
    g["linear_in_a"], g["linear_in_w"], g["linear_in_sx"], g["linear_in_ws"] = a, w, s_x, w_s
    g["linear_out_acc"] = o.linear_i8(a, w)
    g["linear_out_y"] = o.dequant(g["linear_out_acc"], s_x, w_s)
    # FHT.h
    xf = r.standard_normal((3, 1024)).astype(np.float32)
    g["fht_in_x"] = xf
    g["fht_out_y"] = o.fht(xf, 32.0)
    # LayerNorm.h
    xn = (r.standard_normal((4, 256)) * 2).astype(np.float32)
    gam = r.uniform(0.5, 1.5, 256).astype(np.float32)
    g["rmsnorm_in_x"], g["rmsnorm_in_gamma"] = xn, gam
    g["rmsnorm_out_y"] = o.rmsnorm_pref(xn, gam, 1e-5)
    # RoPE.h
    sin_t, cos_t = o.rope_table(128)
    xr = r.standard_normal((5, 3, 64)).astype(np.float32)
    g["rope_in_x"], g["rope_in_sin"], g["rope_in_cos"] = xr, sin_t, cos_t
    g["rope_out_y"] = o.rope(xr, sin_t, cos_t, 64)
    # Swish.h / gate
    ga = (r.standard_normal((2, 128)) * 3).astype(np.float32)
    up = r.standard_normal((2, 128)).astype(np.float32)
    g["swiglu_in_gate"], g["swiglu_in_up"] = ga, up
    g["swiglu_out_h"] = o.gate(o.swish(ga), up)
    # MHA_i8xi8.h: prefill attention with static scales (4 query heads on 2 KV heads), then one decode step
    S, QH, KVH, HD = 48, 4, 2, 64
    q = r.standard_normal((S, QH, HD)).astype(np.float32)
    k = r.standard_normal((S, KVH, HD)).astype(np.float32)
    v = r.standard_normal((S, KVH, HD)).astype(np.float32)
    q_s = np.full(QH, 4.2 / 127, np.float32); k_s = np.full(KVH, 4.5 / 127, np.float32)
    v_s = np.full(KVH, 4.4 / 127, np.float32); a_s = np.full(QH, 1.0 / 255, np.float32)
    g["mha_in_q"], g["mha_in_k"], g["mha_in_v"] = q, k, v
    g["mha_in_qs"], g["mha_in_ks"], g["mha_in_vs"], g["mha_in_as"] = q_s, k_s, v_s, a_s
    res = o.mha_prefill(q, k, v, q_s, k_s, v_s, a_s, want_p=True)
    for key in ("q8", "k8", "v8", "p8", "o"):
        g["mha_out_" + key] = res[key]
    qd = r.integers(-128, 128, (QH, HD)).astype(np.int8)
    g["mhadec_in_q8"] = qd
    g["mhadec_out_o"], g["mhadec_out_p8"] = o.mha_decode(qd, res["k8"], res["v8"], q_s, k_s, v_s, a_s, want_p=True)
    # Logits.h: fp16 output head and top-k sampling
    table = (r.standard_normal((96, 128)) * 0.05).astype(np.float16).view(np.uint16)
    nvec = r.standard_normal(128).astype(np.float32)
    g["head_in_table"], g["head_in_n"] = table, nvec
    g["head_out_logits"] = o.lm_head(table, nvec)
    lg = (r.standard_normal(512) * 4).astype(np.float32)
    g["topk_in_logits"] = lg
    g["topk_in_rand"] = np.array([0.0, 0.27, 0.61, 0.97], np.float32)
    toks, idxs, vals, probs = [], [], [], []
    for rnd in g["topk_in_rand"]:
        t, i, vv, p = o.sample_topk(lg, 5, float(rnd), 8)
        toks.append(t); idxs.append(i); vals.append(vv); probs.append(p)
    g["topk_out_token"] = np.array(toks, np.int32)
    g["topk_out_idx"], g["topk_out_val"], g["topk_out_prob"] = np.stack(idxs), np.stack(vals), np.stack(probs)
    # W4A4 linear (quant.h asymmetric uint4 x int4 weights)
    x4 = r.standard_normal((4, 128)).astype(np.float32)
    w4 = r.integers(-8, 8, (32, 128)).astype(np.int8)
    w4s = r.uniform(0.01, 0.05, 32).astype(np.float32)
    w4sum = (w4.astype(np.float32).sum(1) * w4s).astype(np.float32)
    g["w4a4_in_x"], g["w4a4_in_w"], g["w4a4_in_ws"], g["w4a4_in_wsum"] = x4, w4, w4s, w4sum
    g["w4a4_out_y"] = o.w4a4_linear(x4, w4, w4s, w4sum)
    # HMT.h: memory retrieval over 8 slots
    hq = r.standard_normal(64).astype(np.float32)
    km = r.standard_normal((8, 64)).astype(np.float32); km[5:] = 0.0      # empty slots take part in the softmax
    mm = r.standard_normal((8, 64)).astype(np.float32); mm[5:] = 0.0
    g["hmt_in_q"], g["hmt_in_kmem"], g["hmt_in_mmem"] = hq, km, mm
    g["hmt_out_a"], g["hmt_out_p"] = o.hmt_retrieve(hq, km, mm, 8.0)
    return g


def main():
    from oracle import oracle as o
    o.build()
    g = cases(o)
    np.savez_compressed(OUT, **g)
    print("wrote %s: %d arrays, %d bytes" % (OUT, len(g), os.path.getsize(OUT)))


if __name__ == "__main__":
    main()
