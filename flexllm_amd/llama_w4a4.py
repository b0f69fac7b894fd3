"""The reference's shipped configuration - W4A4 linears (asymmetric uint4 activations x symmetric int4 weights), int8
attention, fp32 everything else - as a layer graph sequenced from the host over the library's entry points, one kernel
per stage.  The order of stages is that of the reference's task graph (SpinQuant_Llama_32_1B/SpinQuant_Prefilling.h:
807-1050 and SpinQuant_Decoding_mem_opt.h:947-1128; the same list appears stage by stage in
HMT_SpinQuant_Prefilling_mem_opt.h:948-1042):

  x -> RMSNorm -> quant u4 -> q/k/v linears -> dequant (zero point x row sum) -> RoPE(q, k) -> static int8 q (8 Q_s), k, v
    -> K/V cache -> q.K^T -> softmax -> uint8 P -> P.V -> o -> quant u4 -> o_proj -> dequant + residual
    -> RMSNorm -> quant u4 -> gate, up -> dequant -> Swish(gate) * up -> Hadamard / sqrt(n) -> quant u4 -> down
    -> dequant + residual.

This is the functional drop-in for that configuration; the benchmarked, fused path of this library is the W8A8 graph
(`llama.Llama`).  Weights: per layer and projection int4 values (int8 arrays in [-8, 7], [out][in]), per-channel scales
and row sums (`w_<proj>_s`, `w_<proj>_sum` of the reference's headers).
"""
import numpy as np

from . import ops
from .device import DeviceArray, to_device

_PROJ = ("q", "k", "v", "o", "g", "u", "d")


class LlamaW4A4:
    def __init__(self, cfg, w):
        """w: host dictionary with lists w<p> (int8 [n][k] in [-8,7]), s<p>, sum<p> (fp32 [n]) per layer for p in
        q,k,v,o,g,u,d; gamma [2L+1][hidden]; q_s, k_s, v_s, a_s [L][heads]; rope_sin, rope_cos."""
        self.cfg = cfg
        L = cfg["layers"]
        # decode streams the nibble-packed weights (half the bytes); prefill multiplies the same values held one per
        # byte on the direct-load MFMA kernel of the int8 path
        self.w8 = {p: [to_device(np.ascontiguousarray(w["w" + p][l], np.int8)) for l in range(L)] for p in _PROJ}
        self.w4 = {p: [ops.pack_nibbles(self.w8[p][l]) for l in range(L)] for p in _PROJ}
        self.ws = {p: [to_device(np.asarray(w["s" + p][l], np.float32)) for l in range(L)] for p in _PROJ}
        self.wsum = {p: [to_device(np.asarray(w["sum" + p][l], np.float32)) for l in range(L)] for p in _PROJ}
        self.gamma = [to_device(np.ascontiguousarray(w["gamma"][i], np.float32)) for i in range(2 * L + 1)]
        self.scales = [ops.Scales(w["q_s"][l], w["k_s"][l], w["v_s"][l], w["a_s"][l]) for l in range(L)]
        self.q_s = [to_device(np.asarray(w["q_s"][l], np.float32)) for l in range(L)]
        self.sin_t, self.cos_t = to_device(w["rope_sin"]), to_device(w["rope_cos"])
        self.caches = [ops.kv_cache(cfg["kv_heads"], cfg["max_pos"]) for _ in range(L)]

    # one W4A4 linear: per-token asymmetric uint4 quantisation, int4 x uint4 product, dequantisation (+ residual)
    def _linear(self, x, p, l, residual=None):
        q, s, b = ops.quant_asym_u8(x, bits=4)
        if x.shape[0] > 1 and self.w8[p][l].shape[0] % 4 == 0:
            return ops.linear_i8_gemm_dequant_asym(q, s, b, self.w8[p][l], self.ws[p][l], self.wsum[p][l], residual=residual)
        a4 = ops.pack_nibbles(q)
        if x.shape[0] == 1:
            k2 = a4.shape[-1]
            y = ops.linear_u4i4_gemv_dequant(a4.view(0, (k2,)), s, b, self.w4[p][l], self.ws[p][l], self.wsum[p][l],
                                             residual=residual.view(0, (residual.shape[-1],)) if residual is not None else None)
            return y.view(0, (1, y.shape[-1]))
        return ops.linear_u4i4_gemm_dequant(a4, s, b, self.w4[p][l], self.ws[p][l], self.wsum[p][l], residual=residual)

    def _layer(self, x, l, pos0):
        c = self.cfg
        S, H, KV, hd = x.shape[0], c["hidden"], c["kv_hidden"], c["head_dim"]
        kc, vc = self.caches[l]
        n = ops.rmsnorm_f32(x, self.gamma[2 * l], eps=c["eps"])
        q = self._linear(n, "q", l); k = self._linear(n, "k", l); v = self._linear(n, "v", l)
        q = ops.rope_f32(q.view(0, (S, c["q_heads"], hd)), self.sin_t, self.cos_t, pos0)
        k = ops.rope_f32(k.view(0, (S, c["kv_heads"], hd)), self.sin_t, self.cos_t, pos0)
        q8 = ops.static_quant_i8(q, self.q_s[l], factor=8.0)
        ops.kv_append_i8(k, v.view(0, (S, c["kv_heads"], hd)), kc, vc, self.scales[l], pos0)
        if S == 1:
            o, _ = ops.mha_i8_decode(q8.view(0, (c["q_heads"], hd)), kc, vc, self.scales[l], pos0 + 1)
        else:
            assert pos0 == 0, "prefill starts at position 0"
            o, _ = ops.mha_i8_prefill(q8, kc, vc, self.scales[l])
        x2 = self._linear(o.view(0, (S, H)), "o", l, residual=x)
        n2 = ops.rmsnorm_f32(x2, self.gamma[2 * l + 1], eps=c["eps"])
        gate = self._linear(n2, "g", l); up = self._linear(n2, "u", l)
        h = ops.swiglu_f32(gate, up)
        hf = ops.fht_f32(h, c["fht_scale"])
        return self._linear(hf, "d", l, residual=x2)

    def prefill_hidden(self, x):
        """x: device fp32 [S][hidden], S a multiple of 32; fills the caches from position 0; returns the residual
        stream after the last layer."""
        for l in range(self.cfg["layers"]):
            x = self._layer(x, l, 0)
        return x

    def decode_hidden(self, x, pos):
        """x: device fp32 [hidden], one token at position pos."""
        x = x.view(0, (1, self.cfg["hidden"]))
        for l in range(self.cfg["layers"]):
            x = self._layer(x, l, pos)
        return x.view(0, (self.cfg["hidden"],))

    def final_norm(self, hidden):
        return ops.rmsnorm_f32(hidden.view(0, (1, self.cfg["hidden"])), self.gamma[2 * self.cfg["layers"]], eps=self.cfg["eps"])
