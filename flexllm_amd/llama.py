"""Llama-3.2-1B W8A8 SpinQuant graph: configuration, seeded synthetic weights (host and device, bit-identical)
and the wrapper over the C ABI model object (flexllm_llama_*)."""
import ctypes as C
import math

import numpy as np

from . import synth
from ._lib import lib, check, LlamaConfig, LlamaWeights, LlamaW4A4Weights
from .device import DeviceArray, to_device, _s
from .ops import rope_table

# Model constants of the reference (Modules/config.h:19-44 of the reference tree).
LLAMA32_1B = dict(layers=16, hidden=2048, kv_hidden=512, inter=8192, q_heads=32, kv_heads=8, head_dim=64,
                  vocab=128256, max_pos=4096, eps=1e-5, fht_scale=90.50966799)

_PROJ = dict(q=("hidden", "hidden"), k=("kv_hidden", "hidden"), v=("kv_hidden", "hidden"), o=("hidden", "hidden"),
             g=("inter", "hidden"), u=("inter", "hidden"), d=("hidden", "inter"))


def make_config(**over):
    cfg = dict(LLAMA32_1B)
    cfg.update(over)
    return cfg


def _seed(base, layer, tensor):
    return (base * 1000003 + layer * 101 + tensor) & 0xFFFFFFFFFFFF


def synth_weights(cfg, seed=1, device=False, embed_range=1.7):
    """Random-init int8 weights U[-127,127] with per-channel scales sized so that activations stay O(1),
    RMSNorm gains U[0.5,1.5], static attention scales with a seeded +-20% jitter per head, fp16 embedding
    U[-embed_range, embed_range] (with the default range a token's own row wins the tied head by a wide margin; a
    range of a few hundredths gives logits of order one and top-k distributions with several live candidates).
    device=False -> numpy arrays on the host; device=True -> DeviceArrays filled on the GPU by the
    same counter-based generator."""
    i8 = synth.device_i8 if device else synth.host_i8
    f32 = synth.device_uniform_f32 if device else synth.host_uniform_f32
    f16 = synth.device_uniform_f16 if device else synth.host_uniform_f16
    w = {}
    for t, (name, (n_key, k_key)) in enumerate(_PROJ.items()):
        n, k = cfg[n_key], cfg[k_key]
        base = 1.0 / (73.0 * math.sqrt(k))
        w["w" + name] = [i8((n, k), _seed(seed, l, t)) for l in range(cfg["layers"])]
        w["s" + name] = [f32((n,), _seed(seed, l, 20 + t), 0.5 * base, 1.5 * base) for l in range(cfg["layers"])]
    L = cfg["layers"]
    w["gamma"] = f32((2 * L + 1, cfg["hidden"]), _seed(seed, 99, 1), 0.5, 1.5)
    w["q_s"] = f32((L, cfg["q_heads"]), _seed(seed, 99, 2), 0.8 * 0.004, 1.2 * 0.004)
    w["k_s"] = f32((L, cfg["kv_heads"]), _seed(seed, 99, 3), 0.8 * 0.03, 1.2 * 0.03)
    w["v_s"] = f32((L, cfg["kv_heads"]), _seed(seed, 99, 4), 0.8 * 0.03, 1.2 * 0.03)
    w["a_s"] = f32((L, cfg["q_heads"]), _seed(seed, 99, 5), 1.0 / 255, 1.0 / 255)
    w["embed"] = f16((cfg["vocab"], cfg["hidden"]), _seed(seed, 99, 6), -embed_range, embed_range)
    sin_t, cos_t = rope_table(cfg["max_pos"], cfg["head_dim"])
    if device:
        w["rope_sin"], w["rope_cos"] = to_device(sin_t), to_device(cos_t)
    else:
        w["rope_sin"], w["rope_cos"] = sin_t, cos_t
        w["embed"] = w["embed"].view(np.uint16)
    return w


def synth_weights_w4a4(cfg, seed=1, device=False, embed_range=1.7):
    """Random-init weights of the W4A4 configuration: int4 values U[-8,7] held one per byte, per-channel scales sized
    so that activations stay O(1), the row sums of the dequantised weights (`sum<p>`, the generated headers'
    w_<proj>_sum), an int4 output head (`head_w`, `head_s`, `head_sum`) and everything synth_weights gives besides the
    matrices.  device as in synth_weights; the row sums of device matrices are taken on the device too (a GEMV with
    a vector of ones)."""
    w = synth_weights(cfg, seed, device, embed_range)
    i8 = synth.device_i8 if device else synth.host_i8
    f32 = synth.device_uniform_f32 if device else synth.host_uniform_f32

    def row_sums(q, s):
        if not device:
            return (q.sum(1, dtype=np.int64).astype(np.float32) * s).astype(np.float32)
        from . import ops
        tot = ops.linear_i8_gemv(to_device(np.ones(q.shape[1], np.int8)), q).numpy()
        return to_device((tot.astype(np.float32) * s.numpy()).astype(np.float32))

    for t, (name, (n_key, k_key)) in enumerate(_PROJ.items()):
        n, k = cfg[n_key], cfg[k_key]
        base = 1.0 / (4.6 * math.sqrt(k))
        w["w" + name] = [i8((n, k), _seed(seed, l, 40 + t), -8, 7) for l in range(cfg["layers"])]
        w["s" + name] = [f32((n,), _seed(seed, l, 60 + t), 0.5 * base, 1.5 * base) for l in range(cfg["layers"])]
        w["sum" + name] = [row_sums(w["w" + name][l], w["s" + name][l]) for l in range(cfg["layers"])]
    V, H = cfg["vocab"], cfg["hidden"]
    base = 1.0 / (4.6 * math.sqrt(H))
    w["head_w"] = i8((V, H), _seed(seed, 99, 7), -8, 7)
    w["head_s"] = f32((V,), _seed(seed, 99, 8), 0.5 * base, 1.5 * base)
    w["head_sum"] = row_sums(w["head_w"], w["head_s"])
    return w


class Llama:
    """Device model object.  `weights` holds DeviceArrays (see synth_weights(device=True)); with the keys of
    synth_weights_w4a4 (`sum<p>`, `head_w`, ...) it is the W4A4 model (flexllm_llama_create_w4a4): it decodes in the
    persistent kernel's W4A4 instance, and prefill_hidden / generate run the W4A4 prefill graph (uint4 activations x int4
    weights held one per byte on the int8 MFMA kernel, asymmetric dequantisation in the epilogues)."""

    def __init__(self, cfg, weights):
        self.cfg = cfg
        c = LlamaConfig()
        for n in ("layers", "hidden", "kv_hidden", "inter", "q_heads", "kv_heads", "head_dim", "vocab", "max_pos"):
            setattr(c, n, int(cfg[n]))
        c.eps = float(cfg["eps"]); c.fht_scale = float(cfg["fht_scale"])
        L = cfg["layers"]
        keep = []
        w = LlamaWeights()
        for n in ("wq", "wk", "wv", "wo", "wg", "wu", "wd", "sq", "sk", "sv", "so", "sg", "su", "sd"):
            arr = (C.c_void_p * L)(*[weights[n][l].ptr for l in range(L)])
            keep.append(arr)
            setattr(w, n, C.cast(arr, C.c_void_p))
        for n in ("gamma", "q_s", "k_s", "v_s", "a_s", "rope_sin", "rope_cos", "embed"):
            setattr(w, n, weights[n].ptr)
        self._gamma, self._embed = weights["gamma"], weights["embed"]
        h = C.c_void_p()
        self.w4a4 = "sumq" in weights
        if self.w4a4:
            w4 = LlamaW4A4Weights()
            w4.base = w
            for n in ("sumq", "sumk", "sumv", "sumo", "sumg", "sumu", "sumd"):
                arr = (C.c_void_p * L)(*[weights[n][l].ptr for l in range(L)])
                keep.append(arr)
                setattr(w4, n, C.cast(arr, C.c_void_p))
            for n in ("head_w", "head_s", "head_sum"):
                setattr(w4, n, weights[n].ptr)
            check(lib().flexllm_llama_create_w4a4(C.byref(h), C.byref(c), C.byref(w4)))
        else:
            check(lib().flexllm_llama_create(C.byref(h), C.byref(c), C.byref(w)))
        self.handle = h
        cache_shape_k = (L, cfg["kv_heads"], cfg["max_pos"], cfg["head_dim"])
        cache_shape_v = (L, cfg["kv_heads"], cfg["max_pos"] // 64, cfg["head_dim"], 64)
        kp, vp = C.c_void_p(), C.c_void_p()
        check(lib().flexllm_llama_kv_cache(self.handle, C.byref(kp), C.byref(vp)))
        self.k_cache = _borrow(kp.value, cache_shape_k, np.int8)
        self.v_cache = _borrow(vp.value, cache_shape_v, np.int8)

    def decode_hidden(self, x_in, pos, want_logits=False, stream=None):
        hidden = DeviceArray((self.cfg["hidden"],), np.float32)
        logits = DeviceArray((self.cfg["vocab"],), np.float32) if want_logits else None
        check(lib().flexllm_llama_decode_hidden(self.handle, C.c_void_p(x_in.ptr), int(pos), C.c_void_p(hidden.ptr),
                                                C.c_void_p(logits.ptr) if logits else None, _s(stream)))
        return hidden, logits

    def decode_greedy(self, token_io, pos0, steps, tokens_out, use_graph=True, stream=None):
        check(lib().flexllm_llama_decode_greedy(self.handle, C.c_void_p(token_io.ptr), int(pos0), int(steps),
                                                C.c_void_p(tokens_out.ptr), int(use_graph), _s(stream)))

    def decode_sample(self, token_io, pos0, steps, rands, top_k, tokens_out, stream=None):
        """Top-k sampling loop; rands: device float32 [steps] in [0,1)."""
        check(lib().flexllm_llama_decode_sample(self.handle, C.c_void_p(token_io.ptr), int(pos0), int(steps),
                                                C.c_void_p(rands.ptr), int(top_k), C.c_void_p(tokens_out.ptr), _s(stream)))

    def generate(self, prompt, steps, top_k=0, rands=None, stream=None):
        """Prompt (host sequence of token ids) -> `steps` generated ids (host list): prefill of all prompt tokens but
        the last, then the decode loop from the last one, greedy (top_k = 0) or top-k sampling with the host-supplied
        uniform numbers `rands` - the flow of SpinQuant_Prefilling_Decoding_mem_opt_tb.cpp:753-930."""
        prompt = np.ascontiguousarray(prompt, np.int32).reshape(-1)
        d_prompt = to_device(prompt)
        out = DeviceArray((max(int(steps), 1),), np.int32)
        if top_k and rands is None:
            raise ValueError("top-k sampling needs `rands`, one uniform number in [0,1) per step")
        d_rands = to_device(np.ascontiguousarray(rands, np.float32).reshape(-1)) if top_k else None
        if top_k and d_rands.size < steps:
            raise ValueError("%d uniform numbers for %d steps" % (d_rands.size, steps))
        check(lib().flexllm_llama_generate(self.handle, C.c_void_p(d_prompt.ptr), int(prompt.size), int(steps),
                                           C.c_void_p(d_rands.ptr) if d_rands is not None else None, int(top_k),
                                           C.c_void_p(out.ptr), _s(stream)))
        if stream is not None:
            stream.sync()
        self.check()
        return out.numpy()[:int(steps)].tolist()

    def generate_int4_head(self, token, pos0, steps, rands, top_k, head, embed_f32=None):
        """The reference's generation loop with its int4 output head and top-k sampling (SpinQuant_Decoding_mem_opt.h:
        924-940, Modules/Logits.h:145-279), sequenced from the host: embedding -> layer stack -> final RMSNorm ->
        `ops.lm_head_u4i4` -> `ops.sample_topk_f32` -> next token.  head = (w4, w_s, w_sum) device arrays
        (nibble-packed int4 [vocab_pad][hidden/2], fp32 [vocab_pad] each); rands: host floats in [0,1), one per step;
        embed_f32: optional device fp32 [vocab][hidden] table (the reference's embedding file), else the model's fp16
        table.  Returns the sampled token ids (host list)."""
        from . import ops
        hidden = self.cfg["hidden"]
        w4, w_s, w_sum = head
        gamma_final = self._gamma.view(2 * self.cfg["layers"] * hidden * 4, (hidden,), np.float32)
        out = []
        tok = int(token)
        rows = embed_f32.shape[0] if embed_f32 is not None else self._embed.shape[0]
        for i in range(int(steps)):
            if not 0 <= tok < rows:
                # the head may have more rows than the embedding table (padding rows): such an id has no embedding
                raise ValueError("step %d: token id %d outside the embedding table (%d rows)" % (i, tok, rows))
            if embed_f32 is not None:
                x = embed_f32.view(tok * hidden * 4, (hidden,), np.float32)
            else:
                x = ops.embed_f16(self._embed, to_device(np.array([tok], np.int32)))
            hid, _ = self.decode_hidden(x, pos0 + i, want_logits=False)
            n_vec = ops.rmsnorm_f32(hid.view(0, (1, hidden)), gamma_final, eps=self.cfg["eps"])
            logits = ops.lm_head_u4i4(n_vec.view(0, (hidden,)), w4, w_s, w_sum)
            tok, _, _, _ = ops.sample_topk_f32(logits, top_k=top_k, rand=float(rands[i]))
            out.append(tok)
        return out

    def set_decode_mode(self, mode):
        """0: persistent one-kernel-per-token schedule (default), 1: one kernel per stage."""
        check(lib().flexllm_llama_set_decode_mode(self.handle, int(mode)))

    def exchange_info(self):
        """How the persistent decode kernel's exchange memory was placed at creation: {"two_copies": bool (one copy of
        every exchanged array per I/O die, each in that die's memory), "die_mask": int (bit x = die of XCD x),
        "near_us", "far_us": measured exchange round through own-die / other-die memory}."""
        two, mask, near, far = C.c_int(0), C.c_uint(0), C.c_float(0.0), C.c_float(0.0)
        check(lib().flexllm_llama_exchange_info(self.handle, C.byref(two), C.byref(mask), C.byref(near), C.byref(far)))
        return {"two_copies": bool(two.value), "die_mask": int(mask.value), "near_us": float(near.value), "far_us": float(far.value)}

    def check(self):
        """Synchronise and raise if the persistent decode kernel reported a barrier time-out."""
        check(lib().flexllm_llama_check(self.handle))

    def prefill_hidden(self, x_in, stream=None, out=None):
        s = x_in.shape[0]
        hidden = out if out is not None else DeviceArray((s, self.cfg["hidden"]), np.float32)
        if hidden.shape != (s, self.cfg["hidden"]) or hidden.dtype != np.float32:
            raise ValueError("out must be float32 [%d][%d]" % (s, self.cfg["hidden"]))
        check(lib().flexllm_llama_prefill_hidden(self.handle, C.c_void_p(x_in.ptr), s, C.c_void_p(hidden.ptr), _s(stream)))
        return hidden

    def caches_token_major(self):
        """int8 caches as numpy [layer][pos][kv_hidden] (token-major)."""
        c = self.cfg
        k = self.k_cache.numpy().transpose(0, 2, 1, 3).reshape(c["layers"], c["max_pos"], c["kv_hidden"])
        v = self.v_cache.numpy().transpose(0, 2, 4, 1, 3).reshape(c["layers"], c["max_pos"], c["kv_hidden"])
        return k, v

    def load_caches_token_major(self, k, v):
        c = self.cfg
        L, P, KH, HD = c["layers"], c["max_pos"], c["kv_heads"], c["head_dim"]
        self.k_cache.copy_from(np.ascontiguousarray(k.reshape(L, P, KH, HD).transpose(0, 2, 1, 3)))
        self.v_cache.copy_from(np.ascontiguousarray(v.reshape(L, P // 64, 64, KH, HD).transpose(0, 3, 1, 4, 2)))

    def close(self):
        if self.handle:
            lib().flexllm_llama_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _borrow(ptr, shape, dtype):
    a = DeviceArray.__new__(DeviceArray)
    a.shape = tuple(shape); a.dtype = np.dtype(dtype)
    a.nbytes = int(np.prod(shape, dtype=np.int64)) * a.dtype.itemsize
    a.ptr = ptr; a._owner = False
    return a
