"""ctypes binding of libflexllm_hip.so.  The library must have been built (python -m flexllm_amd.build);
there is deliberately no fallback path."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libflexllm_hip.so")


class LibraryMissing(RuntimeError):
    pass


class FlexLLMError(RuntimeError):
    pass


class MhaScales(C.Structure):
    _fields_ = [("q_s", C.c_void_p), ("k_s", C.c_void_p), ("v_s", C.c_void_p), ("a_s", C.c_void_p)]


class MhaDynScales(C.Structure):
    _fields_ = [("q_s", C.c_void_p), ("k_s", C.c_void_p), ("v_s", C.c_void_p), ("v_ch_s", C.c_void_p),
                ("q_scale_div", C.c_float)]


class LlamaConfig(C.Structure):
    _fields_ = [(n, C.c_int) for n in
                ("layers", "hidden", "kv_hidden", "inter", "q_heads", "kv_heads", "head_dim", "vocab", "max_pos")] + \
               [("eps", C.c_float), ("fht_scale", C.c_float)]


class LlamaWeights(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in
                ("wq", "wk", "wv", "wo", "wg", "wu", "wd", "sq", "sk", "sv", "so", "sg", "su", "sd",
                 "gamma", "q_s", "k_s", "v_s", "a_s", "rope_sin", "rope_cos", "embed")]


class LlamaW4A4Weights(C.Structure):
    _fields_ = [("base", LlamaWeights)] + [(n, C.c_void_p) for n in
                ("sumq", "sumk", "sumv", "sumo", "sumg", "sumu", "sumd", "head_w", "head_s", "head_sum")]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise LibraryMissing(
                "%s not found: build it with `python -m flexllm_amd.build` (hipcc, gfx950). "
                "There is no CPU fallback." % LIB_PATH)
        _lib = C.CDLL(LIB_PATH)
        _lib.flexllm_last_error.restype = C.c_char_p
        _lib.flexllm_build_info.restype = C.c_char_p
        # Every entry point with a size_t parameter is typed: an untyped Python int is passed as a 32-bit C int, which
        # would silently cut a size of 4 GiB to zero.
        vp, sz, i, u64, f = C.c_void_p, C.c_size_t, C.c_int, C.c_uint64, C.c_float
        for name, args in (("flexllm_rt_malloc", [vp, sz]), ("flexllm_rt_mem_info", [vp, vp]),
                           ("flexllm_rt_memcpy_h2d", [vp, vp, sz, vp]), ("flexllm_rt_memcpy_d2h", [vp, vp, sz, vp]),
                           ("flexllm_rt_memcpy_d2d", [vp, vp, sz, vp]), ("flexllm_rt_memset", [vp, i, sz, vp]),
                           ("flexllm_rt_fill_i8", [vp, sz, u64, i, i, vp]), ("flexllm_rt_fill_uniform_f32", [vp, sz, u64, f, f, vp]),
                           ("flexllm_rt_fill_uniform_f16", [vp, sz, u64, f, f, vp]),
                           ("flexllm_probe_hbm_read", [vp, sz, i, i, vp, vp]), ("flexllm_pack_nibbles", [vp, vp, sz, vp]),
                           ("flexllm_swish_f32", [vp, vp, sz, vp]), ("flexllm_swiglu_f32", [vp, vp, vp, sz, vp]),
                           ("flexllm_residual_add_f32", [vp, vp, vp, sz, vp])):
            getattr(_lib, name).argtypes = args
    return _lib


def check(rc):
    if rc != 0:
        raise FlexLLMError("flexllm error %d: %s" % (rc, lib().flexllm_last_error().decode()))
