"""Reads and writes a model in the reference's on-disk parameter format (directory `parameters/`).

What the reference's testbench reads (SpinQuant_Llama_32_1B/SpinQuant_Prefilling_Decoding_mem_opt_tb.cpp):
  * `<proj>_L%02d.bin` for proj in q_proj, k_proj, v_proj, o_proj, gate_proj, up_proj, down_proj: one signed byte
    per weight, row-major [out_channel][in_channel] (:30-47, :385-429)
  * `model_embed_tokens_fp32.bin`: fp32 [vocab][hidden], one row per token id (:150-172, :579)
  * generated headers with C arrays (:435-443): `w_<proj>_s_sum.h` holding `w_<proj>_s[layers][out]` (per-channel
    weight scale) and `w_<proj>_sum[layers][out]` (row sums, used by the asymmetric 4-bit path only),
    `w_rmsnorm.h` holding `RMSNorm_weight[2*layers+1][hidden]` (:485-486, :727-734: rows 2l and 2l+1 are layer l's
    two norms, the last row the final norm)
  * `Q_s.h`, `K_s.h`, `V_s.h`, `A_s.h`: static attention scales `Q_s[layers][q_heads]`, `K_s[layers][kv_heads]`,
    `V_s[layers][kv_heads]`, `A_s[layers][q_heads]` (SpinQuant_Llama_32_1B/MHA_i8xi8.h:11-14, :32, :63, :245)

The reference tree ships none of these files, so the header syntax is taken from how the arrays are indexed: any C
initialiser `name[d0][d1] = { ... }` (or one-dimensional) is accepted, numbers are C floating literals (decimal or
hexadecimal, with or without an `f` suffix).  The rotary
table (`parameters/RoPE_sin_cos.h`) is regenerated from the formula.  For the W8A8 model the output head is the
embedding matrix in fp16 (tied) and `lm_head.bin` / `w_lm_head_lm_head.h` are not read; with w4a4=True the loader also
returns the row sums (`sum<p>`) and the int4 output head (`lm_head.bin`, row-major int8 `[vocab][hidden]` holding -8..7,
with `w_lm_head_lm_head_s[vocab]` and `w_lm_head_lm_head_sum[vocab]`, SpinQuant_Prefilling_Decoding_mem_opt_tb.cpp:
187-192, 442, 655-660, 716-719; the file's row count is not pinned by anything the reference ships - the testbench
reads the padded vocabulary's rows from it - so any whole number of rows >= vocab is accepted): the dictionary `llama.Llama` turns into the W4A4 model.  A row sum is the sum of the
row's DEQUANTISED weights (the zero point of the activations multiplies it directly, Modules/quant.h:147-152; the
linear testbench accumulates qval * scale, Linear_Layer_Decoding_tb.cpp:171-188).

`save_reference_parameters` writes the same files from a host weight dictionary, e.g. to hand a synthetic model to
the reference's own testbench.
"""
import os
import re

import numpy as np

from .device import to_device
from .ops import rope_table

_PROJ_FILES = dict(q="q_proj", k="k_proj", v="v_proj", o="o_proj", g="gate_proj", u="up_proj", d="down_proj")
_PROJ_DIMS = dict(q=("hidden", "hidden"), k=("kv_hidden", "hidden"), v=("kv_hidden", "hidden"), o=("hidden", "hidden"),
                  g=("inter", "hidden"), u=("inter", "hidden"), d=("hidden", "inter"))
_STATIC = dict(q_s=("Q_s", "q_heads"), k_s=("K_s", "kv_heads"), v_s=("V_s", "kv_heads"), a_s=("A_s", "q_heads"))
# a C floating literal: hexadecimal (0x1.8p-3) or decimal, with an optional f/F/l/L suffix that is dropped
_NUM = re.compile(r"[-+]?(?:0[xX](?:[0-9a-fA-F]+\.?[0-9a-fA-F]*|\.[0-9a-fA-F]+)(?:[pP][-+]?\d+)?"
                  r"|(?:\d+\.\d*|\.\d+|\d+)(?:[eE][-+]?\d+)?)")


def _c_float(tok):
    return float.fromhex(tok) if "x" in tok or "X" in tok else float(tok)


class ParameterError(ValueError):
    pass


def parse_c_array(text, name):
    """The float32 array initialised as `name[d0]...[dn] = { ... }` in C source `text`, shaped by its declared
    dimensions when all of them are integer literals, flat otherwise.  Comments are ignored."""
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    text = re.sub(r"//[^\n]*", " ", text)
    m = re.search(r"\b" + re.escape(name) + r"\s*((?:\[\s*\w*\s*\]\s*)+)=\s*\{", text)
    if not m:
        raise ParameterError("array %s not found" % name)
    dims = re.findall(r"\[\s*(\w*)\s*\]", m.group(1))
    depth, i = 1, m.end()
    while depth and i < len(text):
        depth += {"{": 1, "}": -1}.get(text[i], 0)
        i += 1
    if depth:
        raise ParameterError("array %s: unbalanced braces" % name)
    body = text[m.end():i - 1]
    with np.errstate(over="ignore"):
        vals = np.array([_c_float(v) for v in _NUM.findall(body)], dtype=np.float64).astype(np.float32)
    if not all(d.isdigit() for d in dims):
        return vals                                # sizes given by macros or left open: flat, the caller knows the shape
    shape = [int(d) for d in dims]
    if vals.size != int(np.prod(shape)):
        raise ParameterError("array %s: %d values do not fit %s" % (name, vals.size, shape))
    return vals.reshape(shape)


def _read_header_array(param_dir, fname, name, shape, padded=False):
    """padded=True accepts a one-dimensional array longer than `shape` (an export padded to the reference's
    VOCAB_SIZE_PAD) and returns its first entries."""
    path = os.path.join(param_dir, fname)
    if not os.path.exists(path):
        raise ParameterError("missing %s" % path)
    with open(path) as f:
        arr = parse_c_array(f.read(), name)
    want = int(np.prod(shape))
    if padded and arr.size > want:
        arr = arr.reshape(-1)[:want]
    if arr.size != want:
        raise ParameterError("%s: %s has %d values, expected %s" % (path, name, arr.size, shape))
    return np.ascontiguousarray(arr.reshape(shape))


def load_reference_parameters(param_dir, cfg, device=True, w4a4=False):
    """Weight dictionary for `llama.Llama` from a reference `parameters/` directory.  device=False returns numpy
    arrays (the layout of `llama.synth_weights(device=False)`).  w4a4=True adds the row sums and the int4 output head
    (the layout of `llama.synth_weights_w4a4`)."""
    L, H = cfg["layers"], cfg["hidden"]
    w = {}
    for key, stem in _PROJ_FILES.items():
        n, k = cfg[_PROJ_DIMS[key][0]], cfg[_PROJ_DIMS[key][1]]
        mats = []
        for l in range(L):
            path = os.path.join(param_dir, "%s_L%02d.bin" % (stem, l))
            if not os.path.exists(path):
                raise ParameterError("missing %s" % path)
            if os.path.getsize(path) != n * k:
                raise ParameterError("%s: %d bytes, expected %d x %d" % (path, os.path.getsize(path), n, k))
            mats.append(np.fromfile(path, dtype=np.int8).reshape(n, k))
        w["w" + key] = mats
        s = _read_header_array(param_dir, "w_%s_s_sum.h" % stem, "w_%s_s" % stem, (L, n))
        w["s" + key] = [np.ascontiguousarray(s[l]) for l in range(L)]
        if w4a4:
            sm = _read_header_array(param_dir, "w_%s_s_sum.h" % stem, "w_%s_sum" % stem, (L, n))
            w["sum" + key] = [np.ascontiguousarray(sm[l]) for l in range(L)]
            for l in range(L):
                if mats[l].min() < -8 or mats[l].max() > 7:
                    raise ParameterError("%s_L%02d.bin holds values outside -8..7: not an int4 export" % (stem, l))
    w["gamma"] = _read_header_array(param_dir, "w_rmsnorm.h", "RMSNorm_weight", (2 * L + 1, H))
    for key, (name, heads) in _STATIC.items():
        w[key] = _read_header_array(param_dir, name + ".h", name, (L, cfg[heads]))
    path = os.path.join(param_dir, "model_embed_tokens_fp32.bin")
    if not os.path.exists(path):
        raise ParameterError("missing %s" % path)
    if os.path.getsize(path) != 4 * cfg["vocab"] * H:
        raise ParameterError("%s: %d bytes, expected fp32 %d x %d" % (path, os.path.getsize(path), cfg["vocab"], H))
    embed = np.memmap(path, dtype=np.float32, mode="r", shape=(cfg["vocab"], H))
    w["embed"] = np.asarray(embed).astype(np.float16).view(np.uint16)      # tied fp16 table (round to nearest even)
    w["rope_sin"], w["rope_cos"] = rope_table(cfg["max_pos"], cfg["head_dim"])
    if w4a4:
        path = os.path.join(param_dir, "lm_head.bin")
        if not os.path.exists(path):
            raise ParameterError("missing %s" % path)
        # The testbench reads VOCAB_SIZE_PAD (131072) rows from this file and VOCAB_SIZE (128256) scale pairs
        # (:196-201, :716-719); no such file ships with the reference, so its row count is not pinned: any whole
        # number of rows >= vocab is accepted and the first vocab rows are used, likewise for the two arrays.
        size = os.path.getsize(path)
        if size < cfg["vocab"] * H or size % H:
            raise ParameterError("%s: %d bytes, expected at least %d whole rows of %d" % (path, size, cfg["vocab"], H))
        w["head_w"] = np.ascontiguousarray(np.fromfile(path, dtype=np.int8, count=cfg["vocab"] * H).reshape(cfg["vocab"], H))
        if w["head_w"].min() < -8 or w["head_w"].max() > 7:
            raise ParameterError("lm_head.bin holds values outside -8..7: not an int4 export")
        w["head_s"] = _read_header_array(param_dir, "w_lm_head_lm_head.h", "w_lm_head_lm_head_s", (cfg["vocab"],), padded=True)
        w["head_sum"] = _read_header_array(param_dir, "w_lm_head_lm_head.h", "w_lm_head_lm_head_sum", (cfg["vocab"],), padded=True)
    if not device:
        return w
    dev = {}
    for key, val in w.items():
        if isinstance(val, list):
            dev[key] = [to_device(a) for a in val]
        elif key == "embed":
            dev[key] = to_device(val.view(np.float16))
        else:
            dev[key] = to_device(val)
    return dev


def _fmt(v):
    t = "%.9g" % v                                 # nine significant digits reproduce a float32 exactly
    return t + "f" if ("." in t or "e" in t or "n" in t) else t + ".0f"


def _write_header(path, arrays):
    with open(path, "w") as f:
        for name, arr in arrays:
            arr = np.asarray(arr, dtype=np.float32)
            f.write("static const float %s%s = {\n" % (name, "".join("[%d]" % d for d in arr.shape)))
            for r in arr.reshape(-1, arr.shape[-1]):
                row = ", ".join(_fmt(v) for v in r)
                f.write("  {%s},\n" % row if arr.ndim > 1 else "  %s,\n" % row)
            f.write("};\n\n")


def save_reference_parameters(param_dir, cfg, w):
    """Writes host weights `w` (layout of `llama.synth_weights(device=False)`, or of `llama.synth_weights_w4a4` with its
    row sums and int4 head) as a reference `parameters/` directory."""
    os.makedirs(param_dir, exist_ok=True)
    L = cfg["layers"]
    for key, stem in _PROJ_FILES.items():
        for l in range(L):
            np.ascontiguousarray(w["w" + key][l], dtype=np.int8).tofile(os.path.join(param_dir, "%s_L%02d.bin" % (stem, l)))
        s = np.stack([np.asarray(w["s" + key][l], dtype=np.float32) for l in range(L)])
        if "sum" + key in w:
            sums = np.stack([np.asarray(w["sum" + key][l], dtype=np.float32) for l in range(L)])
        else:                                      # sum of the dequantised row: integer row sum times the row's scale
            sums = np.stack([np.asarray(w["w" + key][l], dtype=np.int64).sum(1).astype(np.float32) for l in range(L)]) * s
        _write_header(os.path.join(param_dir, "w_%s_s_sum.h" % stem), [("w_%s_s" % stem, s), ("w_%s_sum" % stem, sums)])
    _write_header(os.path.join(param_dir, "w_rmsnorm.h"), [("RMSNorm_weight", w["gamma"])])
    for key, (name, _) in _STATIC.items():
        _write_header(os.path.join(param_dir, name + ".h"), [(name, w[key])])
    embed = np.asarray(w["embed"])
    embed = embed.view(np.float16) if embed.dtype == np.uint16 else embed
    embed.astype(np.float32).tofile(os.path.join(param_dir, "model_embed_tokens_fp32.bin"))
    if "head_w" in w:
        np.ascontiguousarray(w["head_w"], dtype=np.int8).tofile(os.path.join(param_dir, "lm_head.bin"))
        _write_header(os.path.join(param_dir, "w_lm_head_lm_head.h"),
                      [("w_lm_head_lm_head_s", np.asarray(w["head_s"], np.float32)), ("w_lm_head_lm_head_sum", np.asarray(w["head_sum"], np.float32))])
