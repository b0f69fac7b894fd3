"""The parameter-directory format against the reference's own READING code instead of against the loader itself.

(1) `loader.save_reference_parameters` writes a small model; `tests/loader_reader.cpp` - a reader that #includes the
generated headers where the testbench does (inside a function body, the static attention scales at file scope),
indexes the arrays the way it does and fetches weight and embedding rows with its seekg/read loop
(SpinQuant_Prefilling_Decoding_mem_opt_tb.cpp:30-47, 150-172, 187-217, 435-486, 716-736; MHA_i8xi8.h:11-14) - is
compiled with g++ against those files and must see exactly the source arrays.
(2) A writer in this file that shares no code with loader.py (other number formats, line breaks inside rows,
comments, macro-sized dimensions, a padded output head) produces a directory; `loader.load_reference_parameters`
must return exactly what was written."""
import os
import shutil
import struct
import subprocess

import numpy as np
import pytest

from flexllm_amd import llama, loader

HERE = os.path.dirname(os.path.abspath(__file__))
SMALL = dict(layers=2, hidden=128, kv_hidden=64, inter=256, q_heads=2, kv_heads=1, head_dim=64, vocab=96, max_pos=128)
ORDER = (("q", "hidden"), ("k", "kv_hidden"), ("v", "kv_hidden"), ("o", "hidden"), ("g", "inter"), ("u", "inter"), ("d", "hidden"))


def run_reader(tmp_path, cfg, with_head):
    exe = str(tmp_path / "loader_reader")
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-I", str(tmp_path), os.path.join(HERE, "loader_reader.cpp"), "-o", exe,
           "-DFX_LAYERS=%d" % cfg["layers"], "-DFX_HIDDEN=%d" % cfg["hidden"], "-DFX_KV_HIDDEN=%d" % cfg["kv_hidden"],
           "-DFX_INTER=%d" % cfg["inter"], "-DFX_Q_HEADS=%d" % cfg["q_heads"], "-DFX_KV_HEADS=%d" % cfg["kv_heads"],
           "-DFX_VOCAB=%d" % cfg["vocab"]] + (["-DFX_WITH_HEAD"] if with_head else [])
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, "the generated headers do not compile as the testbench includes them:\n" + r.stdout[-3000:]
    dump = str(tmp_path / "dump.bin")
    r = subprocess.run([exe, dump] + (["head"] if with_head else []), cwd=str(tmp_path), stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout
    return open(dump, "rb").read()


def expected_dump(cfg, w, with_head):
    L, H, V = cfg["layers"], cfg["hidden"], cfg["vocab"]
    out = []
    for key, _ in ORDER:
        s = np.stack([np.asarray(w["s" + key][l], np.float32) for l in range(L)])
        if "sum" + key in w:
            sm = np.stack([np.asarray(w["sum" + key][l], np.float32) for l in range(L)])
        else:
            sm = np.stack([np.asarray(w["w" + key][l], np.int64).sum(1).astype(np.float32) for l in range(L)]) * s
        out.append(np.stack([s, sm], axis=-1).astype(np.float32).tobytes())
    g = np.asarray(w["gamma"], np.float32)
    out.append(np.stack([g[0:2 * L:2], g[1:2 * L:2]], axis=-1).tobytes())
    out.append(g[2 * L].tobytes())
    for key in ("q_s", "k_s", "v_s", "a_s"):
        out.append(np.asarray(w[key], np.float32).tobytes())
    for key, _ in ORDER:
        for l in range(L):
            out.append(np.ascontiguousarray(w["w" + key][l], np.int8).tobytes())
    emb = np.asarray(w["embed"]).view(np.float16).astype(np.float32)
    out.append(emb[[V - 1, 0, 5, V // 2]].tobytes())
    if with_head:
        out.append(np.ascontiguousarray(w["head_w"], np.int8).tobytes())
        out.append(np.stack([np.asarray(w["head_s"], np.float32), np.asarray(w["head_sum"], np.float32)], axis=-1).tobytes())
    return b"".join(out)


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
@pytest.mark.parametrize("w4a4", [False, True], ids=["w8a8", "w4a4"])
def test_written_directory_is_read_by_testbench_shaped_code(tmp_path, w4a4):
    cfg = llama.make_config(**SMALL)
    w = (llama.synth_weights_w4a4 if w4a4 else llama.synth_weights)(cfg, seed=17, device=False)
    w["sq"][1][5] = np.float32(1.17549435e-38)            # float32 extremes must survive the C compiler's reading too
    w["gamma"][0, 0] = np.float32(3.4028235e38)
    w["gamma"][1, 3] = np.float32(-1.4e-45)               # a denormal
    loader.save_reference_parameters(str(tmp_path / "parameters"), cfg, w)
    got = run_reader(tmp_path, cfg, with_head=w4a4)
    want = expected_dump(cfg, w, with_head=w4a4)
    assert len(got) == len(want)
    if got != want:
        i = next(k for k in range(len(got)) if got[k] != want[k])
        raise AssertionError("the testbench-shaped reader sees other values from byte %d of %d" % (i, len(got)))


def independent_write(d, cfg, w, vocab_pad=0):
    """A `parameters/` directory in a deliberately different hand than loader.save_reference_parameters: %.8e numbers
    without the f suffix in one header and hex floats in another, rows broken over several lines, comments, macro-sized
    dimensions, `const float` without `static`, byte files written value by value."""
    os.makedirs(d, exist_ok=True)
    L = cfg["layers"]
    names = dict(q="q_proj", k="k_proj", v="v_proj", o="o_proj", g="gate_proj", u="up_proj", d="down_proj")

    def c_rows(arr, fmt, per_line):
        rows = []
        for r in np.asarray(arr, np.float32).reshape(-1, np.asarray(arr).shape[-1]):
            vals = [fmt(float(v)) for v in r]
            lines = [", ".join(vals[i:i + per_line]) for i in range(0, len(vals), per_line)]
            rows.append("{ " + ",\n    ".join(lines) + " }")
        return ",\n  ".join(rows)

    e8 = lambda v: "%.8e" % v                                    # nine significant digits, exponent form, no suffix
    hexf = lambda v: float(v).hex() + "f"                        # C99/C++17 hexadecimal float with the f suffix
    for key, stem in names.items():
        for l in range(L):
            with open(os.path.join(d, "%s_L%02d.bin" % (stem, l)), "wb") as f:
                for row in np.asarray(w["w" + key][l]):
                    f.write(struct.pack("%db" % len(row), *[int(v) for v in row]))
        s = np.stack([w["s" + key][l] for l in range(L)]); sm = np.stack([w["sum" + key][l] for l in range(L)])
        with open(os.path.join(d, "w_%s_s_sum.h" % stem), "w") as f:
            f.write("/* exported: %s */\n#define N_L %d\n" % (stem, L))
            f.write("const float w_%s_s[N_L][%d] = {\n  %s\n};\n" % (stem, s.shape[1], c_rows(s, e8, 5)))
            f.write("// row sums of the dequantised weights\n")
            f.write("const float w_%s_sum [ %d ][ %d ] = {\n  %s };\n#undef N_L\n" % (stem, L, sm.shape[1], c_rows(sm, hexf, 7)))
    with open(os.path.join(d, "w_rmsnorm.h"), "w") as f:
        f.write("static const float RMSNorm_weight[%d][%d] = {\n  %s\n};\n" % (2 * L + 1, cfg["hidden"], c_rows(w["gamma"], hexf, 3)))
    for key, name in (("q_s", "Q_s"), ("k_s", "K_s"), ("v_s", "V_s"), ("a_s", "A_s")):
        with open(os.path.join(d, name + ".h"), "w") as f:
            f.write("const float %s[%d][%d] = {%s};\n" % (name, L, w[key].shape[1], c_rows(w[key], e8, 100)))
    emb = np.asarray(w["embed"]).view(np.float16)
    with open(os.path.join(d, "model_embed_tokens_fp32.bin"), "wb") as f:
        for row in emb:
            f.write(struct.pack("<%df" % len(row), *[float(v) for v in row]))
    if "head_w" in w:
        V = cfg["vocab"]
        pad_rows = vocab_pad - V if vocab_pad else 0
        with open(os.path.join(d, "lm_head.bin"), "wb") as f:
            f.write(np.asarray(w["head_w"], np.int8).tobytes())
            f.write(bytes(pad_rows * cfg["hidden"]))
        hs = np.concatenate([w["head_s"], np.ones(pad_rows, np.float32)]); hm = np.concatenate([w["head_sum"], np.zeros(pad_rows, np.float32)])
        with open(os.path.join(d, "w_lm_head_lm_head.h"), "w") as f:
            f.write("const float w_lm_head_lm_head_s[%d] = {\n %s\n};\n" % (len(hs), ",\n ".join(e8(float(v)) for v in hs)))
            f.write("const float w_lm_head_lm_head_sum[%d] = { %s };\n" % (len(hm), ", ".join(hexf(float(v)) for v in hm)))


@pytest.mark.parametrize("vocab_pad", [0, 128], ids=["exact_head", "padded_head"])
def test_loader_reads_an_independently_written_directory(tmp_path, vocab_pad):
    cfg = llama.make_config(**SMALL)
    w = llama.synth_weights_w4a4(cfg, seed=23, device=False)
    w["so"][0][7] = np.float32(1.17549435e-38)
    w["gamma"][2, 1] = np.float32(3.4028235e38)
    d = str(tmp_path / "parameters")
    independent_write(d, cfg, w, vocab_pad)
    for w4a4 in (True, False):
        r = loader.load_reference_parameters(d, cfg, device=False, w4a4=w4a4)
        keys = [p + q for p in (("w", "s", "sum") if w4a4 else ("w", "s")) for q in "qkvogud"]
        for key in keys:
            for l in range(cfg["layers"]):
                assert r[key][l].dtype == w[key][l].dtype and np.array_equal(r[key][l], w[key][l]), (key, l)
        for key in ("gamma", "q_s", "k_s", "v_s", "a_s") + (("head_w", "head_s", "head_sum") if w4a4 else ()):
            assert r[key].dtype == w[key].dtype and np.array_equal(r[key], w[key]), key
        assert np.array_equal(r["embed"], np.asarray(w["embed"]).view(np.uint16))
    # the same directory also passes the testbench-shaped reader (exact head only: it reads FX_VOCAB rows)
    if not vocab_pad and shutil.which("g++"):
        assert run_reader(tmp_path, cfg, with_head=True) == expected_dump(cfg, w, with_head=True)
    # a head file that is not a whole number of rows, or too short, is refused by name
    with open(os.path.join(d, "lm_head.bin"), "ab") as f:
        f.write(b"\0")
    with pytest.raises(loader.ParameterError, match="lm_head.bin"):
        loader.load_reference_parameters(d, cfg, device=False, w4a4=True)
