"""The reference's on-disk parameter format: C-array header parsing and a write -> read round trip on the host."""
import numpy as np
import pytest

from flexllm_amd import llama, loader

SMALL = dict(layers=2, hidden=128, kv_hidden=64, inter=256, q_heads=2, kv_heads=1, head_dim=64, vocab=96, max_pos=128)


def test_parse_c_array_forms():
    src = """
    // generated
    static const float w_k_proj_s[2][3] = { {1.5f, -2e-3f, 3}, /* row 1 */ {4.0, .5f, -6.25e+1F} };
    const float RMSNorm_weight[LAYERS][HIDDEN] = {{1,2},{3,4}};
    float one_d[] = {0.25f, 1e-3f};
    """
    a = loader.parse_c_array(src, "w_k_proj_s")
    assert a.shape == (2, 3) and a.dtype == np.float32
    assert np.array_equal(a, np.array([[1.5, -2e-3, 3], [4.0, 0.5, -62.5]], np.float32))
    assert np.array_equal(loader.parse_c_array(src, "RMSNorm_weight"), np.array([1, 2, 3, 4], np.float32))   # macro sizes: flat
    assert np.array_equal(loader.parse_c_array(src, "one_d"), np.array([0.25, 1e-3], np.float32))
    with pytest.raises(loader.ParameterError):
        loader.parse_c_array(src, "w_q_proj_s")
    with pytest.raises(loader.ParameterError):
        loader.parse_c_array("float bad[2][2] = {1,2,3};", "bad")


def test_round_trip_small_model(tmp_path):
    cfg = llama.make_config(**SMALL)
    w = llama.synth_weights(cfg, seed=7, device=False)
    w["sq"][1][5] = np.float32(1.17549435e-38)            # extremes of float32 survive the text form
    w["gamma"][0, 0] = np.float32(3.4028235e38)
    d = str(tmp_path / "parameters")
    loader.save_reference_parameters(d, cfg, w)
    r = loader.load_reference_parameters(d, cfg, device=False)
    for key in ("wq", "wk", "wv", "wo", "wg", "wu", "wd", "sq", "sk", "sv", "so", "sg", "su", "sd"):
        for l in range(cfg["layers"]):
            assert r[key][l].dtype == w[key][l].dtype and np.array_equal(r[key][l], w[key][l]), (key, l)
    for key in ("gamma", "q_s", "k_s", "v_s", "a_s", "rope_sin", "rope_cos"):
        assert np.array_equal(r[key], w[key]), key
    assert np.array_equal(r["embed"], w["embed"])          # fp16 -> fp32 file -> fp16 is the identity
    # the row sums the asymmetric 4-bit path reads are written as well
    sums = loader.parse_c_array(open(d + "/w_down_proj_s_sum.h").read(), "w_down_proj_sum")
    # (the sum of the DEQUANTISED row: integer row sum times the row's scale)
    assert np.array_equal(sums[1], w["wd"][1].astype(np.int64).sum(1).astype(np.float32) * w["sd"][1])


def test_round_trip_w4a4_model(tmp_path):
    """The W4A4 dictionary (int4 values one per byte, row sums, int4 output head) through the reference's files."""
    cfg = llama.make_config(**SMALL)
    w = llama.synth_weights_w4a4(cfg, seed=8, device=False)
    d = str(tmp_path / "parameters")
    loader.save_reference_parameters(d, cfg, w)
    r = loader.load_reference_parameters(d, cfg, device=False, w4a4=True)
    for key in [p + q for p in ("w", "s", "sum") for q in "qkvogud"]:
        for l in range(cfg["layers"]):
            assert r[key][l].dtype == w[key][l].dtype and np.array_equal(r[key][l], w[key][l]), (key, l)
    for key in ("head_w", "head_s", "head_sum", "gamma", "q_s", "a_s"):
        assert r[key].dtype == w[key].dtype and np.array_equal(r[key], w[key]), key
    assert w["wq"][0].min() >= -8 and w["wq"][0].max() <= 7
    # an int8 export is refused where int4 values are expected
    w8 = llama.synth_weights(cfg, seed=7, device=False)
    d8 = str(tmp_path / "parameters8")
    loader.save_reference_parameters(d8, cfg, w8)
    with pytest.raises(loader.ParameterError, match="-8..7"):
        loader.load_reference_parameters(d8, cfg, device=False, w4a4=True)


def test_missing_and_misshapen_files(tmp_path):
    cfg = llama.make_config(**SMALL)
    w = llama.synth_weights(cfg, seed=3, device=False)
    d = str(tmp_path / "parameters")
    loader.save_reference_parameters(d, cfg, w)
    import os
    os.remove(d + "/K_s.h")
    with pytest.raises(loader.ParameterError, match="K_s.h"):
        loader.load_reference_parameters(d, cfg, device=False)
    loader.save_reference_parameters(d, cfg, w)
    with open(d + "/up_proj_L01.bin", "ab") as f:
        f.write(b"\0")
    with pytest.raises(loader.ParameterError, match="up_proj_L01"):
        loader.load_reference_parameters(d, cfg, device=False)
