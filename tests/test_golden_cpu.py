"""The committed regression vectors (tests/golden/modules_small.npz) against the oracle as it is now: every stored
array must come out bit for bit.  The vectors were written by tests/golden/make_golden.py."""
import importlib.util
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden", "modules_small.npz")


def _generator():
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(HERE, "golden", "make_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_oracle_reproduces_the_committed_vectors(oracle):
    stored = np.load(GOLDEN)                       # allow_pickle stays False
    fresh = _generator().cases(oracle)
    assert sorted(stored.files) == sorted(fresh.keys())
    for name in stored.files:
        a, b = stored[name], np.asarray(fresh[name])
        assert a.dtype == b.dtype and a.shape == b.shape, name
        assert np.array_equal(a.view(np.uint8), np.ascontiguousarray(b).view(np.uint8)), "%s changed" % name


def test_vectors_hold_the_edge_cases_they_claim():
    g = np.load(GOLDEN)
    assert not g["quant_in_x"][1].any() and g["quant_out_s8"][1] == 1.0 and not g["quant_out_q8"][1].any()
    assert g["mha_out_p8"].dtype == np.uint8 and g["mha_out_p8"][:, 0, 1:].max() == 0      # causal: row 0 sees key 0 only
    assert g["mha_out_p8"][:, 0, 0].min() == 255                                             # ... with probability 1 = 255 * A_s
    assert not g["hmt_in_kmem"][5:].any() and (g["hmt_out_a"][5:] > 0).all()                # empty slots keep their share
    assert abs(float(g["hmt_out_a"].sum()) - 1.0) < 1e-5
