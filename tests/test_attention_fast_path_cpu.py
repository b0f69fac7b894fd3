"""Float32 model (numpy) of the two ways `pf_attention_kernel` forms a probability byte, csrc/attn_prefill.h:

* exact: the reference's expression, exp(fl(fl(tv*Q_s)*K_s) - max) with the kernels' two-part exponential, times
  1/sum, divided by A_s, rounded half away (Modules/Softmax.h:456-635 as the oracle restates it);
* fast: e~ = 2^(tv*c2 - m2), q~ = e~ * kq, rounded by the conversion instruction, taken unless a q~ of its group of
  four lies within its own window (proportional to q~) of a tie.

The kernel's claim is that outside the window both give the same byte.  The model draws rows over a range of scales
and score spreads, perturbs every hardware 2^x by up to one ulp either way, and checks exactly that, plus the size
of the deviation against the bound the window is built from."""
import numpy as np

f32 = np.float32
LOG2E = f32(1.44269502162933349609375)
C_LO = f32(1.92596299e-8)
LN2 = f32(0.693147182464599609375)


def fma(a, b, c):
    # one rounding: the double product of two floats is exact
    return (np.float64(a) * np.float64(b) + np.float64(c)).astype(f32)


def exp2_hw(t, rng):
    e = np.exp2(np.float64(t)).astype(f32)
    n = rng.integers(-1, 2, size=np.shape(t))
    return np.where(n == 0, e, np.nextafter(e, np.where(n > 0, f32(np.inf), f32(0)), dtype=f32)).astype(f32)


def exp_f(x, rng):
    t = (x * LOG2E).astype(f32)
    lo = fma(x, C_LO, fma(x, LOG2E, -t))
    e = exp2_hw(t, rng)
    return fma(e, (lo * LN2).astype(f32), e)


def rows(seed, n_rows, n_keys, sq, sk, spread, a_s=f32(1.0 / 255)):
    rng = np.random.default_rng(seed)
    sq, sk = f32(sq), f32(sk)
    outside, redone, total_n, worst = 0, 0, 0, 0.0
    for _ in range(n_rows):
        tv = np.clip(np.rint(rng.standard_normal(n_keys) * spread / (float(sq) * float(sk))), -1000000, 1000000).astype(np.int64)
        im = tv.max()
        imf, tvf = f32(im), tv.astype(f32)
        # exact path
        t1 = (imf * sq).astype(f32)
        mx = (t1 * sk).astype(f32)
        x = (((tvf * sq).astype(f32) * sk).astype(f32) - mx).astype(f32)
        e = exp_f(x, rng)
        # fast path (pf_fast_row_begin / pf_fast_exp / pf_fast_row_finish)
        c2 = ((sq * sk).astype(f32) * LOG2E).astype(f32)
        m2 = (imf * c2).astype(f32)
        ef = exp2_hw(fma(tvf, c2, -m2), rng)
        total = ef.sum(dtype=f32)
        r1, r2, rr = fma(imf, sq, -t1), fma(t1, sk, -mx), fma(imf, c2, -m2)
        offset = (r2 + (r1 * sk).astype(f32) - (rr * LN2).astype(f32)).astype(f32)
        cd = (f32(1) / (total * (f32(1) + offset)).astype(f32)).astype(f32)
        kq = ((f32(1) / total).astype(f32) * (f32(1) / a_s).astype(f32)).astype(f32)
        x_max = max(0.0, float(np.log(kq)) + 0.92)
        rel = 5.9604645e-8 * (3.0 * abs(float(mx)) + 9.0 * x_max + 12.0) + 1.4e-6
        win = 1e-6 + 1.01 * float(kq) * rel
        qf = (ef * kq).astype(f32)
        qe = ((e * cd).astype(f32) / a_s).astype(f32)
        d = np.abs((qf - np.floor(qf)) - f32(0.5))
        assert float(qf.max()) <= 1.01 * float(kq)                  # the group check's window covers every element's own
        near_el = d < fma(qf, f32(rel), f32(1e-6))                  # the element's own window
        grp = (d.reshape(-1, 4).min(axis=1) < win) & near_el.reshape(-1, 4).any(axis=1)   # groups of four redone exactly
        near = np.repeat(grp, 4)
        p_exact = np.minimum(255, np.floor(qe.astype(np.float64) + 0.5)).astype(np.int64)      # half away from zero
        p_fast = np.minimum(255, np.rint(qf.astype(np.float64))).astype(np.int64)              # nearest, ties to even
        outside += int(((p_exact != p_fast) & ~near).sum())
        redone += int(near.sum())
        total_n += n_keys
        m = qe > 0.3
        if m.any():
            worst = max(worst, float((np.abs(qf.astype(np.float64) - qe.astype(np.float64))[m] / (qe.astype(np.float64)[m] * rel)).max()))
    return outside, redone / total_n, worst


def test_fast_probabilities_equal_the_exact_ones_outside_the_window():
    cases = [(0.004, 0.03, 1.0), (0.004, 0.03, 3.0), (0.004, 0.03, 8.0), (0.0005, 0.01, 2.0), (0.02, 0.1, 4.0), (0.004, 0.03, 0.2)]
    for i, (sq, sk, spread) in enumerate(cases):
        for n_keys, n_rows in ((48, 1500), (1500, 500), (4096, 200)):
            outside, share, worst = rows(100 + i, n_rows, n_keys, sq, sk, spread)
            assert outside == 0, (sq, sk, spread, n_keys)
            assert worst < 0.5, "deviation %.2f of the bound the window is built from" % worst
            assert share < (1e-3 if n_keys < 1024 else 5e-5), "share of elements redone exactly: %.1e" % share
