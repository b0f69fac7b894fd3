#!/usr/bin/env python3
"""Headline benchmark: full 16-layer Llama-3.2-1B W8A8 SpinQuant greedy decode, batch 1, int8 KV cache
pre-filled so that the context grows to 4096 positions; plus the 1024-token prefill time.

A "step" is one generated token (embedding -> 16 layers -> final norm -> fp16 lm_head -> argmax).  The
persistent decode kernel generates up to 64 consecutive tokens per launch (the arg-max and the hand-over of
the token to the next step happen inside the kernel).  Inputs (weights, caches) are resident in HBM before the timed region.  Prints ONE JSON
line.  One GPU only.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
INT8_PEAK_TOPS = 5000.0        # MI355X published dense int8 MFMA rate
TOKENS_PER_LAUNCH = 64         # the library's cap on tokens per persistent-kernel launch (kMegaMaxSteps)
PMC_SUMMARY = os.path.join(ROOT, "profiles", "decode_mega_kernel_llama32_1b_ctx4096_pmc.txt")
MEGA_SOURCE = os.path.join(ROOT, "flexllm_amd", "csrc", "decode_mega.h")


def kernel_source_hash():
    """SHA-256 (first 16 hex digits) of the persistent kernel's source with // comments and white space removed: the
    identity of the code that a counter summary was measured on."""
    import hashlib
    import re
    src = open(MEGA_SOURCE, encoding="utf-8").read()
    src = re.sub(r"//[^\n]*", "", src)
    src = re.sub(r"\s+", "", src)
    return hashlib.sha256(src.encode("utf-8")).hexdigest()[:16]


def measured_traffic_per_token():
    """HBM bytes per generated token of the persistent decode kernel as the committed counter summary gives them
    (FETCH_SIZE / WRITE_SIZE per dispatch of an 8-token launch, each scaled by the same counter's reading for a 1 GiB
    device copy), or None when that summary was taken on another revision of the kernel: the summary records the
    hash of the kernel's source (kernel_source_hash), and a figure measured on other code is not reported."""
    import re
    try:
        txt = open(PMC_SUMMARY).read()
        sha = kernel_source_hash()
        m = re.search(r"kernel source sha256\[:16\]: ([0-9a-f]{16})", txt)
        if not m or m.group(1) != sha:
            return None
        num = lambda pat: float(re.search(pat, txt).group(1).replace(",", ""))
        fetch = num(r"FETCH_SIZE\s+decode_mega_kernel \(8 tokens\)\s+\d+\s+([\d,\.]+)")
        write = num(r"WRITE_SIZE\s+decode_mega_kernel \(8 tokens\)\s+\d+\s+([\d,\.]+)")
        f_fac = num(r"true fetch 1,048,576 KiB -> factor ([\d\.]+)")
        w_fac = num(r"true write 1,048,576 KiB -> factor ([\d\.]+)")
        return int((fetch * f_fac + write * w_fac) * 1024 / 8)
    except (OSError, AttributeError, ValueError):
        return None


def bytes_per_token(cfg, mean_len):
    """Algorithmic HBM bytes of one decode step at context length mean_len."""
    H, KV, I, L, V = cfg["hidden"], cfg["kv_hidden"], cfg["inter"], cfg["layers"], cfg["vocab"]
    w = L * (H * H + 2 * KV * H + H * H + 2 * I * H + H * I)            # int8 weights
    scales = 4 * L * (H + 2 * KV + H + 2 * I + H)
    gamma = 4 * (2 * L + 1) * H
    lm_head = 2 * V * H
    kv_read = L * 2 * KV * mean_len
    kv_write = L * 2 * KV
    return w + scales + gamma + lm_head + kv_read + kv_write


def _time(stream, Event, fn, reps):
    fn(0)
    stream.sync()
    e0, e1 = Event(), Event()
    e0.record(stream)
    for i in range(reps):
        fn(i)
    e1.record(stream)
    e1.sync()
    return e0.elapsed_ms(e1) * 1e3 / reps          # microseconds per call


def measured_peaks(fx, lib, synth, stream, Event):
    """What this GPU sustains on the two resources the rooflines are priced against, beside the published peaks:
    HBM as a read-only stream over 4 GiB (16 times the memory-side cache) and as a 1 GiB device copy (read + write),
    and the int8 matrix cores alone (no global memory) with zero and with pseudo-random operands, from registers and
    re-read from LDS at every step, with the shader clock read inside the kernel under that load."""
    P = lambda a: C.c_void_p(a.ptr)
    out = {}
    n = 1 << 32
    buf = fx.empty((n,), np.int8)
    fx.check(lib.flexllm_rt_fill_i8(P(buf), C.c_size_t(n), C.c_uint64(77), -100, 100, stream.handle))
    sink = fx.empty((16384 * 4,), np.uint32)
    us, wgs, nt = min((_time(stream, Event, lambda i: lib.flexllm_probe_hbm_read(P(buf), C.c_size_t(n), g, t, P(sink), stream.handle), 4), g, t)
                      for g in (256, 512, 1024, 2048, 4096) for t in (0, 1))       # the best grid size and load kind are reported
    one = 1 << 30
    us_c = _time(stream, Event, lambda i: lib.flexllm_rt_memcpy_d2d(C.c_void_p(buf.ptr + 2 * one), P(buf), C.c_size_t(one), stream.handle), 5)
    out["hbm"] = {"published_GBs": HBM_PEAK_GBS, "read_stream_GBs": round(n / us / 1e3, 1), "read_stream_bytes": n, "read_stream_workgroups": wgs, "read_stream_non_temporal": bool(nt),
                  "copy_GBs_read_plus_write": round(2 * one / us_c / 1e3, 1), "copy_bytes": one,
                  "note": "read_stream: 16-byte loads over 4 GiB in contiguous 32 KiB blocks per workgroup, read-only (the decode path's traffic is 99 % reads); "
                          "copy: hipMemcpyAsync device to device of 1 GiB, bytes read + bytes written"}
    del buf
    iters, cus = 4000, 256
    sink_i = fx.empty((cus * 256,), np.int32)
    clocks = fx.zeros((2,), np.uint64)
    mf = {"published_TOPs": INT8_PEAK_TOPS}
    ops_launch = cus * 4 * iters * 16 * 65536.0
    for name, rnd, lds in (("zeros_regs", 0, 0), ("random_regs", 1, 0), ("zeros_lds", 0, 1), ("random_lds", 1, 1)):
        us = _time(stream, Event, lambda i: lib.flexllm_probe_mfma_i8(iters, rnd, lds, cus, P(sink_i), P(clocks), stream.handle), 3)
        cyc, ticks = [int(v) for v in clocks.numpy()]
        mf[name + "_TOPs"] = round(ops_launch / us / 1e6, 1)
        mf[name + "_shader_clock_GHz"] = round(cyc / max(ticks, 1) * 0.1, 3)
    mf["note"] = ("256 workgroups x 4 waves issuing v_mfma_i32_32x32x32_i8 back to back on 16 accumulator tiles per wave, no global "
                  "memory; lds = the 8 operand fragments re-read from LDS for every 16 instructions; random operands draw more power "
                  "than zeros and the clock drops accordingly; random_lds is what a GEMM's inner loop can reach at best")
    out["mfma_i8"] = mf
    return out


def cpu_module_legs(oracle, cfg, n_threads):
    """The CPU oracle (all OpenMP threads of the host) on the same module-level workloads as module_legs, so that each
    GPU figure has the reference-semantics CPU figure beside it.  Bounded: the S = 4096 attention is timed on 4 of its
    32 query heads."""
    r = np.random.default_rng(5)
    out = {}

    def timed(fn, reps=1):
        fn()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        return (time.perf_counter() - t0) / reps * 1e3

    i8 = lambda *sh: r.integers(-127, 128, sh, dtype=np.int8)
    K = N = 2048
    x = r.standard_normal((1, K)).astype(np.float32); w = i8(N, K); ws = r.uniform(1e-3, 1e-2, N).astype(np.float32)
    def lin1():
        q, s = oracle.quant_sym(x)
        oracle.dequant(oracle.linear_i8(q, w), s, ws)
    out["linear_decode_2048x2048"] = {"ms_quant_gemv_dequant": round(timed(lin1, 20), 4)}
    for n in (2048, 8192):
        xf = r.standard_normal((1024, n)).astype(np.float32)
        out["fht_quant_1024x%d" % n] = {"ms": round(timed(lambda: oracle.quant_sym(oracle.fht(xf, float(np.sqrt(n))))), 3)}
    M, H, KV, I = 1024, 2048, 512, 8192
    a = i8(M, H); a8 = i8(M, I); sx = r.uniform(0.01, 0.02, M).astype(np.float32)
    res = r.standard_normal((M, H)).astype(np.float32)
    scn = r.uniform(1e-4, 2e-4, 2 * I).astype(np.float32)
    stack = {}
    wq = i8(H + 2 * KV, H); stack["qkv"] = timed(lambda: oracle.dequant(oracle.linear_i8(a, wq), sx, scn[:H + 2 * KV]))
    wo = i8(H, H); stack["o+res"] = timed(lambda: oracle.residual(oracle.dequant(oracle.linear_i8(a, wo), sx, scn[:H]), res))
    wg = i8(2 * I, H)
    def gu():
        y = oracle.dequant(oracle.linear_i8(a, wg), sx, scn)
        oracle.gate(y[:, 1::2], oracle.swish(y[:, 0::2]))
    stack["gate_up+swiglu"] = timed(gu)
    wd = i8(H, I); stack["down+res"] = timed(lambda: oracle.residual(oracle.dequant(oracle.linear_i8(a8, wd), sx, scn[:H]), res))
    del wq, wo, wg, wd
    stack = {k: round(v, 2) for k, v in stack.items()}
    stack["total"] = round(sum(stack.values()), 2)
    out["prefill_linear_stack_M1024"] = {"ms": stack}
    sc = (np.full(32, 4e-3, np.float32), np.full(8, 0.03, np.float32), np.full(8, 0.03, np.float32), np.full(32, 1.0 / 255, np.float32))
    S = 1024
    q8 = i8(S, 32, 64); k8 = r.integers(-100, 101, (S, 8, 64), dtype=np.int8); v8 = r.integers(-100, 101, (S, 8, 64), dtype=np.int8)
    out["attention_prefill_S1024"] = {"ms": round(timed(lambda: oracle.mha_prefill_i8(q8, k8, v8, *sc)), 2)}
    S = 4096
    q8 = i8(S, 4, 64); k8 = r.integers(-100, 101, (S, 1, 64), dtype=np.int8); v8 = r.integers(-100, 101, (S, 1, 64), dtype=np.int8)
    sc4 = (sc[0][:4], sc[1][:1], sc[2][:1], sc[3][:4])
    t0 = time.perf_counter(); oracle.mha_prefill_i8(q8, k8, v8, *sc4); t4 = (time.perf_counter() - t0) * 1e3
    out["attention_prefill_S4096"] = {"ms_4_of_32_heads": round(t4, 1), "note": "one KV head with its 4 query heads: an eighth of the leg's work"}
    K, N = 2048, 8192
    w4 = r.integers(-8, 8, (N, K), dtype=np.int8); w4s = r.uniform(1e-3, 1e-2, N).astype(np.float32); w4m = r.uniform(-1, 1, N).astype(np.float32)
    x1 = r.standard_normal((1, K)).astype(np.float32); xm = r.standard_normal((1024, K)).astype(np.float32)
    out["w4a4_linear_decode_2048x8192"] = {"ms": round(timed(lambda: oracle.w4a4_linear(x1, w4, w4s, w4m), 10), 4)}
    out["w4a4_linear_prefill_M1024_2048x8192"] = {"ms": round(timed(lambda: oracle.w4a4_linear(xm, w4, w4s, w4m)), 2)}
    for v in out.values():
        v["threads"] = n_threads
    return out


def module_legs(fx, lib, synth, ops, stream, Event, peaks=None):
    """Single-module timings on seeded synthetic inputs, weights cycled through rings larger than the 256 MB
    memory-side cache: (1) decode linear 2048x2048, (2) Hadamard + per-token quantisation of 1024 tokens,
    (3) the prefill linear stack of one layer at M=1024, (4) prefill attention at S=1024 and 4096, (5) the W4A4
    linears (decode GEMV and prefill GEMM on nibble-packed operands)."""
    P = lambda a: C.c_void_p(a.ptr) if a is not None else None
    out = {}
    # (1) quantise -> GEMV -> dequant, 1 x 2048 against 2048 x 2048
    K = N = 2048
    ring = [synth.device_i8((N, K), 9000 + i) for i in range(80)]                       # 336 MB
    x = synth.device_uniform_f32((1, K), 9100, -3, 3)
    w_s = synth.device_uniform_f32((N,), 9101, 1e-3, 1e-2)
    xq = fx.empty((1, K), np.int8); xs = fx.empty((1,), np.float32); y = fx.empty((N,), np.float32)
    def leg1(i):
        lib.flexllm_quant_sym_i8(P(x), P(xq), P(xs), 1, K, stream.handle)
        lib.flexllm_linear_i8_gemv_dequant(P(xq), P(xs), P(ring[i % len(ring)]), P(w_s), None, P(y), K, N, stream.handle)
    us = _time(stream, Event, leg1, 160)
    def leg1b(i):
        lib.flexllm_linear_i8_gemv_dequant(P(xq), P(xs), P(ring[i % len(ring)]), P(w_s), None, P(y), K, N, stream.handle)
    us_b = _time(stream, Event, leg1b, 160)
    def leg1c(i):
        lib.flexllm_quant_linear_i8_gemv_dequant(P(x), P(ring[i % len(ring)]), P(w_s), None, P(y), None, None, K, N, stream.handle)
    us_c = _time(stream, Event, leg1c, 160)
    b1 = N * K + 4 * N + 4 * K + 4 * N
    out["linear_decode_2048x2048"] = {"bytes": b1, "us_quant_gemv_dequant": round(us, 2), "us_gemv_dequant": round(us_b, 2),
                                      "us_fused_one_launch": round(us_c, 2), "GBs_fused": round(b1 / us_c / 1e3, 1),
                                      "hbm_frac_fused": round(b1 / us_c / 1e3 / HBM_PEAK_GBS, 4),
                                      "GBs_gemv": round(b1 / us_b / 1e3, 1), "hbm_frac_gemv": round(b1 / us_b / 1e3 / HBM_PEAK_GBS, 4)}
    del ring
    # (2) FHT / sqrt(n) -> per-token int8, 1024 tokens
    for n in (2048, 8192):
        xf = synth.device_normal_f32((1024, n), 9200 + n) if hasattr(synth, "device_normal_f32") else synth.device_uniform_f32((1024, n), 9200 + n, -2, 2)
        q = fx.empty((1024, n), np.int8); sc = fx.empty((1024,), np.float32)
        def leg2(i):
            lib.flexllm_fht_quant_i8(P(xf), P(q), P(sc), 1024, n, C.c_float(float(np.sqrt(n))), stream.handle)
        us = _time(stream, Event, leg2, 20)
        b2 = 1024 * (4 * n + n + 4)
        out["fht_quant_1024x%d" % n] = {"bytes": b2, "us": round(us, 2), "GBs": round(b2 / us / 1e3, 1),
                                        "hbm_frac": round(b2 / us / 1e3 / HBM_PEAK_GBS, 4)}
    # (3) prefill linear stack of one layer, M = 1024
    M, H, KV, I = 1024, 2048, 512, 8192
    a = synth.device_i8((M, H), 9300); a8 = synth.device_i8((M, I), 9301)
    s_x = synth.device_uniform_f32((M,), 9302, 0.01, 0.02)
    res = synth.device_uniform_f32((M, H), 9303, -1, 1)
    nl = 6                                                                               # 6 x 60.8 MB = 365 MB of weights
    wq = [synth.device_i8((H + 2 * KV, H), 9310 + i) for i in range(nl)]
    wo = [synth.device_i8((H, H), 9320 + i) for i in range(nl)]
    wg = [synth.device_i8((2 * I, H), 9330 + i) for i in range(nl)]
    wd = [synth.device_i8((H, I), 9340 + i) for i in range(nl)]
    sc_n = synth.device_uniform_f32((2 * I,), 9350, 1e-4, 2e-4)
    yq = fx.empty((M, H + 2 * KV), np.float32); yo = fx.empty((M, H), np.float32); yh = fx.empty((M, I), np.float32)
    legs = {
        "qkv": (lambda i: lib.flexllm_linear_i8_gemm_dequant(P(a), P(s_x), P(wq[i % nl]), P(sc_n), None, P(yq), M, H, H + 2 * KV, stream.handle), 2 * M * H * (H + 2 * KV)),
        "o+res": (lambda i: lib.flexllm_linear_i8_gemm_dequant(P(a), P(s_x), P(wo[i % nl]), P(sc_n), P(res), P(yo), M, H, H, stream.handle), 2 * M * H * H),
        "gate_up+swiglu": (lambda i: lib.flexllm_linear_i8_gemm_swiglu(P(a), P(s_x), P(wg[i % nl]), P(sc_n), P(yh), M, H, I, stream.handle), 2 * M * H * 2 * I),
        "down+res": (lambda i: lib.flexllm_linear_i8_gemm_dequant(P(a8), P(s_x), P(wd[i % nl]), P(sc_n), P(res), P(yo), M, I, H, stream.handle), 2 * M * I * H),
    }
    stack = {}
    tot_us, tot_ops = 0.0, 0
    for name, (fn, opsn) in legs.items():
        us = _time(stream, Event, fn, 4 * nl)
        stack[name] = {"us": round(us, 2), "TOPs": round(opsn / us / 1e6, 1), "mfma_frac": round(opsn / us / 1e6 / INT8_PEAK_TOPS, 4)}
        tot_us += us; tot_ops += opsn
    stack["total"] = {"us": round(tot_us, 2), "GOP": round(tot_ops / 1e9, 2), "TOPs": round(tot_ops / tot_us / 1e6, 1),
                      "mfma_frac": round(tot_ops / tot_us / 1e6 / INT8_PEAK_TOPS, 4)}
    if peaks:
        for leg in stack.values():
            leg["mfma_frac_of_measured_peak"] = round(leg["TOPs"] / peaks["mfma_i8"]["random_lds_TOPs"], 4)
    out["prefill_linear_stack_M1024"] = stack
    del wq, wo, wg, wd
    # (4) prefill attention, S = 1024 and the maximum context 4096, 32/8 heads, reading the int8 cache
    QH, KVH = 32, 8
    scl = ops.Scales(np.full(QH, 4e-3, np.float32), np.full(KVH, 0.03, np.float32), np.full(KVH, 0.03, np.float32), np.full(QH, 1.0 / 255, np.float32))
    for S in (1024, 4096):
        q8 = synth.device_i8((S, QH, 64), 9400)
        kc, vc = ops.kv_cache(KVH, S)
        lib.flexllm_rt_fill_i8(P(kc), C.c_size_t(kc.size), C.c_uint64(9401), -100, 100, stream.handle)
        lib.flexllm_rt_fill_i8(P(vc), C.c_size_t(vc.size), C.c_uint64(9402), -100, 100, stream.handle)
        o = fx.empty((S, QH, 64), np.float32)
        def leg4(i):
            lib.flexllm_mha_i8_prefill(P(q8), P(kc), P(vc), scl.ref(), P(o), None, S, QH, KVH, 64, S, stream.handle)
        us = _time(stream, Event, leg4, 20 if S == 1024 else 5)
        ops4 = 2 * 2 * QH * S * S * 64
        out["attention_prefill_S%d" % S] = {"us": round(us, 2), "GOP_full_S2": round(ops4 / 1e9, 2), "TOPs_full_S2": round(ops4 / us / 1e6, 1),
                                            "mfma_frac_full_S2": round(ops4 / us / 1e6 / INT8_PEAK_TOPS, 4),
                                            "note": ("causal half computed, scores and then their exponentials kept in registers between the softmax passes"
                                                     if S <= 1024 else "causal half computed, scores formed again in each of the three passes (maximum, sum, probabilities)")
                                                    + "; bound by the exponential and rounding per probability"}
        del q8, kc, vc, o
    # (4b) the same attention with dynamic per-(token, head) scales (the variant the metric's source names for the module
    # test): S = 1024, 32/8 heads; rows of up to 1024 keys keep their scores in registers
    S = 1024
    q8 = synth.device_i8((S, QH, 64), 9410)
    kc, vc = ops.kv_cache(KVH, S)
    lib.flexllm_rt_fill_i8(P(kc), C.c_size_t(kc.size), C.c_uint64(9411), -100, 100, stream.handle)
    lib.flexllm_rt_fill_i8(P(vc), C.c_size_t(vc.size), C.c_uint64(9412), -100, 100, stream.handle)
    dq = synth.device_uniform_f32((S, QH), 9413, 0.003, 0.005); dk = synth.device_uniform_f32((S, KVH), 9414, 0.02, 0.04)
    dv = synth.device_uniform_f32((S, KVH), 9415, 0.02, 0.04)
    dsc = ops._dyn_scales(dq, dk, dv, None, 8.0)
    o = fx.empty((S, QH, 64), np.float32); ps = fx.empty((S, QH), np.float32)
    def leg4b(i):
        lib.flexllm_mha_i8_prefill_dyn(P(q8), P(kc), P(vc), C.byref(dsc), P(o), None, P(ps), S, QH, KVH, 64, S, stream.handle)
    us = _time(stream, Event, leg4b, 20)
    ops4 = 2 * 2 * QH * S * S * 64
    out["attention_prefill_dyn_S1024"] = {"us": round(us, 2), "GOP_full_S2": round(ops4 / 1e9, 2), "TOPs_full_S2": round(ops4 / us / 1e6, 1),
                                          "mfma_frac_full_S2": round(ops4 / us / 1e6 / INT8_PEAK_TOPS, 4),
                                          "note": "per-(token, head) Q/K/V scales, V's scale folded into int8 probabilities (own formulation: no reference counterpart for the P.V side)"}
    del q8, kc, vc, o
    # (5) W4A4 linears (the reference's shipped precision): decode GEMV 2048 -> 8192 on nibble-packed weights
    # (half the bytes of the int8 path) and the prefill GEMM at M = 1024
    K, N = 2048, 8192
    ring4 = [synth.device_i8((N, K // 2), 9500 + i) for i in range(48)]                  # 48 x 8.4 MB = 403 MB
    x4 = synth.device_i8((K // 2,), 9550)
    sx = fx.to_device(np.array([0.1], np.float32)); bx = fx.to_device(np.array([-0.7], np.float32))
    w_s = synth.device_uniform_f32((N,), 9551, 1e-3, 1e-2); w_sum = synth.device_uniform_f32((N,), 9552, -1, 1)
    y = fx.empty((N,), np.float32)
    def leg5(i):
        lib.flexllm_linear_u4i4_gemv_dequant(P(x4), P(sx), P(bx), P(ring4[i % len(ring4)]), P(w_s), P(w_sum), None, P(y), K, N, stream.handle)
    us = _time(stream, Event, leg5, 96)
    b5 = N * K // 2 + 8 * N + K // 2 + 4 * N
    out["w4a4_linear_decode_2048x8192"] = {"bytes": b5, "us": round(us, 2), "GBs": round(b5 / us / 1e3, 1),
                                           "hbm_frac": round(b5 / us / 1e3 / HBM_PEAK_GBS, 4)}
    M = 1024
    a4 = synth.device_i8((M, K // 2), 9560)
    sxm = synth.device_uniform_f32((M,), 9561, 0.05, 0.1); bxm = synth.device_uniform_f32((M,), 9562, -1, 0)
    ym = fx.empty((M, N), np.float32)
    def leg5b(i):
        lib.flexllm_linear_u4i4_gemm_dequant(P(a4), P(sxm), P(bxm), P(ring4[i % len(ring4)]), P(w_s), P(w_sum), None, P(ym), M, K, N, stream.handle)
    us = _time(stream, Event, leg5b, 24)
    ops5 = 2 * M * K * N
    out["w4a4_linear_prefill_M1024_2048x8192"] = {"us": round(us, 2), "TOPs": round(ops5 / us / 1e6, 1),
                                                  "mfma_frac": round(ops5 / us / 1e6 / INT8_PEAK_TOPS, 4),
                                                  "note": "nibbles widened to int8 on the way to LDS, int8 MFMA (gfx950 has no int4 MFMA)"}
    # the same product with both operands held one value per byte, on the direct-load kernel of the int8 path
    ring8 = [synth.device_i8((N, K), 9600 + i, -8, 7) for i in range(24)]                # 24 x 16.8 MB = 403 MB
    a8 = synth.device_i8((M, K), 9650, 0, 15)
    def leg5c(i):
        lib.flexllm_linear_i8_gemm_dequant_asym(P(a8), P(sxm), P(bxm), P(ring8[i % len(ring8)]), P(w_s), P(w_sum), None, P(ym), M, K, N, stream.handle)
    us = _time(stream, Event, leg5c, 24)
    out["w4a4_linear_prefill_M1024_2048x8192_byte_held"] = {"us": round(us, 2), "TOPs": round(ops5 / us / 1e6, 1),
                                                            "mfma_frac": round(ops5 / us / 1e6 / INT8_PEAK_TOPS, 4),
                                                            "note": "4-bit values one per byte (weights widened once at load time): direct global-to-LDS loads, int8 MFMA"}
    del ring4, ring8
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-prefill", action="store_true", help="skip the prefill timing")
    ap.add_argument("--no-modules", action="store_true", help="skip the module-level legs")
    ap.add_argument("--decode-mode", type=int, default=0, choices=[0, 1],
                    help="0: persistent decode kernel (default), 1: one kernel per stage replayed as a HIP graph")
    ap.add_argument("--copy-probe", action="store_true",
                    help="only run three 1 GiB device-to-device copies and exit: the transfer of known size that scales "
                         "the FETCH_SIZE / WRITE_SIZE counters")
    ap.add_argument("--peaks-probe", action="store_true",
                    help="only run the measured-peak probes (HBM read stream, device copy, matrix cores alone) and exit: the "
                         "short command the profiler summary of the probes uses")
    ap.add_argument("--module-probe", action="store_true",
                    help="only run the single-module legs (decode linear, Hadamard + quantisation, prefill linear stack, "
                         "prefill attention, W4A4 linears) and exit: the short command the per-kernel counter runs use")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import flexllm_amd as fx
    from flexllm_amd import llama, synth, ops
    from flexllm_amd.device import Event, device_sync

    lib = fx.lib()
    if args.copy_probe:
        n = 1 << 30
        src = synth.device_i8((n,), 1)
        dst = fx.empty((n,), np.int8)
        device_sync()
        for _ in range(3):
            fx.check(lib.flexllm_rt_memcpy_d2d(C.c_void_p(dst.ptr), C.c_void_p(src.ptr), C.c_size_t(n), None))
        device_sync()
        print(json.dumps({"copy_probe_bytes": n, "copies": 3}))
        return
    if args.peaks_probe:
        from flexllm_amd.device import Stream
        print(json.dumps({"peaks": measured_peaks(fx, lib, synth, Stream(), Event)}))
        return
    if args.module_probe:
        from flexllm_amd.device import Stream
        print(json.dumps({"modules": module_legs(fx, lib, synth, ops, Stream(), Event)}))
        return
    cfg = llama.make_config()
    K, W = args.steps, args.warmup
    assert K + W < cfg["max_pos"]
    # fp16 embedding in +-0.03: logits of order one, so that the greedy ids keep changing (with a wide table a token's
    # own row always wins the tied head and the loop would feed the same id back for ever)
    dev_w = llama.synth_weights(cfg, seed=1, device=True, embed_range=0.03)
    model = llama.Llama(cfg, dev_w)
    exchange_info = model.exchange_info()
    exchange_info["near_us"], exchange_info["far_us"] = round(exchange_info["near_us"], 3), round(exchange_info["far_us"], 3)
    model.set_decode_mode(args.decode_mode)
    # cache pre-filled with seeded int8 values directly in cache layout, as the reference's decode harness does
    C_fill = lib.flexllm_rt_fill_i8
    fx.check(C_fill(C.c_void_p(model.k_cache.ptr), C.c_size_t(model.k_cache.size), C.c_uint64(901), -100, 100, None))
    fx.check(C_fill(C.c_void_p(model.v_cache.ptr), C.c_size_t(model.v_cache.size), C.c_uint64(902), -100, 100, None))
    stream = fx.Stream()
    pos_end = cfg["max_pos"]
    pos_timed = pos_end - K
    pos_warm = pos_timed - W
    tok = fx.to_device(np.array([12345], np.int32))
    out_w = fx.zeros((max(W, 1),), np.int32)
    out = fx.zeros((K,), np.int32)
    device_sync()

    # ---- decode: W warm-up steps (also captures the graph), then exactly K timed steps -----------------
    if W:
        model.decode_greedy(tok, pos_warm, W, out_w, use_graph=True, stream=stream)
    stream.sync()
    e0, e1 = Event(), Event()
    device_sync()
    t0 = time.perf_counter()
    e0.record(stream)
    model.decode_greedy(tok, pos_timed, K, out, use_graph=True, stream=stream)
    e1.record(stream)
    e1.sync()
    device_sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ev_ms = e0.elapsed_ms(e1)
    model.check()                       # a barrier time-out or an id outside the vocabulary invalidates the figure: raise
    timed_tokens = out.numpy()
    ms_per_step = wall_ms / K
    tok_s = 1e3 / ms_per_step
    n_launch = (K + TOKENS_PER_LAUNCH - 1) // TOKENS_PER_LAUNCH
    mean_len = (pos_timed + 1 + pos_end) / 2.0
    bpt = bytes_per_token(cfg, mean_len)
    token_gbs = bpt / (ms_per_step * 1e-3) / 1e9

    # ---- dominant kernel: the fused gate/up GEMV (+SwiGLU), 33.6 MB of int8 weights per launch ---------
    H, I, L = cfg["hidden"], cfg["inter"], cfg["layers"]
    wgu = [synth.device_i8((2 * I, H), 7000 + l) for l in range(L)]            # 16 distinct buffers = 537 MB: streams from HBM
    sgu = synth.device_uniform_f32((2 * I,), 7100, 1e-4, 3e-4)
    xq = synth.device_i8((H,), 7200)
    xs = fx.to_device(np.array([0.02], np.float32))
    y = fx.empty((I,), np.float32)
    reps = 20
    for l in range(L):
        fx.check(lib.flexllm_linear_i8_gemv_swiglu(C.c_void_p(xq.ptr), C.c_void_p(xs.ptr), C.c_void_p(wgu[l].ptr),
                                                   C.c_void_p(sgu.ptr), C.c_void_p(y.ptr), H, I, stream.handle))
    k0, k1 = Event(), Event()
    k0.record(stream)
    for _ in range(reps):
        for l in range(L):
            lib.flexllm_linear_i8_gemv_swiglu(C.c_void_p(xq.ptr), C.c_void_p(xs.ptr), C.c_void_p(wgu[l].ptr),
                                              C.c_void_p(sgu.ptr), C.c_void_p(y.ptr), H, I, stream.handle)
    k1.record(stream)
    k1.sync()
    kern_ms = k0.elapsed_ms(k1) / (reps * L)
    kern_bytes = 2 * I * H + 4 * 2 * I + H + 4 + 4 * I            # weights + scales + x + s_x + y
    kern_gbs = kern_bytes / (kern_ms * 1e-3) / 1e9
    del wgu

    # ---- prefill: 1024 synthetic tokens through the 16 layers ------------------------------------------
    prefill_ms = None
    prefill_ms_4096 = None
    if not args.no_prefill:
        try:
            S = 1024
            x_in = synth.device_uniform_f32((S, H), 4243, -1.7, 1.7)
            model.prefill_hidden(x_in, stream=stream)
            stream.sync()
            p0, p1 = Event(), Event()
            p0.record(stream)
            for _ in range(3):
                model.prefill_hidden(x_in, stream=stream)
            p1.record(stream)
            p1.sync()
            prefill_ms = p0.elapsed_ms(p1) / 3
            if cfg["max_pos"] >= 4096:                       # the maximum context in one pass
                x4 = synth.device_uniform_f32((4096, H), 4244, -1.7, 1.7)
                model.prefill_hidden(x4, stream=stream)
                stream.sync()
                p0.record(stream)
                model.prefill_hidden(x4, stream=stream)
                p1.record(stream)
                p1.sync()
                prefill_ms_4096 = p0.elapsed_ms(p1)
                del x4
        except Exception as e:  # prefill path not available in this build
            print("prefill leg skipped: %s" % e, file=sys.stderr)

    # ---- module-level legs: the other configurations the metric's source names, each against its roofline ----
    modules = None
    peaks = None
    if not args.no_modules:
        # measured peaks of this GPU (HBM stream, matrix cores alone), beside the published ones
        peaks = measured_peaks(fx, lib, synth, stream, Event)
        modules = module_legs(fx, lib, synth, ops, stream, Event, peaks)
        if not args.no_prefill and cfg["max_pos"] >= 1024:
            # HMT plug-in at the reference's segment sizes (990 tokens, summary 495, recurrent 32, 64 memory slots):
            # one middle segment = stage 0 (512 rows) + retrieval + stage 1 (1024 rows) + memory update
            from flexllm_amd import hmt
            wq = synth.device_uniform_f32((H, H), 9401, -0.02, 0.02); wk = synth.device_uniform_f32((H, H), 9402, -0.02, 0.02)
            t_emb = synth.device_uniform_f32((H,), 9403, -1.0, 1.0)
            emb = synth.device_uniform_f32((3 * 990, H), 9404, -1.7, 1.7)
            plug = hmt.Hmt(model, wq, wk, t_emb)
            plug.run(emb, stream=stream); stream.sync()
            h0, h1 = Event(), Event()
            h0.record(stream)
            plug.run(emb, stream=stream)
            h1.record(stream); h1.sync()
            ms = h0.elapsed_ms(h1)
            modules["hmt_3_segments_of_990"] = {"ms": round(ms, 3), "prefill_passes": 5, "tokens_per_s": round(3 * 990 / ms * 1e3, 1),
                                                "note": "segment loop incl. host sequencing: 3 stage-1 passes of 1024 rows and 2 stage-0 passes of 512 rows through the 16 layers"}
            del plug, wq, wk, emb
        # top-k sampling loop (the reference's own generation loop): one launch sequence per token, top_k = 5
        n_s = 32
        rands = fx.to_device(np.random.default_rng(7).random(n_s).astype(np.float32))
        tok_s_io = fx.to_device(np.array([12345], np.int32)); out_s = fx.zeros((n_s,), np.int32)
        model.decode_sample(tok_s_io, cfg["max_pos"] - 2 * n_s, n_s, rands, 5, out_s, stream=stream); stream.sync()
        s0, s1 = Event(), Event()
        s0.record(stream)
        model.decode_sample(tok_s_io, cfg["max_pos"] - n_s, n_s, rands, 5, out_s, stream=stream)
        s1.record(stream); s1.sync()
        ms = s0.elapsed_ms(s1)
        # prompt -> tokens (the reference's combined prefill + decode harness): 1025-token prompt, 64 greedy tokens
        n_p, n_g = 1025, 64
        prompt = fx.to_device(np.random.default_rng(11).integers(0, cfg["vocab"], n_p).astype(np.int32))
        out_g = fx.zeros((n_g,), np.int32)
        gen = lambda: fx.check(lib.flexllm_llama_generate(model.handle, C.c_void_p(prompt.ptr), n_p, n_g, None, 0, C.c_void_p(out_g.ptr), stream.handle))
        gen(); stream.sync()
        g0, g1 = Event(), Event()
        g0.record(stream); gen(); g1.record(stream); g1.sync()
        modules["generate_prompt1025_greedy64"] = {"ms": round(g0.elapsed_ms(g1), 3), "prefilled_tokens": n_p - 1, "generated_tokens": n_g}
        modules["decode_top5_sampling_ctx4096"] = {"ms_per_token": round(ms / n_s, 4), "tokens_per_s": round(n_s / ms * 1e3, 1), "steps": n_s}
        # the shipped W4A4 configuration decoded by the persistent kernel's W4A4 instance (nibble-packed weights, int4
        # output head): same loop as the headline, 64 greedy tokens per launch up to the maximum context, with its own
        # HBM roofline line (half the weight bytes per token)
        w4 = llama.synth_weights_w4a4(cfg, seed=5, device=True, embed_range=0.03)
        model4 = llama.Llama(cfg, w4)
        del w4
        lib.flexllm_rt_fill_i8(C.c_void_p(model4.k_cache.ptr), C.c_size_t(model4.k_cache.size), C.c_uint64(911), -100, 100, stream.handle)
        lib.flexllm_rt_fill_i8(C.c_void_p(model4.v_cache.ptr), C.c_size_t(model4.v_cache.size), C.c_uint64(912), -100, 100, stream.handle)
        n4 = TOKENS_PER_LAUNCH
        tok4 = fx.to_device(np.array([12345], np.int32)); out4 = fx.zeros((n4,), np.int32)
        model4.decode_greedy(tok4, cfg["max_pos"] - 2 * n4, n4, out4, use_graph=False, stream=stream); stream.sync()
        q0, q1 = Event(), Event()
        q0.record(stream)
        model4.decode_greedy(tok4, cfg["max_pos"] - n4, n4, out4, use_graph=False, stream=stream)
        q1.record(stream); q1.sync()
        model4.check()
        us4 = q0.elapsed_ms(q1) * 1e3 / n4
        x4 = synth.device_uniform_f32((1024, cfg["hidden"]), 4245, -1.7, 1.7)
        model4.prefill_hidden(x4, stream=stream); stream.sync()
        r0, r1 = Event(), Event()
        r0.record(stream)
        for _ in range(2):
            model4.prefill_hidden(x4, stream=stream)
        r1.record(stream); r1.sync()
        pf4_ms = r0.elapsed_ms(r1) / 2
        del x4
        Hh, KVh, Ih, Lh, Vh = cfg["hidden"], cfg["kv_hidden"], cfg["inter"], cfg["layers"], cfg["vocab"]
        n_w = Lh * (Hh * Hh + 2 * KVh * Hh + Hh * Hh + 2 * Ih * Hh + Hh * Ih)
        rows = Lh * (Hh + 2 * KVh + Hh + 2 * Ih + Hh)
        bytes4 = n_w // 2 + 8 * rows + 4 * (2 * Lh + 1) * Hh + Vh * Hh // 2 + 8 * Vh \
            + Lh * 2 * KVh * (cfg["max_pos"] - n4 / 2.0) + Lh * 2 * KVh
        modules["w4a4_decode_ctx4096"] = {
            "us_per_token": round(us4, 2), "tokens_per_s": round(1e6 / us4, 1), "bytes_per_token": int(bytes4),
            "roofline": {"bound": "hbm", "kernel": "decode_mega_w4_kernel (1 launch of %d tokens)" % n4,
                         "achieved": round(bytes4 / us4 / 1e3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(bytes4 / us4 / 1e3 / HBM_PEAK_GBS, 4)},
            "distinct_tokens": int(len(set(out4.numpy().tolist()))),
            "prefill_ms_1024": round(pf4_ms, 3),
            "note": "int4 weights two per byte + scale and row sum per output row, int4 output head, int8 KV cache; "
                    "the kernel is bound by its exchanges between workgroups, not by bytes"}
        model4.close()
        del model4

    # ---- CPU baseline: the oracle (scalar C port of the reference modules), measured, not extrapolated -----
    # whole tokens of the same model (16 layers, context 4096, full fp16 head over 128256 rows) on the host's cores:
    # single thread, then all threads (OpenMP over independent output rows / heads; same arithmetic, same results)
    cpu = None
    if not args.no_cpu:
        from oracle import oracle
        hw = {k: ([a.numpy() for a in v] if isinstance(v, list) else v.numpy()) for k, v in dev_w.items()}
        hw["embed"] = hw["embed"].view(np.uint16)
        om = oracle.OracleModel(cfg, hw)
        kc, vc = om.new_caches()
        rr = np.random.default_rng(903)
        kc[:] = rr.integers(-100, 101, kc.shape, dtype=np.int8)
        vc[:] = rr.integers(-100, 101, vc.shape, dtype=np.int8)
        x = synth.host_normal_f32((H,), 905)
        olib = oracle.lib()
        n_threads = int(olib.fxo_max_threads())

        def timed_tokens_cpu(n_tok, budget_s):
            t0 = time.perf_counter()
            done = 0
            for i in range(n_tok):
                om.decode_token(x, cfg["max_pos"] - n_tok + i, kc, vc, want_logits=True)
                done += 1
                if time.perf_counter() - t0 > budget_s:
                    break
            return done, time.perf_counter() - t0

        olib.fxo_set_threads(1)
        n1, t1 = timed_tokens_cpu(8, 12.0)
        olib.fxo_set_threads(n_threads)
        om.decode_token(x, cfg["max_pos"] - 1, kc, vc, want_logits=True)       # thread pool start-up outside the timing
        nN, tN = timed_tokens_cpu(32, 10.0)
        cpu = {"value": round(nN / tN, 4), "unit": "tok/s", "cores": n_threads, "kind": "port",
               "single_core_value": round(n1 / t1, 4),
               "sample": "%d whole tokens (16 layers, context 4096, full head) on %d OpenMP threads in %.1f s; single thread: "
                         "%d tokens in %.1f s (C oracle, host reports %d cpus)" % (nN, n_threads, tN, n1, t1, os.cpu_count())}
        del om, kc, vc
        # the CPU figure beside the prefill leg: one full-size layer on 1024 tokens, measured (a 16-layer prefill is 16 of them)
        if prefill_ms is not None:
            cfg1 = llama.make_config(layers=1, vocab=256, max_pos=1024)
            hw1 = {k: (v[:1] if isinstance(v, list) else v) for k, v in hw.items()}
            hw1["embed"] = hw["embed"][:256]; hw1["rope_sin"] = hw["rope_sin"][:1024]; hw1["rope_cos"] = hw["rope_cos"][:1024]
            hw1["gamma"] = np.ascontiguousarray(hw["gamma"][:3])
            for n in ("q_s", "k_s", "v_s", "a_s"):
                hw1[n] = np.ascontiguousarray(hw[n][:1])
            om1 = oracle.OracleModel(cfg1, hw1)
            k1, v1 = om1.new_caches()
            xp = synth.host_normal_f32((1024, H), 906)
            t0 = time.perf_counter(); om1.prefill(xp, k1, v1); t_layer = time.perf_counter() - t0
            cpu["prefill_1024_one_layer_ms"] = round(t_layer * 1e3, 1)
            cpu["prefill_1024_16_layers_ms_at_that_rate"] = round(16 * t_layer * 1e3, 1)
        # and beside every module leg
        if modules is not None:
            for name, fig in cpu_module_legs(oracle, cfg, n_threads).items():
                if name in modules:
                    modules[name]["cpu_oracle"] = fig

    traffic_tok = measured_traffic_per_token()
    # prefill against the int8 MFMA roofline: 16 x (linear stack 2*M*sum(K*N) + attention 2*2*heads*S*S*64, full S^2)
    prefill_roof = None
    if prefill_ms is not None:
        S = 1024
        lin = 2 * S * (H * (H + 2 * cfg["kv_hidden"]) + H * H + 2 * I * H + I * H)
        att = 2 * 2 * cfg["q_heads"] * S * S * cfg["head_dim"]
        ops_total = L * (lin + att)
        prefill_roof = {"bound": "mfma", "ops": int(ops_total), "achieved": round(ops_total / (prefill_ms * 1e-3) / 1e12, 1),
                        "peak": INT8_PEAK_TOPS, "unit": "TOP/s", "frac": round(ops_total / (prefill_ms * 1e-3) / 1e12 / INT8_PEAK_TOPS, 4),
                        "frac_of_measured_peak": None if not peaks else round(ops_total / (prefill_ms * 1e-3) / 1e12 / peaks["mfma_i8"]["random_lds_TOPs"], 4),
                        "note": "whole 1024-token prefill (16 layers: norms, quantisation, GEMMs, attention with the full S^2 counted, Hadamard)"}
    result = {
        "metric": "decode tok/s + prefill ms (1024 tok), Llama-3.2-1B W8A8, % HBM/MFMA roofline",
        "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": "Llama-3.2-1B W8A8 SpinQuant greedy decode, batch 1, int8 KV cache, context %d..%d, "
                               "fp16 tied lm_head, %s" % (pos_timed + 1, pos_end, ("one persistent-kernel launch per %d tokens" % TOKENS_PER_LAUNCH)
                                                         if args.decode_mode == 0 else "one kernel per stage, HIP graph replay"),
                   "layers": cfg["layers"], "context": pos_end, "device": fx.device.device_name()},
        "decode": {"bytes_per_token": int(bpt), "achieved_GBs": round(token_gbs, 1),
                   "hbm_frac": round(token_gbs / HBM_PEAK_GBS, 4), "event_ms_per_step": round(ev_ms / K, 5),
                   "last_tokens": timed_tokens[-4:].tolist(), "distinct_tokens": int(len(set(timed_tokens.tolist()))),
                   # where the words that workgroups hand to each other live: one copy per I/O die when the
                   # calibration at model creation could tell the dies' memory apart
                   "exchange_memory": exchange_info},
        "prefill_ms_1024": None if prefill_ms is None else round(prefill_ms, 3),
        "prefill_ms_4096": None if prefill_ms_4096 is None else round(prefill_ms_4096, 3),
        "prefill_roofline": prefill_roof,
        # dominant kernel: the persistent decode kernel (all layers + lm_head + arg-max of every token of a
        # launch); algorithmic bytes per launch = bytes_per_token x tokens in the launch, duration from HIP
        # events around the timed launches (nothing else runs between them).  `traffic` is per launch too.
        "roofline": {"bound": "hbm", "kernel": "decode_mega_kernel (%d launches of <= %d tokens)" % (n_launch, TOKENS_PER_LAUNCH),
                     "achieved": round(bpt * K / (ev_ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(bpt * K / (ev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "frac_of_measured_peak": None if not peaks else round(bpt * K / (ev_ms * 1e-3) / 1e9 / peaks["hbm"]["read_stream_GBs"], 4),
                     "traffic": int(traffic_tok * K / n_launch) if (traffic_tok and cfg["layers"] == 16 and pos_end == 4096) else None,
                     "bytes_per_launch": int(bpt * K / n_launch), "tokens_per_launch": round(K / n_launch, 2),
                     "avg_us": round(ev_ms / n_launch * 1e3, 2), "us_per_token": round(ev_ms / K * 1e3, 2)},
        "gemv_gate_up": {"kernel": "gemv_i8_kernel<2,4,swiglu> stand-alone (2048->2x8192), 16 distinct weight buffers",
                         "achieved_GBs": round(kern_gbs, 1), "hbm_frac": round(kern_gbs / HBM_PEAK_GBS, 4),
                         "bytes_per_launch": int(kern_bytes), "avg_us": round(kern_ms * 1e3, 3)},
        "peaks": peaks,
        "modules": modules,
        "cpu_baseline": cpu,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
