"""HMT long-context plug-in on top of the prefill graph (Modules/HMT.h, HMT_SpinQuant_Llama_32_1B/HMT_SpinQuant_Unit.h).

A long text is cut into segments of `seg_len` tokens.  For segment n > 0, stage 0 runs the layer stack on
[T, first `sum_seg_len` tokens of the segment, T] (T = the summary-prompt embedding) and takes the hidden state of the
last T as S_n; the query Wq S_n attends over the ring of `mem_num` memory embeddings (keys Wk M_j) and returns P_n.
Stage 1 runs the layer stack on [P_n, last `rec_seg_len` tokens before the segment, the segment, P_n]; the hidden state
of the trailing P_n becomes the memory M_n of slot n % mem_num.  The hidden states of the segment's own tokens are
the plug-in's output.

Everything stays on the device; the host only sequences the stages, as the reference's segment loader does
(hmt_segment_loader_sync_template, Modules/HMT.h:8-195).  Sequences are padded with zero rows to a multiple of 32
(the prefill tile) instead of the reference's token-parallel factor of 8: rows behind a token do not influence it.
"""
import ctypes as C
import math

import numpy as np

from ._lib import lib, check
from .device import DeviceArray, zeros, _s

PAD = 32


def _p(a):
    return C.c_void_p(a.ptr) if a is not None else None


def linear_f32_gemv(x, w, stream=None, out=None):
    """y = W x in fp32 (dec_Linear_Layer_fp32xfp32, Modules/Linear_Layer.h:1041-1100); w: [n][k]."""
    n, k = w.shape
    y = out if out is not None else DeviceArray((n,), np.float32)
    check(lib().flexllm_linear_f32_gemv(_p(x), _p(w), _p(y), k, n, _s(stream)))
    return y


def hmt_retrieve(q, kmem, mmem, scale, stream=None):
    """(softmaxed scores over all slots, retrieved embedding) - Modules/HMT.h:278-316."""
    mem_num, hidden = mmem.shape
    a = DeviceArray((mem_num,), np.float32)
    p = DeviceArray((hidden,), np.float32)
    check(lib().flexllm_hmt_retrieve(_p(q), _p(kmem), _p(mmem), _p(a), _p(p), mem_num, hidden, C.c_float(scale), _s(stream)))
    return a, p


def hmt_stage_input(emb, t_embed, p_buf, stage, seq_off, cur_len, cur_sum_len, rec_len, tail_p, rows, stream=None, out=None):
    """Assembled input sequence [rows][hidden] of one stage (Modules/HMT.h:48-98, :125-170)."""
    hidden = emb.shape[1]
    x = out if out is not None else DeviceArray((rows, hidden), np.float32)
    check(lib().flexllm_hmt_stage_input(_p(emb), _p(t_embed), _p(p_buf), _p(x), stage, seq_off, cur_len, cur_sum_len, rec_len,
                                        int(bool(tail_p)), rows, hidden, _s(stream)))
    return x


class Hmt:
    """Segment loop around a `llama.Llama` model.  wq, wk: device [hidden][hidden] fp32 (the plug-in's query and key
    projections, `hmt_wq_wk_mmaps` of the reference); t_embed: device [hidden] fp32."""

    def __init__(self, model, wq, wk, t_embed, seg_len=990, sum_seg_len=495, rec_seg_len=32, mem_num=64, scale=None):
        hidden = model.cfg["hidden"]
        if wq.shape != (hidden, hidden) or wk.shape != (hidden, hidden) or t_embed.shape != (hidden,):
            raise ValueError("wq, wk must be [hidden][hidden] and t_embed [hidden]")
        if not (0 < sum_seg_len <= seg_len and rec_seg_len >= 0 and 0 < mem_num <= 1024):
            raise ValueError("bad segment parameters")
        longest = (1 + rec_seg_len + seg_len + 1 + PAD - 1) // PAD * PAD
        if longest > model.cfg["max_pos"]:
            raise ValueError("a stage of %d rows exceeds the model's max_pos %d" % (longest, model.cfg["max_pos"]))
        self.model, self.wq, self.wk, self.t_embed = model, wq, wk, t_embed
        self.seg_len, self.sum_seg_len, self.rec_seg_len, self.mem_num = seg_len, sum_seg_len, rec_seg_len, mem_num
        self.scale = float(scale) if scale is not None else math.sqrt(hidden)     # sqrt_HIDDEN_DIM (HMT_SpinQuant_Unit.h:103)
        # Stage buffers live as long as the plug-in: freeing device memory waits for the device, which would stall
        # the host between the stages of every segment.
        self._x = DeviceArray((longest, hidden), np.float32)
        self._h = DeviceArray((longest, hidden), np.float32)
        self._q = DeviceArray((hidden,), np.float32)
        self._k = DeviceArray((hidden,), np.float32)
        self.reset()

    def reset(self):
        hidden = self.model.cfg["hidden"]
        self.mmem = zeros((self.mem_num, hidden), np.float32)      # memory and key caches start at zero (HMT.h:369-378, :428-437)
        self.kmem = zeros((self.mem_num, hidden), np.float32)
        self.p_buf = zeros((hidden,), np.float32)                  # HMT.h:29-35

    def _row(self, arr, r):
        hidden = arr.shape[1]
        return arr.view(r * hidden * 4, (hidden,), np.float32)

    def run(self, emb, stream=None):
        """emb: device [seq_len][hidden] fp32 token embeddings.  Returns (list of device [cur_len][hidden] hidden states,
        one per segment; list of retrieved embeddings P_n for n >= 1)."""
        seq_len, hidden = emb.shape
        seg_num = (seq_len + self.seg_len - 1) // self.seg_len
        up = lambda n: (n + PAD - 1) // PAD * PAD
        outs, ps = [], []
        copy = lib().flexllm_rt_memcpy_d2d
        for seg in range(seg_num):
            cur = self.seg_len if seg < seg_num - 1 else seq_len - seg * self.seg_len
            cur_sum = min(cur, self.sum_seg_len)
            off = seg * self.seg_len
            last = seg == seg_num - 1
            if seg > 0:
                rows0 = up(1 + cur_sum + 1)
                x0 = hmt_stage_input(emb, self.t_embed, self.p_buf, 0, off, cur, cur_sum, self.rec_seg_len, False, rows0, stream,
                                     out=self._x.view(0, (rows0, hidden)))
                h0 = self.model.prefill_hidden(x0, stream=stream, out=self._h.view(0, (rows0, hidden)))
                q_n = linear_f32_gemv(self._row(h0, 1 + cur_sum), self.wq, stream, out=self._q)
                _, p_n = hmt_retrieve(q_n, self.kmem, self.mmem, self.scale, stream)
                self.p_buf = p_n
                ps.append(p_n)
            rows1 = up(1 + self.rec_seg_len + cur + 1)
            x1 = hmt_stage_input(emb, self.t_embed, self.p_buf, 1, off, cur, cur_sum, self.rec_seg_len, not last, rows1, stream,
                                 out=self._x.view(0, (rows1, hidden)))
            h1 = self.model.prefill_hidden(x1, stream=stream, out=self._h.view(0, (rows1, hidden)))
            out = DeviceArray((cur, hidden), np.float32)
            check(copy(_p(out), C.c_void_p(h1.ptr + (1 + self.rec_seg_len) * hidden * 4), C.c_size_t(cur * hidden * 4), _s(stream)))
            outs.append(out)
            if not last:
                slot = seg % self.mem_num                                       # HMT.h:403, :465-466
                m_row = self._row(h1, 1 + self.rec_seg_len + cur)
                check(copy(C.c_void_p(self.mmem.ptr + slot * hidden * 4), _p(m_row), C.c_size_t(hidden * 4), _s(stream)))
                k_n = linear_f32_gemv(m_row, self.wk, stream, out=self._k)
                check(copy(C.c_void_p(self.kmem.ptr + slot * hidden * 4), _p(k_n), C.c_size_t(hidden * 4), _s(stream)))
        return outs, ps
