#!/usr/bin/env python3
"""Benchmark of the fused per-layer row kernels on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extra]

A step is one pass of the dense 27B-class prefill chunk's three fused op-sets over one synthetic batch that is already
resident in HBM (4096 tokens x hidden 5120, bf16 activations, fp32 residual). Consecutive steps take different copies of the
batch (eight in rotation, 5.6 GB), so no launch finds a line of its own inputs or outputs in the 256 MB Infinity Cache: the
figures are HBM figures. (`same_batch` in the output is the same loop on one copy, where part of each launch is served by that cache.)
  (i)   residual add (bf16 addend) + RMSNorm -> fp32 residual + bf16 normed rows          camx_add_rms_bf16
  (ii)  QK-norm + YaRN rotary on 64 Q + 8 KV heads (+ 8 V heads) of dim 128 -> fp16          camx_qk_rope_bf16
  (iii) SwiGLU on a 4096 x 17408 gate / up pair -> q8_1 blocks in the MMQ layout              camx_swiglu_mmq_q8_1
The value is algorithmic bytes (every input read once, every output written once) per second over the whole step.
One JSON line goes to stdout; `roofline` describes the dominant kernel, `cpu_baseline` the CPU oracle timed on a bounded
sample of the same workload on this host, `opsets` the other shapes (decode token, embedding gather, hybrid verify
batch, batched decode with the Q8 KV codec) in microseconds and GB/s per launch.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
TRAFFIC_FILE = os.path.join(ROOT, 'profiles', 'prefill_chunk_step_hbm_traffic.txt')


def hbm_traffic():
    """HBM bytes per launch of each kernel of the step, from the committed rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summary (lines
    `traffic_bytes <entry point> <device kernel> <bytes>`). The summary names the device kernel it was measured on: a kernel that the
    library no longer contains makes the figure stale, and this raises instead of reporting it."""
    out = {}
    lib_bytes = open(os.path.join(ROOT, 'caminus_amd', 'libcamx.so'), 'rb').read()
    for line in open(TRAFFIC_FILE):
        f = line.split()
        if len(f) == 4 and f[0] == 'traffic_bytes':
            if f[2].encode() not in lib_bytes:
                raise RuntimeError(f'{TRAFFIC_FILE} was measured on kernel {f[2]}, which libcamx.so no longer has: re-run the counter profile')
            out[f[1]] = int(f[3])
    return out


I, F, L64 = C.c_int, C.c_float, C.c_int64
NULL = C.c_void_p(None)


def _p(t):
    return C.c_void_p(t.data_ptr()) if t is not None else NULL


class Bench:
    def __init__(self):
        import torch
        from caminus_amd.device import lib
        self.torch = torch
        self.L = lib.load()
        self.check = lib.check
        self.dev = torch.device('cuda:0')
        torch.cuda.set_device(self.dev)
        self.stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        self.flush_buf = None

    def call(self, name, *args):
        self.check(getattr(self.L, name)(*args, self.stream))

    def acts(self, shape, dtype, seed, frac=1e-3, scale=50.0):
        """N(0, 1) with `frac` of the entries scaled by `scale`, generated on the device"""
        torch = self.torch
        g = torch.Generator(device=self.dev); g.manual_seed(seed)
        x = torch.randn(shape, generator=g, device=self.dev, dtype=torch.float32)
        m = torch.rand(shape, generator=g, device=self.dev) < frac
        x = torch.where(m, x * scale, x)
        return x.to(dtype).contiguous()

    def gamma(self, n, seed):
        torch = self.torch
        g = torch.Generator(device=self.dev); g.manual_seed(seed)
        return (1.0 + 0.1 * torch.randn(n, generator=g, device=self.dev)).contiguous()

    def flush(self):
        """push the previous launch's lines out of L2 / MALL: a 512 MiB fill (untimed)"""
        torch = self.torch
        if self.flush_buf is None: self.flush_buf = torch.empty(512 << 20, dtype=torch.uint8, device=self.dev)
        self.flush_buf.fill_(1)

    def ramp(self, seconds=0.25):
        """keep the GPU busy (device copies of 256 MiB) until it has left its idle clocks"""
        torch = self.torch
        src = torch.ones(256 << 20, dtype=torch.uint8, device=self.dev); dst = torch.empty_like(src)
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            for _ in range(20): dst.copy_(src)
            torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    def time_launch(self, fn, reps=50, warm=10, flush=False):
        """median and mean duration (us) of one launch of fn, HIP events on the launch stream"""
        torch = self.torch
        for _ in range(warm): fn()
        torch.cuda.synchronize()
        ts = []
        for _ in range(reps):
            if flush: self.flush()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(); fn(); b.record(); b.synchronize()
            ts.append(a.elapsed_time(b) * 1e3)
        ts.sort()
        return ts[len(ts) // 2], sum(ts) / len(ts)


def yarn_par(torch, dev, seed, base=1e6, eps=1e-6, yarn=True):
    import numpy as np
    from caminus_amd import rope
    rng = np.random.default_rng(seed)
    qn = (1 + 0.1 * rng.standard_normal(128)).astype(np.float32); kn = (1 + 0.1 * rng.standard_normal(128)).astype(np.float32)
    ts = np.float32(np.float32(base) ** np.float32(-2.0 / 128))
    par = np.concatenate([qn, kn, np.array([ts, eps], np.float32)])
    if yarn: par = np.concatenate([par, rope.yarn_table(128, base, 4.0, 32768)])
    return torch.from_numpy(par.astype(np.float32)).to(dev), par.astype(np.float32)


def config3(B, T=4096, H=5120, nh=64, nkv=8, Fh=17408, seed0=1003):
    """the dense prefill chunk: buffers and the three launches"""
    torch = B.torch
    w = dict(T=T, H=H, nh=nh, nkv=nkv, Fh=Fh)
    w['x'] = B.acts((T, H), torch.float32, seed0)
    w['d'] = B.acts((T, H), torch.bfloat16, seed0 + 1)
    w['nw'] = B.gamma(H, seed0 + 2)
    w['hbf'] = torch.empty((T, H), dtype=torch.bfloat16, device=B.dev)
    ldq = (nh + 2 * nkv) * 128
    w['qkv'] = B.acts((T, ldq), torch.bfloat16, seed0 + 3)
    w['par'], w['par_np'] = yarn_par(torch, B.dev, seed0 + 4)
    w['q16'] = torch.empty((T, nh, 128), dtype=torch.float16, device=B.dev)
    w['cache'] = torch.empty((T, 2 * nkv * 128), dtype=torch.float16, device=B.dev)
    w['gu'] = B.acts((T, 2 * Fh), torch.bfloat16, seed0 + 5)
    kp = (Fh + 511) // 512 * 512
    w['y'] = torch.empty((kp // 128, T, 144), dtype=torch.uint8, device=B.dev)
    w['ldq'] = ldq
    w['bytes'] = {
        'add_rms_bf16': T * H * (4 + 2 + 4 + 2) + H * 4,
        'qk_rope_bf16': T * ldq * 2 + 323 * 4 + T * ldq * 2,
        'swiglu_mmq_q8_1': T * 2 * Fh * 2 + (kp // 128) * T * 144,
    }
    w['launch'] = {
        'add_rms_bf16': lambda: B.call('camx_add_rms_bf16', _p(w['x']), _p(w['d']), _p(w['nw']), F(1e-6), NULL, _p(w['hbf']), I(H), I(T)),
        'qk_rope_bf16': lambda: B.call('camx_qk_rope_bf16', _p(w['qkv']), I(ldq), I(nh), I(nkv), _p(w['par']), I(0), _p(w['q16']), _p(w['cache']), I(T), I(1)),
        'swiglu_mmq_q8_1': lambda: B.call('camx_swiglu_mmq_q8_1', _p(w['gu']), L64(2 * Fh), L64(Fh), _p(w['y']), NULL, I(T), I(1)),
    }
    return w


def extra_opsets(B):
    """the other shapes, one launch each: (name, algorithmic bytes, launch)"""
    import numpy as np
    torch = B.torch
    out = []
    # decode token, hidden 2048 (batch 1)
    N = 2048
    x = B.acts((1, N), torch.float32, 11); d = B.acts((1, 1, N), torch.float32, 12); nw = B.gamma(N, 13)
    h = torch.empty((1, N), device=B.dev); h16 = torch.empty((1, N), dtype=torch.float16, device=B.dev)
    q8 = torch.empty((N // 32) * 36, dtype=torch.uint8, device=B.dev)
    out.append(('c1_add_rms_h_h16', N * 4 * 3 + N * 4 * 2 + N * 2,
                lambda: B.call('camx_q3p_add_rms16', _p(x), _p(d), NULL, I(1), _p(nw), F(1e-6), _p(h), _p(h16), I(N), I(1))))
    out.append(('c1_q8_1', N * 4 + N // 32 * 36, lambda: B.call('camx_gg_quantize_q8_1', _p(h), _p(q8), L64(N), I(0), F(0), NULL)))
    nh, nkv = 32, 4
    ldq = (nh + 2 * nkv) * 128
    qkv = B.acts((1, ldq), torch.float32, 14); par, _ = yarn_par(torch, B.dev, 15, yarn=False)
    q16 = torch.empty((1, nh, 128), dtype=torch.float16, device=B.dev); cache = torch.zeros((4096, 2 * nkv * 128), dtype=torch.float16, device=B.dev)
    out.append(('c1_qk_rope', ldq * 4 + 258 * 4 + nh * 128 * 2 + 2 * nkv * 128 * 2,
                lambda: B.call('camx_q3p_qk_rope', _p(qkv), I(ldq), I(nh), I(nkv), _p(par), I(1234), _p(q16), _p(cache), I(1), I(0))))
    n = 8 * 768
    g = B.acts((n,), torch.float32, 16); u = B.acts((n,), torch.float32, 17); y16 = torch.empty(n, dtype=torch.float16, device=B.dev)
    out.append(('c1_swiglu', n * 10, lambda: B.call('camx_q3p_swiglu', _p(g), _p(u), _p(y16), I(n))))
    # the decode token's attention inputs as the reference's tape chains them (python/caminus/engine/q3moe_one.py:316-318): OP_QK_NR (k) ->
    # OP_KV_APPEND (fp16 rows) and OP_QK_NR (q), three launches, and the one that replaces them
    hd1, M1 = 128, nkv * 128
    q1 = B.acts((nh, hd1), torch.float32, 18); k1 = B.acts((nkv, hd1), torch.float32, 19); v1 = B.acts((1, M1), torch.float32, 20)
    wq1 = B.gamma(hd1, 21); wk1 = B.gamma(hd1, 22); qo1 = torch.empty((nh, hd1), device=B.dev); ko1 = torch.empty((nkv, hd1), device=B.dev)
    posw1 = torch.tensor([1234], dtype=torch.int32, device=B.dev); err1 = torch.zeros(1, dtype=torch.int32, device=B.dev)
    ts6 = float(np.float32(np.float32(1e6) ** np.float32(-2.0 / hd1))); eb1 = int(np.array([1e-6], np.float32).view(np.int32)[0])
    def nr_kv_three():
        B.call('camx_op_qk_nr', _p(k1), I(hd1), I(nkv), I(hd1), _p(wk1), _p(posw1), _p(ko1), I(hd1), F(ts6), I(eb1), I(1))
        B.call('camx_op_kv_append', _p(ko1), _p(v1), _p(cache), _p(posw1), I(M1), I(0), _p(err1), I(4096), I(1))
        B.call('camx_op_qk_nr', _p(q1), I(hd1), I(nh), I(hd1), _p(wq1), _p(posw1), _p(qo1), I(hd1), F(ts6), I(eb1), I(1))
    by1 = (nh + 2 * nkv) * hd1 * 4 + 2 * hd1 * 4 + nh * hd1 * 4 + 2 * M1 * 2
    out.append(('c1_qk_nr_kv_append_three_launches', by1, nr_kv_three))
    out.append(('c1_qk_nr_kv_append_one_launch', by1,
                lambda: B.call('camx_qk_nr_kv', _p(q1), I(hd1), I(nh), _p(wq1), _p(k1), I(hd1), _p(v1), I(M1), I(nkv), _p(wk1), I(hd1), I(hd1), F(ts6), F(1e-6), I(0),
                               _p(posw1), NULL, _p(qo1), NULL, _p(cache), I(0), I(4096), _p(err1), I(1))))
    out.append(('_keep1', 0, [q1, k1, v1, wq1, wk1, qo1, ko1, posw1, err1]))
    # embedding gather, 151936 x 2048, 256 ids
    V, n_tok = 151936, 256
    rng = np.random.default_rng(1002)
    toks = torch.from_numpy(rng.integers(0, V, n_tok).astype(np.int32)).to(B.dev)
    gq = torch.Generator(device=B.dev); gq.manual_seed(1002)
    for fmt, name, rb, blk in ((0, 'q4_k', N // 256 * 144, 144), (1, 'q8_0', N // 32 * 34, 34)):
        tab = torch.randint(0, 256, (V, rb), generator=gq, device=B.dev, dtype=torch.uint8)
        sc = (torch.rand((V, rb // blk, 2 if fmt == 0 else 1), generator=gq, device=B.dev) * 9e-3 + 1e-3).to(torch.float16)
        tab.view(V, rb // blk, blk)[:, :, :(4 if fmt == 0 else 2)] = sc.view(torch.uint8).view(V, rb // blk, -1)
        xo = torch.empty((n_tok, N), device=B.dev); xbf = torch.empty((n_tok, N), dtype=torch.bfloat16, device=B.dev)
        hh = torch.empty((n_tok, N), device=B.dev); qq = torch.empty(n_tok * (N // 32) * 36, dtype=torch.uint8, device=B.dev)
        out.append((f'c2_gather_{name}_f32_bf16', n_tok * (rb + 4 + N * 6),
                    (lambda tab=tab, rb=rb, fmt=fmt, xo=xo, xbf=xbf: B.call('camx_emb_gather', _p(tab), L64(rb), I(V), _p(toks), _p(xo), _p(xbf), I(N), I(n_tok), I(fmt)))))
        out.append((f'c2_gather_{name}_add_rms_q8_1', n_tok * (rb + 4 + N * 4 + N * 2 + N // 32 * 36) + N * 4,
                    (lambda tab=tab, rb=rb, fmt=fmt, xo=xo, xbf=xbf, qq=qq: B.call('camx_emb_gather_add_rms', _p(tab), L64(rb), I(V), _p(toks), _p(xo), _p(xbf), NULL, _p(nw),
                                                                                   F(1e-6), NULL, NULL, _p(qq), I(N), I(n_tok), I(fmt)))))
    # hybrid verify batch: 16 tokens, hidden 5120
    T4, D4 = 16, 256
    qg = B.acts((T4 * 24, 2 * D4), torch.bfloat16, 41); w4 = B.gamma(D4, 42)
    pos = torch.from_numpy(rng.integers(0, 65536, T4).astype(np.int32)).to(B.dev)
    o4 = torch.empty((T4 * 24, D4), dtype=torch.bfloat16, device=B.dev)
    ts7 = float(np.float32(np.float32(1e7) ** np.float32(-2.0 / 64)))
    out.append(('c4_qk_nr_partial_rotary_q', T4 * 24 * D4 * 4 + D4 * 4,
                lambda: B.call('camx_qk_nr_pos', _p(qg), I(2 * D4), I(24), _p(w4), I(D4), I(64), F(ts7), F(1e-6), _p(pos), _p(o4), I(T4), I(1))))
    a4 = B.acts((T4 * 24, D4), torch.bfloat16, 43)
    out.append(('c4_sigmoid_gate', T4 * 24 * D4 * 6,
                lambda: B.call('camx_gate_mul', _p(a4), _p(qg), _p(o4), L64(T4 * 24 * D4), I(D4), I(2 * D4), I(D4), I(2))))
    Cc = 10240
    xc = B.acts((T4, Cc), torch.bfloat16, 44); wc = B.acts((Cc, 4), torch.float32, 45, frac=0); st = B.acts((Cc, 3), torch.float32, 46, frac=0)
    yc = torch.empty((T4, Cc), dtype=torch.bfloat16, device=B.dev)
    out.append(('c4_conv4_silu', T4 * Cc * 4 + Cc * 16 + Cc * 12,
                lambda: B.call('camx_pf_gdn_conv', _p(xc), _p(wc), _p(st), _p(yc), I(Cc), I(T4), I(Cc), I(Cc), I(1))))
    l2o = torch.empty((T4 * 32, 128), dtype=torch.bfloat16, device=B.dev)
    out.append(('c4_l2norm_qk', T4 * 32 * 128 * 4,
                lambda: B.call('camx_pf_gdn_l2', _p(yc), _p(l2o), I(32), I(128), I(Cc), F(1e-6 / 128), I(T4), I(1))))
    # the same op-sets as the reference's engine chains them (python/caminus/engine/q35_dense.py:399-400, 408-418), one launch each
    l2f = torch.empty((T4 * 32, 128), dtype=torch.bfloat16, device=B.dev); ycf = torch.empty((T4, Cc), dtype=torch.bfloat16, device=B.dev)
    out.append(('c4_conv4_silu_l2_one_launch', T4 * Cc * 4 + Cc * 16 + Cc * 12 + T4 * 32 * 128 * 2,
                lambda: B.call('camx_gdn_conv_l2', _p(xc), _p(wc), _p(st), _p(ycf), _p(l2f), I(Cc), I(T4), I(Cc), I(Cc), I(32), F(1e-6 / 128), I(1))))
    # the tape's fp32 forms of the same layer (python/caminus/engine/q35_dense.py:396-400): OP_GDN_GATES, OP_GDN_CONV, OP_GDN_L2 and the one launch for the three
    H4 = 48
    xc32 = B.acts((T4, Cc), torch.float32, 61); st32 = B.acts((Cc, 3), torch.float32, 62, frac=0); xp32 = torch.zeros((T4, Cc), device=B.dev); yc32 = torch.empty((T4, Cc), device=B.dev)
    qk32 = torch.empty((T4 * 32, 128), device=B.dev); par4 = torch.zeros(4, dtype=torch.int32, device=B.dev)
    al4 = B.acts((T4, H4), torch.float32, 63); be4 = B.acts((T4, H4), torch.float32, 64); dt4 = B.acts((H4,), torch.float32, 65, frac=0); a4g = B.acts((H4,), torch.float32, 66, frac=0)
    gt4 = torch.empty((T4, 2 * H4), device=B.dev)
    def gdn_three():
        B.call('camx_op_gdn_gates', _p(al4), _p(be4), _p(dt4), _p(a4g), _p(gt4), I(H4), I(T4))
        B.call('camx_op_gdn_conv', _p(wc), _p(st32), _p(xc32), _p(par4), _p(yc32), _p(xp32), I(Cc), I(T4))
        B.call('camx_op_gdn_l2', _p(yc32), _p(qk32), I(32), I(128), F(1e-6 / 128), I(Cc), I(T4))
    byg = T4 * Cc * 4 * 3 + Cc * 28 + T4 * 32 * 128 * 4 + T4 * H4 * 16
    out.append(('c4_tape_gdn_gates_conv_l2_three_launches', byg, gdn_three))
    out.append(('c4_tape_gdn_gates_conv_l2_one_launch', byg,
                lambda: B.call('camx_op_gdn_conv_l2_gates', _p(wc), _p(st32), _p(xc32), _p(par4), _p(yc32), _p(xp32), _p(qk32), I(Cc), I(T4), I(32), F(1e-6 / 128),
                               _p(al4), _p(be4), _p(dt4), _p(a4g), _p(gt4), I(H4))))
    out.append(('_keep4g', 0, [xc32, st32, xp32, yc32, qk32, par4, al4, be4, dt4, a4g, gt4]))
    kx = B.acts((T4 * 4, D4), torch.bfloat16, 47); wk4 = B.gamma(D4, 48); ok4 = torch.empty((T4 * 4, D4), dtype=torch.bfloat16, device=B.dev)
    out.append(('c4_qk_nr_partial_rotary_k', T4 * 4 * D4 * 4 + D4 * 4,
                lambda: B.call('camx_qk_nr_pos', _p(kx), I(D4), I(4), _p(wk4), I(D4), I(64), F(ts7), F(1e-6), _p(pos), _p(ok4), I(T4), I(1))))
    out.append(('c4_qk_nr_partial_rotary_q_and_k_one_launch', T4 * 28 * D4 * 4 + 2 * D4 * 4,
                lambda: B.call('camx_qk_nr_qk', _p(qg), I(2 * D4), I(24), _p(w4), _p(kx), I(D4), I(4), _p(wk4), I(D4), I(64), F(ts7), F(1e-6), I(0), NULL, _p(pos),
                               _p(o4), _p(ok4), I(T4), I(1))))
    # the dense Q8 line of the same layer shape (fp32, as the reference's decode tape runs it): six launches, and the one that replaces them
    M4 = 4 * D4; rows4 = 65536 + T4; rb4 = 2 * (M4 // 32) * 34
    q32 = B.acts((T4 * 24, 2 * D4), torch.float32, 71); k32 = B.acts((T4, M4), torch.float32, 72); v32 = B.acts((T4, M4), torch.float32, 73)
    ko32 = torch.empty((T4 * 4, D4), device=B.dev); qo32 = torch.empty((T4 * 24, D4), device=B.dev); vr32 = v32.clone()
    cache4 = torch.zeros(rows4 * rb4, dtype=torch.uint8, device=B.dev); err4 = torch.zeros(1, dtype=torch.int32, device=B.dev)
    posw = torch.tensor([40000], dtype=torch.int32, device=B.dev)
    def dense_q8_six():
        B.call('camx_pf_qk_nr', _p(k32), I(D4), I(4), _p(wk4), I(D4), I(64), F(ts7), F(1e-6), I(40000), _p(ko32), I(T4), I(0))
        B.call('camx_pf_hadamard', _p(ko32), I(T4 * 4), I(256), I(1))
        B.call('camx_pf_hadamard', _p(vr32), I(T4 * M4 // 64), I(64), I(1))
        B.call('camx_own_kv_q8_append', _p(ko32), I(M4), _p(vr32), I(M4), I(M4), _p(cache4), I(40000), I(rows4), _p(err4), I(T4))
        B.call('camx_pf_qk_nr', _p(q32), I(2 * D4), I(24), _p(w4), I(D4), I(64), F(ts7), F(1e-6), I(40000), _p(qo32), I(T4), I(0))
        B.call('camx_pf_hadamard', _p(qo32), I(T4 * 24), I(256), I(1))
    by4 = T4 * (24 + 4 + 4) * D4 * 4 + T4 * 24 * D4 * 4 + T4 * rb4 + 2 * D4 * 4
    out.append(('c4_dense_q8_qk_nr_hadamard_append_six_launches', by4, dense_q8_six))
    out.append(('c4_dense_q8_qk_nr_hadamard_append_one_launch', by4,
                lambda: B.call('camx_qk_nr_q8', _p(q32), I(2 * D4), I(24), _p(k32), I(M4), _p(v32), I(M4), I(4), _p(w4), _p(wk4), I(64), F(ts7), F(1e-6), I(0), _p(posw), NULL,
                               _p(qo32), _p(cache4), I(rows4), _p(err4), I(T4))))
    # the attention output of the same line: the Hadamard in chunks of 64 and the gate multiply behind it (q35_dense.py:419-420)
    att32 = B.acts((T4 * 24, D4), torch.float32, 74); gat16 = torch.empty((T4 * 24, D4), dtype=torch.float16, device=B.dev)
    def att_two():
        B.call('camx_op_hadamard', _p(att32), I(T4 * 24 * D4 // 64), I(64), I(1))
        B.call('camx_op_gate_mul16', _p(att32), _p(q32), I(2 * D4), I(D4), _p(gat16), I(T4 * 24 * D4), I(D4))
    bya = T4 * 24 * D4 * (4 + 4 + 2)
    out.append(('c4_dense_q8_att_hadamard_gate_two_launches', bya, att_two))
    out.append(('c4_dense_q8_att_hadamard_gate_one_launch', bya,
                lambda: B.call('camx_op_hadamard_gate_mul16', _p(att32), NULL, _p(q32), I(2 * D4), I(D4), _p(gat16), I(T4 * 24 * D4), I(D4), I(64))))
    out.append(('_keep4', 0, [l2f, ycf, kx, wk4, ok4, q32, k32, v32, ko32, qo32, vr32, cache4, err4, posw, att32, gat16]))
    # batched decode: 256 sequences, Q8 KV codec into a paged cache
    S5 = 256
    x5 = B.acts((S5, N), torch.float32, 51); d5 = B.acts((S5, 1, N), torch.float32, 52)
    h5 = torch.empty((S5, N), device=B.dev); h516 = torch.empty((S5, N), dtype=torch.float16, device=B.dev)
    out.append(('c5_add_rms_256x2048', S5 * N * (12 + 6) + N * 4,
                lambda: B.call('camx_q3p_add_rms16', _p(x5), _p(d5), NULL, I(1), _p(nw), F(1e-6), _p(h5), _p(h516), I(N), I(S5))))
    qkv5 = B.acts((S5, ldq), torch.float32, 53)
    page, n_pages = 256, 65536
    rbq = 2 * (nkv * 128 // 32) * 34
    pos5 = rng.integers(0, 131072, S5).astype(np.int32)
    pt = rng.integers(0, n_pages, (S5, 512)).astype(np.int32)
    pt[np.arange(S5), pos5 // page] = rng.permutation(n_pages)[:S5]          # the pages this launch writes are distinct
    cache5 = torch.zeros(n_pages * page * rbq, dtype=torch.uint8, device=B.dev)
    err5 = torch.zeros(1, dtype=torch.int32, device=B.dev)
    pos5d, ptd = torch.from_numpy(pos5).to(B.dev), torch.from_numpy(pt).to(B.dev)
    q165 = torch.empty((S5, nh, 128), dtype=torch.float16, device=B.dev)
    out.append(('c5_qk_rope_hadamard_q8_paged', S5 * (ldq * 4 + 8 + nh * 128 * 2 + rbq) + 258 * 4,
                lambda: B.call('camx_qk_rope_paged', _p(qkv5), I(ldq), I(nh), I(nkv), _p(par), _p(pos5d), _p(q165), _p(cache5), _p(err5), _p(ptd), I(512),
                               I(page), I(n_pages), I(S5), I(0), I(1))))
    # hyper-connection glue at the one shape the reference publishes per-op times for (T = 2048, 4 streams of 2560; RX 7900 XTX:
    # hc_post_rms with bf16 copy and scale 0.466 ms, hc_mean 0.267 ms; docs/specs/spec-prefill-cache.md:276)
    Th, HC, Nh = 2048, 4, 2560
    bh = B.acts((Th, Nh), torch.float32, 61); injh = B.acts((Th, HC), torch.float32, 62, frac=0); resh = B.acts((Th, HC, Nh), torch.float32, 63)
    wh = B.gamma(HC * Nh, 64); xnbf = torch.empty((Th, HC, Nh), dtype=torch.bfloat16, device=B.dev); sclh = torch.empty(Th * HC, device=B.dev)
    gh = B.acts((Th, HC, Nh), torch.float32, 65); outh = torch.empty((Th, Nh), device=B.dev)
    out.append(('hc_post_rms_2048x4x2560_bf16_scale', Th * Nh * 4 + Th * HC * Nh * (4 + 4 + 2) + HC * Nh * 4 + Th * HC * 8,
                lambda: B.call('camx_pf_hc_post_rms', _p(bh), _p(injh), _p(resh), _p(wh), NULL, _p(xnbf), _p(sclh), I(Th), I(HC), F(0.25), F(1e-6), I(Nh))))
    out.append(('hc_mean_2048x4x2560_from_residual', Th * HC * Nh * 8 + Th * Nh * 4 + HC * Nh * 4 + Th * HC * 4,
                lambda: B.call('camx_pf_hc_mean', _p(resh), _p(sclh), _p(wh), _p(gh), _p(outh), I(Th), I(HC), I(Nh), F(0.25))))
    out.append(('_keep', 0, [x, d, nw, h, h16, q8, qkv, par, q16, cache, g, u, y16, toks, qg, w4, pos, o4, a4, xc, wc, st, yc, l2o, x5, d5, h5, h516, qkv5,
                             cache5, err5, pos5d, ptd, q165, bh, injh, resh, wh, xnbf, sclh, gh, outh]))
    return out


def prefill_scale_sweep(B, T=4096, only=None):
    """every entry point at a prefill-scale size (bench.py --only sweep [--sweep-tokens T]): name -> {us, bytes, GBps, frac_of_8TBps}. Each
    is launched 30 times back to back over enough copies of its buffers, in rotation, that the rotation's footprint is at least 1.2 GB
    (no launch finds its own lines in the 256 MB Infinity Cache); bytes are algorithmic (inputs read once, outputs written once)."""
    import numpy as np
    torch = B.torch; dev = B.dev
    res = {}

    def timeit(name, by, mk, reps=30):
        if only and not any(o in name for o in only.split(',')): return
        ncopy = max(3, min(16, -(-1_200_000_000 // int(by))))
        fns = [mk(i) for i in range(ncopy)]
        for f in fns: f()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for k in range(reps): fns[k % len(fns)]()
        b.record(); b.synchronize()
        us = a.elapsed_time(b) * 1e3 / reps
        res[name] = {'us': round(us, 2), 'bytes': int(by), 'copies': ncopy, 'GBps': round(by / us / 1e3, 1), 'frac_of_8TBps': round(by / us / 1e3 / HBM_PEAK_GBPS, 4)}
        del fns
        torch.cuda.empty_cache()

    N = 2048
    def mk(i):
        x = B.acts((T, N), torch.float32, i); d = B.acts((T, 1, N), torch.float32, i + 10); nw = B.gamma(N, 3); h = torch.empty((T, N), device=dev); h16 = torch.empty((T, N), dtype=torch.float16, device=dev)
        return lambda: B.call('camx_q3p_add_rms16', _p(x), _p(d), NULL, I(1), _p(nw), F(1e-6), _p(h), _p(h16), I(N), I(T))
    timeit(f'q3p_add_rms16 {T}x2048 S=1', T * N * (4 + 4 + 4 + 4 + 2), mk)
    def mk(i):
        x = B.acts((T, N), torch.float32, i); d = B.acts((T, 8, N), torch.float32, i + 10); w = torch.rand((T, 8), device=dev); nw = B.gamma(N, 3); h16 = torch.empty((T, N), dtype=torch.float16, device=dev)
        return lambda: B.call('camx_q3p_add_rms16', _p(x), _p(d), _p(w), I(8), _p(nw), F(1e-6), NULL, _p(h16), I(N), I(T))
    timeit(f'q3p_add_rms16 {T}x2048 S=8 weighted', T * N * (4 + 32 + 4 + 2), mk)
    def mk(i):
        x = B.acts((T, N), torch.float32, i); d = B.acts((T, 1, N), torch.float32, i + 10); nw = B.gamma(N, 3); q8 = torch.empty(T * N // 32 * 36, dtype=torch.uint8, device=dev)
        return lambda: B.call('camx_add_rms_q8_1', _p(x), _p(d), NULL, I(1), _p(nw), F(1e-6), NULL, NULL, _p(q8), I(N), I(T))
    timeit(f'add_rms_q8_1 {T}x2048', T * N * (4 + 4 + 4 + 1.125), mk)
    H = 5120
    def mk(i):
        x = B.acts((T, H), torch.float32, i); d = B.acts((T, H), torch.float32, i + 10); nw = B.gamma(H, 3); h = torch.empty((T, H), device=dev); h16 = torch.empty((T, H), dtype=torch.float16, device=dev)
        return lambda: B.call('camx_q35p_add_rms16', _p(x), _p(d), _p(nw), F(1e-6), _p(h), _p(h16), I(H), I(T))
    timeit(f'q35p_add_rms16 {T}x5120', T * H * (4 + 4 + 4 + 4 + 2), mk)
    def mk(i):
        x = B.acts((2048 * 4, 2560), torch.float32, i); w = B.gamma(4 * 2560, 3); ybf = torch.empty((8192, 2560), dtype=torch.bfloat16, device=dev); scl = torch.empty(8192, device=dev)
        return lambda: B.call('camx_pf_rms_mul', _p(x), _p(w), NULL, _p(ybf), _p(scl), I(8192), I(4), F(1e-6), I(2560))
    timeit('pf_rms_mul 8192x2560 -> bf16', 8192 * 2560 * 6, mk)
    n = T * 8 * 768
    def mk(i):
        g = B.acts((n,), torch.float32, i); u = B.acts((n,), torch.float32, i + 5); y = torch.empty(n, dtype=torch.float16, device=dev)
        return lambda: B.call('camx_q3p_swiglu', _p(g), _p(u), _p(y), I(n))
    timeit(f'q3p_swiglu {T}x6144', n * 10, mk)
    def mk(i):
        gu = B.acts((T, 2 * 17408), torch.bfloat16, i); act = torch.empty((T, 17408), dtype=torch.bfloat16, device=dev)
        return lambda: B.call('camx_silu_mul_bf16', _p(gu), _p(act), I(17408), L64(T * 17408))
    timeit(f'silu_mul_bf16 {T}x17408', T * 17408 * 6, mk)
    def mk(i):
        x = B.acts((n,), torch.float32, i); y = torch.empty(n // 32 * 36, dtype=torch.uint8, device=dev)
        return lambda: B.call('camx_gg_quantize_q8_1', _p(x), _p(y), L64(n), I(0), F(0), NULL)
    timeit(f'gg_quantize_q8_1 {T}x6144', n * 5.125, mk)
    K = 6144
    def mk(i):
        x = B.acts((T, K), torch.float32, i); y = torch.empty(K // 128 * T * 144, dtype=torch.uint8, device=dev)
        return lambda: B.call('camx_quantize_mmq_q8_1', _p(x), NULL, _p(y), L64(K), L64(K), L64(0), L64(0), L64(K), I(T), I(1), I(0), I(1))
    timeit(f'quantize_mmq_q8_1 {T}x6144 DS4', T * K * 5.125, mk)
    nh, nkv = 32, 4; ldq = (nh + 2 * nkv) * 128
    par, _ = yarn_par(torch, dev, 15, yarn=False)
    def mk(i):
        qkv = B.acts((T, ldq), torch.float32, i); q16 = torch.empty((T, nh, 128), dtype=torch.float16, device=dev); cache = torch.empty((T, 2 * nkv * 128), dtype=torch.float16, device=dev)
        return lambda: B.call('camx_q3p_qk_rope', _p(qkv), I(ldq), I(nh), I(nkv), _p(par), I(0), _p(q16), _p(cache), I(T), I(0))
    timeit(f'q3p_qk_rope {T} tok f32 -> f16', T * ldq * 6, mk)
    rbq = 2 * (nkv * 128 // 32) * 34
    def mk(i):
        qkv = B.acts((T, ldq), torch.float32, i); q16 = torch.empty((T, nh, 128), dtype=torch.float16, device=dev); cache = torch.empty(T * rbq, dtype=torch.uint8, device=dev); err = torch.zeros(1, dtype=torch.int32, device=dev)
        return lambda: B.call('camx_q3p_qk_rope_q8', _p(qkv), I(ldq), I(nh), I(nkv), _p(par), I(0), _p(q16), _p(cache), _p(err), I(T), I(0))
    timeit(f'q3p_qk_rope_q8 {T} tok', T * (ldq * 4 + nh * 256 + rbq), mk)
    D = 256
    def mk(i):
        qg = B.acts((T * 24, 2 * D), torch.bfloat16, i); w4 = B.gamma(D, 2); o = torch.empty((T * 24, D), dtype=torch.bfloat16, device=dev)
        return lambda: B.call('camx_pf_qk_nr', _p(qg), I(2 * D), I(24), _p(w4), I(D), I(64), F(0.6), F(1e-6), I(0), _p(o), I(T), I(1))
    timeit(f'pf_qk_nr {T}x24x256 bf16', T * 24 * D * 4, mk)
    def mk(i):
        a = B.acts((T * 24, D), torch.bfloat16, i); qg = B.acts((T * 24, 2 * D), torch.bfloat16, i + 3); o = torch.empty((T * 24, D), dtype=torch.bfloat16, device=dev)
        return lambda: B.call('camx_gate_mul', _p(a), _p(qg), _p(o), L64(T * 24 * D), I(D), I(2 * D), I(D), I(2))
    timeit(f'gate_mul {T}x24x256 bf16', T * 24 * D * 6, mk)
    Cc = 10240
    def mk(i):
        xc = B.acts((T, Cc), torch.bfloat16, i); wc = B.acts((Cc, 4), torch.float32, 45, frac=0); st = B.acts((Cc, 3), torch.float32, 46, frac=0); yc = torch.empty((T, Cc), dtype=torch.bfloat16, device=dev)
        return lambda: B.call('camx_pf_gdn_conv', _p(xc), _p(wc), _p(st), _p(yc), I(Cc), I(T), I(Cc), I(Cc), I(1))
    timeit(f'pf_gdn_conv {T}x10240 bf16', T * Cc * 4, mk)
    def mk(i):
        xc = B.acts((T, Cc), torch.bfloat16, i); o = torch.empty((T * 32, 128), dtype=torch.bfloat16, device=dev)
        return lambda: B.call('camx_pf_gdn_l2', _p(xc), _p(o), I(32), I(128), I(Cc), F(1e-6 / 128), I(T), I(1))
    timeit(f'pf_gdn_l2 {T}x32x128 bf16', T * 32 * 128 * 4, mk)
    M = 512
    def mk(i):
        k = B.acts((T, M), torch.float32, i); v = B.acts((T, M), torch.float32, i + 2); cache = torch.empty(T * 1088, dtype=torch.uint8, device=dev); err = torch.zeros(1, dtype=torch.int32, device=dev)
        return lambda: B.call('camx_own_kv_q8_append', _p(k), I(M), _p(v), I(M), I(M), _p(cache), I(0), I(T), _p(err), I(T))
    timeit(f'own_kv_q8_append {T}x512', T * (M * 8 + 1088), mk)
    TD = 65536              # the codec at depth: the rows of a long context (the reader is what a decode step walks: kernels/k3_own_atts.h:297-467)
    def mk(i):
        k = B.acts((TD, M), torch.float32, i); v = B.acts((TD, M), torch.float32, i + 2); cache = torch.empty(TD * 1088, dtype=torch.uint8, device=dev); err = torch.zeros(1, dtype=torch.int32, device=dev)
        return lambda: B.call('camx_own_kv_q8_append', _p(k), I(M), _p(v), I(M), I(M), _p(cache), I(0), I(TD), _p(err), I(TD))
    timeit('own_kv_q8_append 65536x512 (at depth)', TD * (M * 8 + 1088), mk)
    def mk(i):
        x = B.acts((T * 36, 128), torch.float32, i); y = torch.empty_like(x)
        return lambda: B.call('camx_hadamard128', _p(x), _p(y), L64(T * 36))
    timeit(f'hadamard128 {T}x36 heads', T * 36 * 128 * 8, mk)
    V = 151936
    tab = torch.randint(0, 256, (V, 1152), device=dev, dtype=torch.uint8)
    tab.view(V, 8, 144)[:, :, :4] = (torch.rand((V, 8, 2), device=dev) * 9e-3 + 1e-3).to(torch.float16).view(torch.uint8).view(V, 8, 4)
    def mk(i):
        toks = torch.randint(0, V, (T,), device=dev, dtype=torch.int32); x = torch.empty((T, N), device=dev)
        return lambda: B.call('camx_q3p_emb', _p(tab), I(1152), I(V), _p(toks), _p(x), I(N), I(T))
    timeit(f'q3p_emb {T} rows Q4_K -> f32', T * (1152 + N * 4), mk)
    Kq = 2048; Mr = 8192
    def mk(i):
        x = B.acts((Mr, Kq), torch.bfloat16, i); y = torch.empty((Mr, Kq), dtype=torch.bfloat16, device=dev); s = torch.empty(Mr, device=dev)
        return lambda: B.call('camx_actq_fwd', _p(x), I(1), _p(y), _p(s), NULL, I(Kq), F(1.0), I(7), I(Mr))
    timeit('actq_fwd bf16 8192x2048', Mr * Kq * 4, mk)
    def mk(i):
        x = B.acts((Mr, Kq), torch.bfloat16, i); g = B.acts((Mr, Kq), torch.bfloat16, i + 1); dx = torch.empty((Mr, Kq), dtype=torch.bfloat16, device=dev)
        return lambda: B.call('camx_actq_bwd', _p(x), I(1), _p(g), _p(dx), I(Kq), F(1.0), I(7), I(Mr))
    timeit('actq_bwd bf16 8192x2048', Mr * Kq * 6, mk)
    def mk(i):
        gu = B.acts((Mr, 2 * Kq), torch.bfloat16, i); y = torch.empty((Mr, Kq), dtype=torch.bfloat16, device=dev); s = torch.empty(Mr, device=dev); c = torch.empty((Mr, Kq // 2), dtype=torch.uint8, device=dev)
        return lambda: B.call('camx_silu_mul_actq_fwd', _p(gu), I(2 * Kq), I(Kq), _p(y), _p(s), _p(c), F(1.0), I(7), I(Mr))
    timeit('silu_mul_actq_fwd 8192x2048', Mr * Kq * 6.5, mk)
    def mk(i):
        gu = B.acts((Mr, 2 * Kq), torch.bfloat16, i); g = B.acts((Mr, Kq), torch.bfloat16, i + 1); d = torch.empty((Mr, 2 * Kq), dtype=torch.bfloat16, device=dev)
        return lambda: B.call('camx_silu_mul_actq_bwd', _p(gu), I(2 * Kq), I(Kq), _p(g), _p(d), F(1.0), I(7), I(Mr))
    timeit('silu_mul_actq_bwd 8192x2048', Mr * Kq * 10, mk)
    De = 1024; nab = 16
    nwe = torch.rand(De, device=dev) + 0.5; wab = (torch.randn(nab, De, device=dev) / 30).to(torch.bfloat16)
    def mk(i):
        x = B.acts((Mr, De), torch.float32, i); y = torch.empty((Mr, De), dtype=torch.bfloat16, device=dev); s = torch.empty(Mr, device=dev)
        c = torch.empty((Mr, De // 2), dtype=torch.uint8, device=dev); ab = torch.empty((Mr, nab), dtype=torch.bfloat16, device=dev); rstd = torch.empty(Mr, device=dev)
        return lambda: B.call('camx_block_entry_fwd', _p(x), _p(nwe), _p(wab), I(nab), F(1e-6), _p(y), _p(s), _p(c), _p(ab), _p(rstd), I(De), F(1.0), I(7), I(Mr))
    timeit('block_entry_fwd 8192x1024, 16 projections', Mr * (De * 6.5 + nab * 2 + 8), mk)
    def mk(i):
        x = B.acts((Mr, De), torch.float32, i); dy = B.acts((Mr, De), torch.bfloat16, i + 1); dab = B.acts((Mr, nab), torch.bfloat16, i + 2)
        rstd = torch.rand(Mr, device=dev) + 0.5; dx = torch.empty((Mr, De), device=dev)
        return lambda: B.call('camx_block_entry_bwd', _p(x), _p(nwe), _p(rstd), _p(wab), I(nab), _p(dy), _p(dab), _p(dx), I(De), F(1.0), I(7), I(Mr))
    timeit('block_entry_bwd 8192x1024, 16 projections', Mr * (De * 10 + nab * 2 + 4), mk)
    def mk(i):
        x = B.acts((Mr * Kq,), torch.float32, i); m = B.acts((Mr * Kq,), torch.bfloat16, i + 1); y = B.acts((Mr * Kq,), torch.bfloat16, i + 2); o = torch.empty(Mr * Kq, device=dev)
        return lambda: B.call('camx_residual3', _p(x), _p(m), _p(y), _p(o), L64(Mr * Kq))
    timeit('residual3 16M', Mr * Kq * 12, mk)
    nys = 1024
    ys = B.acts((nys, Kq), torch.bfloat16, 77); pos = torch.full((Mr,), -1, dtype=torch.int32, device=dev); pos[::Mr // nys] = torch.arange(nys, dtype=torch.int32, device=dev)
    def mk(i):
        x = B.acts((Mr, Kq), torch.float32, i); m = B.acts((Mr, Kq), torch.bfloat16, i + 1); mlp = B.acts((Mr, Kq), torch.bfloat16, i + 2); o = torch.empty((Mr, Kq), device=dev)
        return lambda: B.call('camx_residual_slices_fwd', _p(x), _p(m), _p(mlp), _p(ys), _p(pos), _p(o), I(Kq), L64(Mr * Kq // 4))
    timeit('residual_slices_fwd 8192x2048, 1024 slices', Mr * Kq * 12 + nys * Kq * 2, mk)
    def mk(i):
        do = B.acts((Mr, Kq), torch.float32, i); dm = torch.empty((Mr, Kq), dtype=torch.bfloat16, device=dev); dmlp = torch.empty_like(dm); dys = torch.empty((nys, Kq), dtype=torch.bfloat16, device=dev)
        return lambda: B.call('camx_residual_slices_bwd', _p(do), _p(pos), _p(dm), _p(dmlp), _p(dys), I(Kq), L64(Mr * Kq // 4))
    timeit('residual_slices_bwd 8192x2048, 1024 slices', Mr * Kq * 8 + nys * Kq * 2, mk)
    wn = B.gamma(Kq, 9)
    def mk(i):
        x = B.acts((Mr, Kq), torch.float32, i); o = torch.empty((Mr, Kq), device=dev)
        return lambda: B.call('camx_rmsnorm_f32', _p(x), _p(wn), _p(o), I(Kq), F(1e-6), I(Mr))
    timeit('rmsnorm_f32 8192x2048', Mr * Kq * 8, mk)
    def mk(i):
        x = B.acts((Mr * Kq,), torch.float32, i); o = torch.empty(Mr * Kq, dtype=torch.bfloat16, device=dev)
        return lambda: B.call('camx_cast_bf16', _p(x), _p(o), L64(Mr * Kq))
    timeit('cast_bf16 16M', Mr * Kq * 6, mk)
    ntk, Ks, neu = T, 2048, 8
    def mk(i):
        x = B.acts((ntk, Ks), torch.float32, i); vy = torch.empty((Ks // 128) * ntk * neu * 144, dtype=torch.uint8, device=dev)
        # the compact columns as the router's sort produces them (python/caminus/prefill/glue.py: columns grouped by expert, a group's tokens in
        # order): 128 experts, each token's 8 by the top of random scores
        g = torch.Generator(device=dev); g.manual_seed(900 + i)
        ex = torch.rand((ntk, 128), generator=g, device=dev).topk(neu, dim=1).indices.reshape(-1)
        order = torch.argsort(ex, stable=True); ids = torch.empty(ntk * neu, dtype=torch.int32, device=dev); ids[order] = torch.arange(ntk * neu, dtype=torch.int32, device=dev)
        return lambda: B.call('camx_quantize_mmq_q8_1_scatter', _p(x), _p(ids), _p(vy), L64(Ks), L64(0), L64(Ks), L64(0), L64(Ks), I(ntk * neu), I(1), I(neu), I(1), I(ntk))
    timeit(f'quantize_mmq_q8_1_scatter {T}x2048 to 8 columns each', ntk * Ks * 4 + (Ks // 128) * ntk * neu * 144, mk)
    def mk(i):
        k = B.acts((T, 512), torch.float32, i); v = B.acts((T, 512), torch.float32, i + 2); cache = torch.empty(T * 1088, dtype=torch.uint8, device=dev); err = torch.zeros(1, dtype=torch.int32, device=dev)
        return lambda: B.call('camx_pf_kv_append', _p(k), I(512), _p(v), I(512), I(512), _p(cache), I(0), I(T), _p(err), I(T))
    timeit(f'pf_kv_append {T}x512', T * (512 * 8 + 1088), mk)
    def mk(i):
        x = B.acts((T * 36, 128), torch.float32, i)
        return lambda: B.call('camx_pf_hadamard', _p(x), I(T * 36), I(128), I(4))
    timeit(f'pf_hadamard {T}x36 chunks of 128', T * 36 * 128 * 8, mk)
    rows_n = T * 32
    wg128 = B.gamma(128, 6)
    def mk(i):
        o = B.acts((rows_n, 128), torch.float32, i); z = B.acts((rows_n, 128), torch.float32, i + 1, frac=0); y = torch.empty((rows_n, 128), device=dev)
        return lambda: B.call('camx_pf_gdn_norm', _p(o), _p(wg128), _p(z), _p(y), I(128), F(1e-6), C.c_long(rows_n), I(1))
    timeit(f'pf_gdn_norm {T}x32x128 silu', rows_n * 128 * 12, mk)
    def mk(i):
        k = B.acts((T, 1024), torch.float32, i); v = B.acts((T, 1024), torch.float32, i + 1); cache = torch.empty((T, 2048), dtype=torch.float16, device=dev); err = torch.zeros(1, dtype=torch.int32, device=dev)
        return lambda: B.call('camx_q35p_kv_append16', _p(k), I(1024), _p(v), I(1024), _p(cache), I(1024), I(0), I(T), _p(err), I(T))
    timeit(f'q35p_kv_append16 {T}x1024', T * 1024 * 12, mk)
    def mk(i):
        b = B.acts((2048, 2560), torch.float32, i); inj = B.acts((2048, 4), torch.float32, i + 1, frac=0); r = B.acts((2048, 4, 2560), torch.float32, i + 2)
        return lambda: B.call('camx_pf_hc_post', _p(b), _p(inj), _p(r), I(2048), I(4), I(2560), F(1.0))
    timeit('pf_hc_post 2048x4x2560', 2048 * 2560 * 36, mk)
    def mk(i):
        g = B.acts((Mr * Kq,), torch.float32, i, frac=0); u = B.acts((Mr * Kq,), torch.float32, i + 1); h = torch.empty(Mr * Kq, device=dev)
        return lambda: B.call('camx_gg_silu_mul', _p(g), _p(u), _p(h), I(Mr * Kq))
    timeit('gg_silu_mul 16M', Mr * Kq * 12, mk)
    Cp, Dp = 1024, 256
    wpc = (torch.randn(Cp, 4, device=dev) * 0.5).to(torch.float16); hist = torch.randn(Cp, 6, device=dev)
    def mk(i):
        x = B.acts((T, Cp), torch.float32, i, frac=0); y = torch.empty((T, Cp), device=dev)
        return lambda: B.call('camx_pf_ple_conv', _p(x), NULL, NULL, _p(wpc), _p(hist), _p(y), NULL, NULL, I(Cp), I(T), I(Dp), I(2))
    timeit(f'pf_ple_conv {T}x1024, dilation 2', T * Cp * 8, mk)
    def mk(i):
        kn = B.acts((T, 4, Dp), torch.float32, i, frac=0); q = B.acts((T, 4, Dp), torch.float32, i + 1, frac=0); val = B.acts((T, Dp), torch.float32, i + 2, frac=0)
        gated = torch.empty((T, 4, Dp), device=dev); gate = torch.empty((T, 4), device=dev)
        return lambda: B.call('camx_pf_ple_gate', _p(kn), _p(q), NULL, NULL, _p(val), I(Dp), _p(gated), _p(gate), I(4), I(Dp), I(T))
    timeit(f'pf_ple_gate {T}x4x256', T * 4 * Dp * 12 + T * Dp * 4, mk)
    rows_g, Kg = T * 48, 128
    def mk(i):
        o = B.acts((rows_g, Kg), torch.float32, i); z = B.acts((rows_g, Kg), torch.float32, i + 1, frac=0); wg = B.gamma(Kg, 5); y16 = torch.empty((rows_g, Kg), dtype=torch.float16, device=dev)
        return lambda: B.call('camx_q35p_gdn_norm16', _p(o), _p(wg), _p(z), _p(y16), I(Kg), F(1e-6), C.c_long(rows_g))
    timeit(f'q35p_gdn_norm16 {T}x48x128', rows_g * Kg * 10, mk)
    Dh = 2560
    def mk(i):
        r = B.acts((2048, 4, Dh), torch.float32, i); y = torch.empty((2048, Dh), device=dev)
        return lambda: B.call('camx_pf_hc_avg', _p(r), _p(y), I(2048), I(4), I(Dh), I(Dh))
    timeit('pf_hc_avg 2048x4x2560', 2048 * Dh * 20, mk)
    def mk(i):
        a = B.acts((Mr * Kq,), torch.float32, i); b = B.acts((Mr * Kq,), torch.float32, i + 1); y = B.acts((Mr * Kq,), torch.float32, i + 2)
        return lambda: B.call('camx_pf_add_sum', _p(a), _p(b), _p(y), L64(Mr * Kq))
    timeit('pf_add_sum 16M', Mr * Kq * 16, mk)
    def mk(i):
        x = B.acts((Mr * Kq,), torch.float32, i); y = torch.empty(Mr * Kq, dtype=torch.float16, device=dev)
        return lambda: B.call('camx_op_own_f16', _p(x), _p(y), I(Mr * Kq))
    timeit('op_own_f16 16M', Mr * Kq * 6, mk)
    def mk(i):
        n = T * 2048; d = B.acts((8, n), torch.float32, i); wv = B.acts((8,), torch.float32, i + 1); x = B.acts((n,), torch.float32, i + 2)
        return lambda: B.call('camx_op_own_moe_sum', _p(d), _p(wv), _p(x), I(n), I(8))
    timeit(f'op_own_moe_sum {T}x2048, 8 slots', T * 2048 * 40, mk)
    def mk(i):
        n = T * 2048; moe = B.acts((n,), torch.float32, i); sh = B.acts((n,), torch.float32, i + 1); lg = B.acts((T,), torch.float32, i + 2); o = torch.empty(n, device=dev)
        return lambda: B.call('camx_op_shexp_add', _p(moe), _p(sh), _p(lg), _p(o), I(n), I(T))
    timeit(f'op_shexp_add {T}x2048', T * 2048 * 12, mk)
    def mk(i):
        x = B.acts((4096, 5120), torch.float32, i); y = torch.empty((4096, 5120), dtype=torch.bfloat16, device=dev)
        return lambda: B.call('camx_pf_to_bf16', _p(x), I(5120), _p(y), I(4096), I(4096), I(5120))
    timeit('pf_to_bf16 4096x5120', 4096 * 5120 * 6, mk)
    def mk(i):
        cache = torch.randint(0, 256, (T * 1088,), device=dev, dtype=torch.uint8)
        cache.view(T * 32, 34)[:, :2] = (torch.rand((T * 32, 1), device=dev) * 9e-3 + 1e-3).to(torch.float16).view(torch.uint8).view(T * 32, 2)
        k = torch.empty((T, M), dtype=torch.float16, device=dev); v = torch.empty((T, M), dtype=torch.float16, device=dev); err = torch.zeros(1, dtype=torch.int32, device=dev)
        return lambda: B.call('camx_own_kv_q8_read', _p(cache), NULL, I(0), I(T), I(M), _p(k), I(M), _p(v), I(M), _p(err), I(T), I(1))
    timeit(f'own_kv_q8_read {T}x512 -> f16', T * (1088 + M * 4), mk)
    def mk(i):
        cache = torch.randint(0, 256, (TD * 1088,), device=dev, dtype=torch.uint8)
        cache.view(TD * 32, 34)[:, :2] = (torch.rand((TD * 32, 1), device=dev) * 9e-3 + 1e-3).to(torch.float16).view(torch.uint8).view(TD * 32, 2)
        k = torch.empty((TD, M), dtype=torch.float16, device=dev); v = torch.empty((TD, M), dtype=torch.float16, device=dev); err = torch.zeros(1, dtype=torch.int32, device=dev)
        return lambda: B.call('camx_own_kv_q8_read', _p(cache), NULL, I(0), I(TD), I(M), _p(k), I(M), _p(v), I(M), _p(err), I(TD), I(1))
    timeit('own_kv_q8_read 65536x512 -> f16 (at depth)', TD * (1088 + M * 4), mk)
    page, n_pages = 256, max(64, T // 64)
    def mk(i):
        qkv = B.acts((T, ldq), torch.float32, i); q16 = torch.empty((T, nh, 128), dtype=torch.float16, device=dev)
        cache = torch.empty(n_pages * page * rbq, dtype=torch.uint8, device=dev); err = torch.zeros(1, dtype=torch.int32, device=dev)
        perm = torch.randperm(n_pages * page, device=dev)[:T].to(torch.int32)            # every sequence at its own row: page = row / 256 through a one-column table
        pos = (perm % page).contiguous(); pt = (perm // page).reshape(T, 1).contiguous()
        return lambda: B.call('camx_qk_rope_paged', _p(qkv), I(ldq), I(nh), I(nkv), _p(par), _p(pos), _p(q16), _p(cache), _p(err), _p(pt), I(1), I(page), I(n_pages), I(T), I(0), I(1))
    timeit(f'qk_rope_paged {T} seq Q8', T * (ldq * 4 + 8 + nh * 256 + rbq), mk)
    Th, HC, Nh = max(T // 2, 64), 4, 2560
    def mk(i):
        bh = B.acts((Th, Nh), torch.float32, i); injh = B.acts((Th, HC), torch.float32, i + 1, frac=0); resh = B.acts((Th, HC, Nh), torch.float32, i + 2)
        wh = B.gamma(HC * Nh, 64); xnbf = torch.empty((Th, HC, Nh), dtype=torch.bfloat16, device=dev); sclh = torch.empty(Th * HC, device=dev)
        return lambda: B.call('camx_pf_hc_post_rms', _p(bh), _p(injh), _p(resh), _p(wh), NULL, _p(xnbf), _p(sclh), I(Th), I(HC), F(0.25), F(1e-6), I(Nh))
    timeit(f'pf_hc_post_rms {Th}x4x2560 -> bf16 + scale', Th * Nh * 4 + Th * HC * Nh * 10 + HC * Nh * 4 + Th * HC * 8, mk)
    return res


def batch_ladder(B, tokens=(16, 64, 256, 512, 1024, 2048, 4096), only=None):
    """the op-sets of the configs from a verify batch to a prefill chunk (bench.py --only ladder): us per launch and GB/s at 16 .. 4096
    tokens, 30 launches back to back over copies in rotation (footprint >= 1.2 GB or 16 copies: the small batches stay cache-resident, as
    they are in a decode loop). The launchers switch kernels with the batch size; this shows the switches as a curve."""
    torch = B.torch; dev = B.dev
    out = {}
    nh, nkv = 32, 4; ldq = (nh + 2 * nkv) * 128; rbq = 2 * (nkv * 128 // 32) * 34; N = 2048
    par, _ = yarn_par(torch, dev, 15, yarn=False)
    parb, _ = yarn_par(torch, dev, 16)
    nw = B.gamma(N, 3); nw5 = B.gamma(5120, 4)
    V = 151936
    tab = torch.randint(0, 256, (V, 1152), device=dev, dtype=torch.uint8)
    tab.view(V, 8, 144)[:, :, :4] = (torch.rand((V, 8, 2), device=dev) * 9e-3 + 1e-3).to(torch.float16).view(torch.uint8).view(V, 8, 4)

    def ops(T):
        def add_rms16(i):
            x = B.acts((T, N), torch.float32, i); d = B.acts((T, 1, N), torch.float32, i + 10); h = torch.empty((T, N), device=dev); h16 = torch.empty((T, N), dtype=torch.float16, device=dev)
            return lambda: B.call('camx_q3p_add_rms16', _p(x), _p(d), NULL, I(1), _p(nw), F(1e-6), _p(h), _p(h16), I(N), I(T))
        def add_rms_q8(i):
            x = B.acts((T, N), torch.float32, i); d = B.acts((T, 1, N), torch.float32, i + 10); q8 = torch.empty(T * N // 32 * 36, dtype=torch.uint8, device=dev)
            return lambda: B.call('camx_add_rms_q8_1', _p(x), _p(d), NULL, I(1), _p(nw), F(1e-6), NULL, NULL, _p(q8), I(N), I(T))
        def gather_norm(i):
            toks = torch.randint(0, V, (T,), device=dev, dtype=torch.int32); x = torch.empty((T, N), device=dev); qq = torch.empty(T * (N // 32) * 36, dtype=torch.uint8, device=dev)
            return lambda: B.call('camx_emb_gather_add_rms', _p(tab), L64(1152), I(V), _p(toks), _p(x), NULL, NULL, _p(nw), F(1e-6), NULL, NULL, _p(qq), I(N), I(T), I(0))
        def rope_f32(i):
            qkv = B.acts((T, ldq), torch.float32, i); q16 = torch.empty((T, nh, 128), dtype=torch.float16, device=dev); cache = torch.empty((T, 2 * nkv * 128), dtype=torch.float16, device=dev)
            return lambda: B.call('camx_q3p_qk_rope', _p(qkv), I(ldq), I(nh), I(nkv), _p(par), I(0), _p(q16), _p(cache), I(T), I(0))
        def rope_q8(i):
            qkv = B.acts((T, ldq), torch.float32, i); q16 = torch.empty((T, nh, 128), dtype=torch.float16, device=dev); cache = torch.empty(T * rbq, dtype=torch.uint8, device=dev); err = torch.zeros(1, dtype=torch.int32, device=dev)
            return lambda: B.call('camx_q3p_qk_rope_q8', _p(qkv), I(ldq), I(nh), I(nkv), _p(par), I(0), _p(q16), _p(cache), _p(err), I(T), I(0))
        def add_rms_bf16(i):
            x = B.acts((T, 5120), torch.float32, i); d = B.acts((T, 5120), torch.bfloat16, i + 1); hb = torch.empty((T, 5120), dtype=torch.bfloat16, device=dev)
            return lambda: B.call('camx_add_rms_bf16', _p(x), _p(d), _p(nw5), F(1e-6), NULL, _p(hb), I(5120), I(T))
        def rope_bf16(i):
            l = 80 * 128; qkv = B.acts((T, l), torch.bfloat16, i); q16 = torch.empty((T, 64, 128), dtype=torch.float16, device=dev); cache = torch.empty((T, 2048), dtype=torch.float16, device=dev)
            return lambda: B.call('camx_qk_rope_bf16', _p(qkv), I(l), I(64), I(8), _p(parb), I(0), _p(q16), _p(cache), I(T), I(1))
        def swiglu_mmq(i):
            Fh = 17408; gu = B.acts((T, 2 * Fh), torch.bfloat16, i); y = torch.empty((Fh // 128, T, 144), dtype=torch.uint8, device=dev)
            return lambda: B.call('camx_swiglu_mmq_q8_1', _p(gu), L64(2 * Fh), L64(Fh), _p(y), NULL, I(T), I(1))
        return {'q3p_add_rms16 x2048': (T * N * 18, add_rms16), 'add_rms_q8_1 x2048': (T * N * 13.125, add_rms_q8), 'gather Q4_K + norm + q8_1': (T * (1152 + N * 5.125), gather_norm),
                'q3p_qk_rope f32 40 heads': (T * ldq * 6, rope_f32), 'q3p_qk_rope_q8 40 heads': (T * (ldq * 4 + nh * 256 + rbq), rope_q8),
                'add_rms_bf16 x5120': (T * 5120 * 12, add_rms_bf16), 'qk_rope_bf16 80 heads': (T * 80 * 128 * 4, rope_bf16), 'swiglu_mmq_q8_1 x17408': (T * 17408 * 5.125, swiglu_mmq)}

    for T in tokens:
        for name, (by, mk) in ops(T).items():
            if only and not any(f in name for f in only.split(',')): continue
            ncopy = max(3, min(16, -(-1_200_000_000 // int(by))))
            fns = [mk(i) for i in range(ncopy)]
            for f in fns: f()
            torch.cuda.synchronize()
            loops = []                                       # five loops of 30 launches: the median loop's average (the first loop after the buffers are made can run slow)
            for _ in range(5):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                for k in range(30): fns[k % ncopy]()
                b.record(); b.synchronize()
                loops.append(a.elapsed_time(b) * 1e3 / 30)
            us = sorted(loops)[2]
            out.setdefault(name, {})[str(T)] = {'us': round(us, 2), 'GBps': round(by / us / 1e3, 1), 'us_loops': [round(x, 2) for x in loops]}
            del fns
        torch.cuda.empty_cache()
    return out


def cpu_baseline(w, budget_s=15.0):
    """the CPU oracle (kind "port": oracle/camx_oracle.c, OpenMP over rows) on the whole batch of the same three op-sets: built here,
    on the host that runs it, with -O3 -march=native (the tests' build is -O2), median of at least five passes (more while the
    budget lasts); GB/s by the same byte accounting. One thread: the first 256 tokens, median of three."""
    import numpy as np
    import tempfile
    import oracle as O
    from oracle import build as orc_build
    flags = 'gcc -O2 -ffp-contract=off -fopenmp (prebuilt oracle/liborc.so: the -march=native build failed here)'
    try:
        so = orc_build.build_oracle(fast=True, out=os.path.join(tempfile.mkdtemp(prefix='camx_orc_'), 'liborc_fast.so'))
        O.use_library(so)
        flags = 'gcc -std=c11 -O3 -march=native -ffp-contract=off -fno-fast-math -fopenmp'
    except Exception:                                                  # noqa: BLE001 (no compiler on this host: the prebuilt library serves)
        pass
    import torch
    T, H, nh, nkv, Fh = w['T'], w['H'], w['nh'], w['nkv'], w['Fh']

    def bf_bits(t):
        return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)

    x = w['x'].cpu().numpy(); d = bf_bits(w['d']); nw = w['nw'].cpu().numpy()
    qkv = O.bf2f(bf_bits(w['qkv'])); gu = bf_bits(w['gu'])
    threads = int(os.environ.get('OMP_NUM_THREADS', '0')) or min(os.cpu_count() or 1, 16)
    by = sum(w['bytes'].values())

    def one_pass(n):
        t0 = time.perf_counter()
        O.add_rms_bf16(x[:n], d[:n], nw, 1e-6)
        O.qk_rope(qkv[:n], nh, nkv, w['par_np'], n, pos0=0, yarn=True, rows=n)
        act = O.silu_mul_bf16(gu[:n])
        O.mmq_q8_1(O.bf2f(act), Fh, n, 1)
        return time.perf_counter() - t0

    one_pass(T)                                                            # untimed: page the inputs in
    ts, t_start = [], time.perf_counter()
    while len(ts) < 5 or (time.perf_counter() - t_start < budget_s and len(ts) < 99):
        ts.append(one_pass(T))
    ts.sort(); med = ts[len(ts) // 2]
    T1 = min(T, 256)
    before = O.set_threads(1)
    t1 = sorted(one_pass(T1) for _ in range(3))[1]
    O.set_threads(before)
    return {'value': round(by / med / 1e9, 3), 'unit': 'GB/s', 'cores': threads, 'kind': 'port', 'build': flags,
            'value_1thread': round(by * T1 / T / t1 / 1e9, 3),
            'sample': f'all {T} tokens of the same three op-sets, median of {len(ts)} passes ({med * 1e3:.1f} ms; fastest {ts[0] * 1e3:.1f} ms) in '
                      f'{time.perf_counter() - t_start:.1f} s; one thread: first {T1} tokens, median of 3 ({t1 * 1e3:.1f} ms)'}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=50)
    ap.add_argument('--warmup', type=int, default=10)
    ap.add_argument('--copies', type=int, default=8, help='copies of the batch taken in rotation (8: no launch finds its lines in the Infinity Cache)')
    ap.add_argument('--sweep-tokens', type=int, default=4096, help='rows of the --only sweep shapes')
    ap.add_argument('--sweep-filter', default=None, help='--only sweep / ladder: entries whose name contains one of these comma-separated texts')
    ap.add_argument('--ladder-tokens', default='16,64,256,512,1024,2048,4096', help='--only ladder: the batch sizes')
    ap.add_argument('--no-ramp', action='store_true', help='skip the untimed clock ramp-up after the warm-up steps')
    ap.add_argument('--no-cpu', action='store_true')
    ap.add_argument('--no-extra', action='store_true')
    ap.add_argument('--only', default=None, help='run a single kernel of the step (for profiling)')
    a = ap.parse_args()
    if a.gpus != 1:
        print(f'bench.py: this build measures one GPU only (--gpus {a.gpus} is not supported): the row kernels shard by token with no '
              f'communication, so a multi-GPU figure would be N independent copies of this run', file=sys.stderr)
        sys.exit(2)
    B = Bench()
    torch = B.torch
    if a.only in ('sweep', 'ladder'): B.ramp()
    if a.only == 'sweep':
        print(json.dumps({'metric': 'fused-op HBM GB/s per entry point at prefill-scale sizes, 1 GPU', 'unit': 'GB/s', 'n_gpus': 1, 'data': 'synthetic',
                          'peak_GBps': HBM_PEAK_GBPS, 'tokens': a.sweep_tokens, 'sweep': prefill_scale_sweep(B, a.sweep_tokens, a.sweep_filter)}))
        return
    if a.only == 'ladder':
        print(json.dumps({'metric': 'us per launch and GB/s of the configs\' op-sets from 16 to 4096 tokens, 1 GPU', 'n_gpus': 1, 'data': 'synthetic', 'ladder': batch_ladder(B, tuple(int(t) for t in a.ladder_tokens.split(',')), a.sweep_filter)}))
        return
    if a.only == 'copy_ref':
        # a plain device copy of known size (256 MiB read + 256 MiB written per launch): the yardstick that FETCH_SIZE / WRITE_SIZE
        # counter readings of the kernels above are scaled by
        src = torch.ones(256 << 20, dtype=torch.uint8, device=B.dev); dst = torch.empty_like(src)
        med, mean = B.time_launch(lambda: dst.copy_(src), reps=a.steps, warm=a.warmup)
        print(json.dumps({'kernel': 'copy_ref', 'bytes_read': src.numel(), 'bytes_written': src.numel(), 'us': round(mean, 2),
                          'GBps': round(2 * src.numel() / (mean * 1e-6) / 1e9, 1)}))
        return
    if a.only == 'copy_sizes':
        # the runtime's own device copy (hipMemcpy device to device, through torch) at the sizes of the sweep's launches, timed like them (30
        # back to back over copies in rotation, footprint >= 1.2 GB): what a launch that moves S bytes can reach at all on this machine
        B.ramp()
        res = {}
        for mb in (6, 12, 24, 48, 55, 84, 126, 183, 256, 512):
            n = mb << 20
            nc = max(3, min(16, -(-1_200_000_000 // (2 * n))))
            src = [torch.ones(n, dtype=torch.uint8, device=B.dev) for _ in range(nc)]; dst = [torch.empty(n, dtype=torch.uint8, device=B.dev) for _ in range(nc)]
            for i in range(nc): dst[i].copy_(src[i])
            torch.cuda.synchronize()
            ts = []
            for rep in range(5):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for k in range(30): dst[k % nc].copy_(src[k % nc])
                e1.record(); e1.synchronize()
                ts.append(e0.elapsed_time(e1) * 1e3 / 30)
            ts.sort()
            res[f'{2 * n / 1e6:.1f} MB'] = {'us': round(ts[2], 2), 'GBps': round(2 * n / ts[2] / 1e3, 1), 'frac_of_8TBps': round(2 * n / ts[2] / 1e3 / HBM_PEAK_GBPS, 4)}
            # the library's own flat copy (camx_copy_cols_bf16 on whole rows: 16 bytes per thread, non-temporal both ways), timed the same way
            own = []
            for rep in range(5):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for k in range(30): B.call('camx_copy_cols_bf16', _p(src[k % nc]), I(4096), I(0), _p(dst[k % nc]), I(4096), I(0), I(4096), L64(n // 8192))
                e1.record(); e1.synchronize()
                own.append(e0.elapsed_time(e1) * 1e3 / 30)
            own.sort()
            res[f'{2 * n / 1e6:.1f} MB'].update({'own_copy_us': round(own[2], 2), 'own_copy_frac_of_8TBps': round(2 * n / own[2] / 1e3 / HBM_PEAK_GBPS, 4)})
            del src, dst; torch.cuda.empty_cache()
        print(json.dumps({'metric': 'device-to-device copy by the runtime and by the library, bytes read + written per launch', 'n_gpus': 1, 'copy_sizes': res}))
        return
    traffic = hbm_traffic()
    NC = a.copies
    ws = [config3(B, seed0=1003 + 10 * i) for i in range(NC)]            # independent copies of the batch, taken in rotation
    w = ws[0]
    names = list(w['launch']) if not a.only else [a.only]

    for k in range(max(a.warmup, NC)):
        for n in names: ws[k % NC]['launch'][n]()
    torch.cuda.synchronize()
    # more untimed steps until the GPU has been busy for a quarter of a second: after the host-side set-up the card starts at idle clocks,
    # and the first ~50 ms of work run up to 6 % slower (ten warm-up steps are 1.4 ms)
    ramp_steps = 0
    t_ramp = time.perf_counter()
    while not a.no_ramp and time.perf_counter() - t_ramp < 0.25:
        for k in range(50):
            for n in names: ws[k % NC]['launch'][n]()
        torch.cuda.synchronize()
        ramp_steps += 50
    # the timed region: exactly K steps on one stream, HIP events on that stream around the region; step k works on copy k % NC
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for k in range(a.steps):
        for n in names: ws[k % NC]['launch'][n]()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_step = e0.elapsed_time(e1) / a.steps
    total_bytes = sum(w['bytes'][n] for n in names)
    # the same loop on one copy of the batch: what a caller sees whose buffers were touched by the previous step
    s0, s1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s0.record()
    for k in range(a.steps):
        for n in names: w['launch'][n]()
    s1.record(); s1.synchronize()
    ms_same = s0.elapsed_time(s1) / a.steps
    # each kernel's average launch duration: K launches back to back between one pair of events (the median of five such loops), over the copies in rotation (eight
    # copies: the smallest per-kernel working set, 168 MB, times eight is five times the Infinity Cache). The figure includes the
    # dispatch gap between consecutive launches, as the step itself does.
    per = {}
    for n in names:
        for i in range(NC): ws[i]['launch'][n]()
        torch.cuda.synchronize()
        loops = []                                       # five loops of K launches: the median loop's average (a loop now and then runs 5 - 15 % slow)
        for rep in range(5):
            k0, k1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            k0.record()
            for k in range(a.steps): ws[k % NC]['launch'][n]()
            k1.record(); k1.synchronize()
            loops.append(k0.elapsed_time(k1) * 1e3 / a.steps)
        loops.sort()
        mean = loops[2]
        per[n] = {'us': round(mean, 2), 'us_loops_min_max': [round(loops[0], 2), round(loops[-1], 2)], 'bytes': w['bytes'][n], 'GBps': round(w['bytes'][n] / (mean * 1e-6) / 1e9, 1),
                  'frac_of_8TBps': round(w['bytes'][n] / (mean * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4), 'hbm_traffic_bytes': traffic.get(n)}
    dom = max(per, key=lambda n: per[n]['us'])
    achieved = per[dom]['bytes'] / (per[dom]['us'] * 1e-6) / 1e9
    out = {
        'metric': 'fused-op HBM GB/s (% of MI355X peak) + us per layer op-set, 1 GPU', 'value': round(total_bytes / (ms_step * 1e-3) / 1e9, 1), 'unit': 'GB/s',
        'n_gpus': 1, 'steps': a.steps, 'warmup': a.warmup, 'warmup_ramp_steps': ramp_steps, 'ms_per_step': round(ms_step, 4), 'higher_is_better': True, 'scaling': 'weak',
        'vs_baseline': None, 'dtype': 'f32', 'data': 'synthetic',
        'config': {'workload': 'dense 27B-class prefill chunk: 4096 tokens x hidden 5120, bf16 activations, fp32 residual and norms; op-sets add+RMSNorm, '
                               'QK-norm+YaRN rotary (64 Q + 8 KV heads x 128), SwiGLU 4096x17408 -> q8_1 MMQ (DS4)', 'tokens': 4096, 'hidden': 5120,
                   'kernels': names, 'batch_copies_in_rotation': NC},
        'frac_of_hbm_peak': round(total_bytes / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
        'wall_ms_per_step': round(wall * 1e3 / a.steps, 4),
        'same_batch': {'ms_per_step': round(ms_same, 4), 'GBps': round(total_bytes / (ms_same * 1e-3) / 1e9, 1),
                       'note': 'every step on one copy of the batch: part of each launch is served by the 256 MB Infinity Cache, so this is not an HBM figure'},
        'roofline': {'bound': 'hbm', 'kernel': dom, 'achieved': round(achieved, 1), 'peak': HBM_PEAK_GBPS, 'unit': 'GB/s',
                     'frac': round(achieved / HBM_PEAK_GBPS, 4), 'traffic': traffic.get(dom)},
        'kernels': per,
    }
    if not a.no_extra and not a.only:
        ops = {}
        sets = extra_opsets(B)
        for name, by, fn in sets:
            if name.startswith('_keep'): continue
            med, mean = B.time_launch(fn, reps=50, warm=10, flush=True)
            med_hot, _ = B.time_launch(fn, reps=50, warm=10, flush=False)
            q0, q1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            q0.record()
            for _ in range(50): fn()
            q1.record(); q1.synchronize()
            ops[name] = {'us': round(med, 2), 'us_cache_hot': round(med_hot, 2), 'us_queued': round(q0.elapsed_time(q1) * 1e3 / 50, 2), 'bytes': by, 'GBps': round(by / (med * 1e-6) / 1e9, 1),
                         'frac_of_8TBps': round(by / (med * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)}
        # the only per-op times the reference publishes for this path (another GPU: RX 7900 XTX, docs/specs/spec-prefill-cache.md:276)
        for k, ref_us in (('hc_post_rms_2048x4x2560_bf16_scale', 466.0), ('hc_mean_2048x4x2560_from_residual', 267.0)):
            if k in ops: ops[k]['reference_rx7900xtx_us'] = ref_us
        # a fused launch beside the launches it replaces
        for fused, parts in (('c4_conv4_silu_l2_one_launch', ('c4_conv4_silu', 'c4_l2norm_qk')),
                             ('c4_qk_nr_partial_rotary_q_and_k_one_launch', ('c4_qk_nr_partial_rotary_q', 'c4_qk_nr_partial_rotary_k')),
                             ('c4_dense_q8_qk_nr_hadamard_append_one_launch', ('c4_dense_q8_qk_nr_hadamard_append_six_launches',)),
                             ('c4_dense_q8_att_hadamard_gate_one_launch', ('c4_dense_q8_att_hadamard_gate_two_launches',)),
                             ('c1_qk_nr_kv_append_one_launch', ('c1_qk_nr_kv_append_three_launches',)),
                             ('c4_tape_gdn_gates_conv_l2_one_launch', ('c4_tape_gdn_gates_conv_l2_three_launches',))):
            if fused in ops:
                for key in ('us', 'us_cache_hot', 'us_queued'):
                    ops[fused][key + '_of_the_launches_it_replaces'] = round(sum(ops[p][key] for p in parts), 2)
        out['opsets'] = ops
        # the launch-bound op-sets as they would run in a decode loop: each shape's launches captured once into a HIP graph
        # and replayed (every entry point is stream-ordered, allocates nothing and keeps no host state per call)
        graphs = {}
        by_name = {name: fn for name, _, fn in sets}
        # config 4's row ops of one layer on the dense Q8 line (linear-attention conv + L2, full-attention QK-norm + rotary + Hadamard + Q8 append,
        # the gate), eight layers in one graph: as the separate launches of the reference's tape and as this library's fused launches
        layer_sep = ('c4_layer_separate_', ['c4_conv4_silu', 'c4_l2norm_qk', 'c4_dense_q8_qk_nr_hadamard_append_six_launches', 'c4_dense_q8_att_hadamard_gate_two_launches'], 10)
        layer_fused = ('c4_layer_fused_', ['c4_conv4_silu_l2_one_launch', 'c4_dense_q8_qk_nr_hadamard_append_one_launch', 'c4_dense_q8_att_hadamard_gate_one_launch'], 3)
        # config 1's row ops of one layer on the fp16-cache tape (python/caminus/engine/q3moe_one.py:362-377): add + norm, QK-norm + rotary of k -> append and
        # of q, add + norm, SwiGLU
        c1_sep = ('c1_layer_separate_', ['c1_add_rms_h_h16', 'c1_qk_nr_kv_append_three_launches', 'c1_add_rms_h_h16', 'c1_swiglu'], 6)
        c1_fused = ('c1_layer_fused_', ['c1_add_rms_h_h16', 'c1_qk_nr_kv_append_one_launch', 'c1_add_rms_h_h16', 'c1_swiglu'], 4)
        for prefix, rep in (('c1_', 1), ('c4_', 1), ('c5_', 1), ('c1_', 8), (layer_sep, 8), (layer_fused, 8), (c1_sep, 8), (c1_fused, 8)):      # (x 8: as many launches as a few layers of a decode step queue)
            if isinstance(prefix, tuple):
                prefix, names, per = prefix
                if not all(n in by_name for n in names): continue
                fns = [by_name[n] for n in names] * rep; nl = per * rep
            else:
                fns = [fn for name, _, fn in sets if name.startswith(prefix) and 'one_launch' not in name and 'launches' not in name and not name.endswith('_k')] * rep
                nl = len(fns)
            for fn in fns: fn()
            torch.cuda.synchronize()
            gr = torch.cuda.CUDAGraph()
            main_stream = B.stream
            with torch.cuda.graph(gr):
                B.stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)      # the capture stream
                for fn in fns: fn()
            B.stream = main_stream
            for _ in range(5): gr.replay()
            torch.cuda.synchronize()
            g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            g0.record()
            for _ in range(50): gr.replay()
            g1.record(); g1.synchronize()
            us = g0.elapsed_time(g1) * 1e3 / 50
            graphs[prefix + ('opsets_as_one_graph' if rep == 1 else f'opsets_x{rep}_as_one_graph')] = {'launches': nl, 'us_per_replay': round(us, 2), 'us_per_launch': round(us / nl, 2)}
        out['opset_graphs'] = graphs
    if not a.no_cpu and not a.only:
        out['cpu_baseline'] = cpu_baseline(w)
    print(json.dumps(out))


if __name__ == '__main__':
    main()
