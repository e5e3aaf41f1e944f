#!/usr/bin/env python3
"""Benchmark of the fused-op hot path on ONE MI355X.

A "step" is one forward + backward pass of the attention op over one batch of the workload
"GPT-2-medium-shaped causal attention": fp16, batch 8, seq 1024, 16 heads x 64, causal, dropout 0,
Q/K/V/dO ~ N(0,1) from seed 2013 (synthetic).  All tensors are resident in HBM before the timed
region; the kernels are called through the C ABI (libslapo_amd.so) with preallocated outputs.

value     attention fwd+bwd TFLOP/s = 14 * D * N / time per step, N = attended (query, key) pairs
roofline  the dK/dV backward kernel (the dominant kernel): its algorithmic FLOPs (8 * D * N: the
          four matrix products S, dP, dV, dK) over its own average launch duration, taken with HIP
          events placed around the DKDV stage of the backward on the launching stream, against the
          dense fp16 MFMA peak; "kernels" lists the same figure for the forward and dQ kernels
epilogue  GB/s of the two FusedMLP epilogues (bf16, tokens 8192, 1024 -> 4096 -> 1024) against the
          HBM peak, on a rotating working set larger than the caches
other_attention  forward and backward time of the OPT-2.7B-shaped (padding mask) and the two
          GPT-Neo-1.3B-shaped (global / window 256, dropout 0.1) attention calls, bf16
bert_large_fp32  BASELINE configuration 1, which is DEFINED as the native CPU path: the oracle's
          fp32 forward of B 4, S 512, 16 x 64 on the host cores, and beside it the fp32 FMA kernel
          of this library on the same tensors against the fp32 vector peak (reported, not a target)
cpu_baseline  the oracle's native-PyTorch restatement (fp32 CPU, autograd backward) timed on the
          host cores on a bounded sample of the same workload; every epilogue / other_attention
          entry carries a cpu_baseline of its own (a bounded chunk of its tensors)

The headline is the MEDIAN of `--repeats` (default 25) timed loops of `--steps` steps each,
every loop bracketed by a device synchronisation on both sides and free of events; `ms_per_step` x
`steps` is the duration of that median loop, `median_loop_index` says which one it was (loops are
listed in the order they ran: a 20-step loop lasts under 3 ms, and the first ones run on clocks
that have not settled).  The per-kernel durations come from a separate pass over the same steps
with HIP events around every launch, less the events' own share of the intervals.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 / bf16
FP32_VECTOR_PEAK_TFLOPS = 157.3
# HBM bytes per launch of the dK/dV kernel on WORKLOAD, from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE (KiB per dispatch), each scaled by the same counter's reading for a 256 MiB copy
# (FETCH_SIZE reads half the copied bytes: factor 2.0; WRITE_SIZE factor 1.0):
# (43.93e3 * 2.0 + 32.77e3) KiB = 123.5 MB against 101.7 MB algorithmic.  Summary under profiles/.
DKDV_TRAFFIC_BYTES = (43.46e3 * 2.0 + 32.77e3) * 1024
HBM_PEAK_GBS = 8000.0      # MI355X HBM3E

WORKLOAD = dict(name="gpt2-medium causal attention fwd+bwd", dtype="fp16", batch=8, seq=1024,
                heads=16, head_dim=64, causal=True, p=0.0, seed=2013)


def _pairs(seq, causal):
    return seq * (seq + 1) // 2 if causal else seq * seq


def _make_inputs(cfg, device):
    g = torch.Generator().manual_seed(cfg["seed"])
    shape = (cfg["batch"], cfg["seq"], cfg["heads"], cfg["head_dim"])
    return [torch.randn(shape, generator=g).to(torch.float16).to(device) for _ in range(4)]


SETTLE_SECONDS = 0.03


def _settle(fn):
    """Runs fn back to back for SETTLE_SECONDS of wall time before a timed measurement: a few
    launches are not enough for the device clock to settle after an idle stretch (the first
    10-20 ms of a burst run 5-15 % slow on these boxes).  `--settle-ms 0` switches it off, for
    counter collection, where every dispatch is recorded."""
    t_end = time.perf_counter() + SETTLE_SECONDS
    while time.perf_counter() < t_end:
        for _ in range(8):
            fn()
    torch.cuda.synchronize()


class AttentionStep:
    """Forward + backward of the attention op through the C ABI on preallocated buffers."""

    def __init__(self, cfg, device):
        from slapo_amd import _lib
        from slapo_amd.op import _kernels as K

        self.lib = _lib.load()
        self._lib_mod = _lib
        self.q, self.k, self.v, self.do = _make_inputs(cfg, device)
        q = self.q
        self.o = torch.empty_like(q)
        self.lse = torch.empty(cfg["batch"], cfg["heads"], cfg["seq"], dtype=torch.float32,
                               device=device)
        self.dq, self.dk, self.dv = (torch.empty_like(q) for _ in range(3))
        self.prm = K.make_attn_params(self.q, self.k, self.v, self.o, None, cfg["causal"], 0,
                                      cfg["head_dim"] ** -0.5, 0.0, 0, 0, None)
        nbytes = self.lib.slapo_amd_attn_bwd_workspace_bytes(ctypes.byref(self.prm))
        self.ws = torch.empty(nbytes // 4, dtype=torch.float32, device=device)
        self.ws_bytes = nbytes
        self.strides = [K._bshd_strides(t) for t in (self.dq, self.dk, self.dv)]
        self.stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        P = lambda t: ctypes.c_void_p(t.data_ptr())
        self.fwd_args = (ctypes.byref(self.prm), P(self.q), P(self.k), P(self.v), None, P(self.o),
                         P(self.lse), self.stream)
        self.bwd_args = (ctypes.byref(self.prm), P(self.q), P(self.k), P(self.v), None, P(self.o),
                         P(self.do), P(self.lse), P(self.dq), P(self.dk), P(self.dv),
                         *self.strides, P(self.ws), self.ws_bytes)

    def forward(self):
        rc = self.lib.slapo_amd_attn_fwd(*self.fwd_args)
        if rc:
            raise RuntimeError(f"slapo_amd_attn_fwd failed with status {rc}")

    def backward(self, stages=7):
        rc = self.lib.slapo_amd_attn_bwd_stages(*self.bwd_args, stages, self.stream)
        if rc:
            raise RuntimeError(f"slapo_amd_attn_bwd_stages failed with status {rc}")

    def step(self, ev=None):
        """ev: four events recorded around forward | dQ (+ delta) | dK/dV."""
        if ev is not None:
            ev[0].record()
        self.forward()
        if ev is not None:
            ev[1].record()
        self.backward(self._lib_mod.BWD_PREPARE | self._lib_mod.BWD_DQ)
        if ev is not None:
            ev[2].record()
        self.backward(self._lib_mod.BWD_DKDV)
        if ev is not None:
            ev[3].record()


def bench_epilogues(device, iters=40):
    """GB/s of bias-GeLU fwd and bias-dropout-residual fwd on rotating buffers (> 1 GB)."""
    from slapo_amd import _lib
    from slapo_amd.op import _kernels as K

    lib = _lib.load()
    T, I, Hd = 8192, 4096, 1024
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    bf = torch.bfloat16
    out = {}

    def timed(fn, n_rot):
        for i in range(n_rot):
            fn(i)
        _settle(lambda: fn(0))
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(iters):
            fn(i % n_rot)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters * 1e-3  # seconds per launch

    n_rot = 8
    ys = [torch.randn(T, I, device=device, dtype=bf) for _ in range(n_rot)]
    outs = [torch.empty(T, I, device=device, dtype=bf) for _ in range(n_rot)]
    b = torch.randn(I, device=device, dtype=bf)

    def gelu(i):
        rc = lib.slapo_amd_bias_gelu_fwd(P(ys[i]), P(b), P(outs[i]), T, I, _lib.SLAPO_BF16, st)
        assert rc == 0

    sec = timed(gelu, n_rot)
    nbytes = 2 * T * I * 2 + I * 2
    out["bias_gelu_fwd"] = {"bytes": nbytes, "us": sec * 1e6, "GBps": nbytes / sec / 1e9,
                            "frac_of_hbm_peak": nbytes / sec / 1e9 / HBM_PEAK_GBS}

    gos = outs

    def gelu_bwd(i):
        rc = lib.slapo_amd_bias_gelu_bwd(P(gos[i]), P(ys[i]), P(b), P(outs[(i + 1) % n_rot]),
                                         P(db), P(ws), ws_bytes, T, I, _lib.SLAPO_BF16, st)
        assert rc == 0

    ws_bytes = lib.slapo_amd_colsum_workspace_bytes(T, I)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=device)
    db = torch.empty(I, device=device, dtype=bf)
    sec = timed(gelu_bwd, n_rot)
    nbytes = 3 * T * I * 2 + 2 * I * 2
    out["bias_gelu_bwd"] = {"bytes": nbytes, "us": sec * 1e6, "GBps": nbytes / sec / 1e9,
                            "frac_of_hbm_peak": nbytes / sec / 1e9 / HBM_PEAK_GBS}
    del ys, outs, gos

    n_rot = 24
    xs = [torch.randn(T, Hd, device=device, dtype=bf) for _ in range(n_rot)]
    rs = [torch.randn(T, Hd, device=device, dtype=bf) for _ in range(n_rot)]
    os_ = [torch.empty(T, Hd, device=device, dtype=bf) for _ in range(n_rot)]
    b1 = torch.randn(Hd, device=device, dtype=bf)
    plan = K.dropout_plan(T * Hd, 2, device)

    def dropres(i):
        rc = lib.slapo_amd_bias_dropout_residual_fwd(P(xs[i]), P(b1), P(rs[i]), P(os_[i]), T, Hd,
                                                     _lib.SLAPO_BF16, 0.1, 2013, 0,
                                                     ctypes.byref(plan), st)
        assert rc == 0

    sec = timed(dropres, n_rot)
    nbytes = 3 * T * Hd * 2 + Hd * 2
    out["bias_dropout_residual_fwd"] = {"bytes": nbytes, "us": sec * 1e6,
                                        "GBps": nbytes / sec / 1e9,
                                        "frac_of_hbm_peak": nbytes / sec / 1e9 / HBM_PEAK_GBS}

    # backward of the bias-dropout(-residual) epilogue: dx = dropout mask applied to the upstream
    # gradient (the mask is redrawn from seed and offset), dbias = its column sum
    bws_bytes = lib.slapo_amd_colsum_workspace_bytes(T, Hd)
    bws = torch.empty(bws_bytes // 4, dtype=torch.float32, device=device)
    db1 = torch.empty(Hd, device=device, dtype=bf)

    def dropres_bwd(i):  # reads the gradient (os_), writes dx (xs) and dbias
        rc = lib.slapo_amd_bias_dropout_residual_bwd(P(os_[i]), P(xs[i]), P(db1), P(bws),
                                                     bws_bytes, T, Hd, _lib.SLAPO_BF16, 0.1, 2013,
                                                     0, ctypes.byref(plan), st)
        assert rc == 0

    sec = timed(dropres_bwd, n_rot)
    nbytes = 2 * T * Hd * 2 + Hd * 2
    out["bias_dropout_residual_bwd"] = {"bytes": nbytes, "us": sec * 1e6,
                                        "GBps": nbytes / sec / 1e9,
                                        "frac_of_hbm_peak": nbytes / sec / 1e9 / HBM_PEAK_GBS}

    # bias + dropout + residual + LayerNorm, training form: z, mean, rstd written for the backward
    zs = [torch.empty(T, Hd, device=device, dtype=bf) for _ in range(n_rot)]
    gam = torch.ones(Hd, device=device, dtype=bf)
    bet = torch.zeros(Hd, device=device, dtype=bf)
    mean = torch.empty(T, device=device, dtype=torch.float32)
    rstd = torch.empty(T, device=device, dtype=torch.float32)

    def ln_fwd(i):
        rc = lib.slapo_amd_bias_dropout_residual_ln_fwd(
            P(xs[i]), P(b1), P(rs[i]), P(gam), P(bet), P(zs[i]), P(os_[i]), P(mean), P(rstd), T,
            Hd, _lib.SLAPO_BF16, 1e-5, 0.1, 2013, 0, ctypes.byref(plan), st)
        assert rc == 0

    sec = timed(ln_fwd, n_rot)
    nbytes = 4 * T * Hd * 2 + 3 * Hd * 2 + 2 * T * 4
    out["bias_dropout_residual_ln_fwd"] = {"bytes": nbytes, "us": sec * 1e6,
                                           "GBps": nbytes / sec / 1e9,
                                           "frac_of_hbm_peak": nbytes / sec / 1e9 / HBM_PEAK_GBS}

    lws_bytes = lib.slapo_amd_ln_bwd_workspace_bytes(T, Hd)
    lws = torch.empty(lws_bytes // 4, dtype=torch.float32, device=device)
    dgam, dbet, dbi = (torch.empty(Hd, device=device, dtype=bf) for _ in range(3))

    def ln_bwd(i):  # reads dy (os_), z; writes dx (xs), dresidual (rs) and the three column sums
        rc = lib.slapo_amd_bias_dropout_residual_ln_bwd(
            P(os_[i]), P(zs[i]), P(mean), P(rstd), P(gam), P(xs[i]), P(rs[i]), P(dgam), P(dbet),
            P(dbi), P(lws), lws_bytes, T, Hd, _lib.SLAPO_BF16, 0.1, 2013, 0, ctypes.byref(plan),
            st)
        assert rc == 0

    sec = timed(ln_bwd, n_rot)
    nbytes = 4 * T * Hd * 2 + 4 * Hd * 2 + 2 * T * 4  # partial sums (2 x 6 MB) not credited
    out["bias_dropout_residual_ln_bwd"] = {"bytes": nbytes, "us": sec * 1e6,
                                           "GBps": nbytes / sec / 1e9,
                                           "frac_of_hbm_peak": nbytes / sec / 1e9 / HBM_PEAK_GBS}
    del xs, rs, os_, zs

    # vocab-parallel cross entropy on one shard: GPT-2's unpadded vocabulary, fp16 logits
    V = 50257
    logits = torch.randn(T, V, device=device, dtype=torch.float16)
    grad = torch.empty_like(logits)
    tgt = torch.randint(0, V, (T,), device=device)
    stats = torch.empty(4, T, device=device, dtype=torch.float32)
    gl = torch.ones(T, device=device, dtype=torch.float32)

    def ce_fwd(i):
        rc = lib.slapo_amd_vocab_ce_fwd(P(logits), P(tgt), P(stats[0]), P(stats[1]), P(stats[2]),
                                        P(stats[3]), T, V, 0, _lib.SLAPO_F16, st)
        assert rc == 0

    sec = timed(ce_fwd, 1)
    nbytes = T * V * 2 + T * (8 + 16)
    out["vocab_ce_fwd"] = {"bytes": nbytes, "us": sec * 1e6, "GBps": nbytes / sec / 1e9,
                           "frac_of_hbm_peak": nbytes / sec / 1e9 / HBM_PEAK_GBS}
    inv_s = 1.0 / stats[1]

    def ce_bwd(i):
        rc = lib.slapo_amd_vocab_ce_bwd(P(logits), P(tgt), P(stats[0]), P(inv_s), P(gl), P(grad),
                                        T, V, 0, 0.0, _lib.SLAPO_F16, st)
        assert rc == 0

    sec = timed(ce_bwd, 1)
    nbytes = 2 * T * V * 2 + T * (8 + 12)
    out["vocab_ce_bwd"] = {"bytes": nbytes, "us": sec * 1e6, "GBps": nbytes / sec / 1e9,
                           "frac_of_hbm_peak": nbytes / sec / 1e9 / HBM_PEAK_GBS}
    return out


def _cpu_info():
    """Host description that goes with every CPU figure: logical cores, threads used, model."""
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"os_cpu_count": os.cpu_count(), "torch_num_threads": torch.get_num_threads(),
            "cpu_model": model}


def _use_all_cores():
    torch.set_num_threads(os.cpu_count() or 1)
    return torch.get_num_threads()


def _median_time(fn, reps=3):
    fn()  # warm-up
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return sorted(times)[len(times) // 2]


def cpu_epilogue_baselines():
    """The oracle's epilogues and cross entropy (native PyTorch, fp32 math on 16-bit values) on
    4096 of the 8192 rows (cross entropy: 512); GB/s count the same algorithmic bytes per row as
    the GPU entries."""
    from oracle import cross_entropy as OC
    from oracle import epilogue as OE

    threads = _use_all_cores()
    rows, T, I, Hd, e = 4096, 8192, 4096, 1024, 2
    g = torch.Generator().manual_seed(2013)
    bf = torch.bfloat16
    y = torch.randn(rows, I, generator=g).to(bf)
    bi = torch.randn(I, generator=g).to(bf)
    gr = torch.randn(rows, I, generator=g).to(bf)
    x = torch.randn(rows, Hd, generator=g).to(bf)
    b1 = torch.randn(Hd, generator=g).to(bf)
    res = torch.randn(rows, Hd, generator=g).to(bf)
    keep = torch.rand(rows, Hd, generator=g) >= 0.1
    w, lb = torch.ones(Hd), torch.zeros(Hd)
    sample = f"{rows} of {T} rows, fp32 math, median of 3"
    out = {}

    def entry(name, nbytes_full, fn):
        sec = _median_time(fn)
        out[name] = {"value": nbytes_full * rows / T / sec / 1e9, "unit": "GB/s", "cores": threads,
                     "kind": "port", "sample": f"{sample}, {sec * 1e3:.1f} ms per pass"}

    entry("bias_gelu_fwd", 2 * T * I * e + I * e,
          lambda: OE.bias_gelu(bi, y, torch.float32).to(bf))
    entry("bias_gelu_bwd", 3 * T * I * e + 2 * I * e,
          lambda: OE.bias_gelu_back(gr, bi, y, torch.float32).to(bf))
    entry("bias_dropout_residual_fwd", 3 * T * Hd * e + Hd * e,
          lambda: OE.bias_dropout_residual(x, b1, res, 0.1, keep, torch.float32).to(bf))
    gx = torch.randn(rows, Hd, generator=g).to(bf)

    def dropres_bwd_cpu():
        dx, dbias, _ = OE.bias_dropout_residual_bwd(gx, 0.1, keep, torch.float32)
        return dx.to(bf), dbias.to(bf)

    entry("bias_dropout_residual_bwd", 2 * T * Hd * e + Hd * e, dropres_bwd_cpu)
    entry("bias_dropout_residual_ln_fwd", 4 * T * Hd * e + 3 * Hd * e + 2 * T * 4,
          lambda: OE.bias_dropout_residual_layer_norm(x, b1, res, w, lb, 1e-5, 0.1, keep,
                                                      torch.float32)[0].to(bf))
    _, z, mean, rstd = OE.bias_dropout_residual_layer_norm(x, b1, res, w, lb, 1e-5, 0.1, keep,
                                                           torch.float32, z_dtype=bf)
    gy = torch.randn(rows, Hd, generator=g).to(bf)
    entry("bias_dropout_residual_ln_bwd", 4 * T * Hd * e + 4 * Hd * e + 2 * T * 4,
          lambda: OE.bias_dropout_residual_layer_norm_bwd(gy, z, mean, rstd, w, 0.1, keep,
                                                          torch.float32)[0].to(bf))
    rows_ce, V = 512, 50257
    logits = torch.randn(rows_ce, V, generator=g).to(torch.float16)
    tgt = torch.randint(0, V, (rows_ce,), generator=g)
    ones = torch.ones(rows_ce)
    rows = rows_ce
    sample = f"{rows} of {T} rows, fp32 math, median of 3"
    entry("vocab_ce_fwd", T * V * 2 + T * (8 + 16),
          lambda: OC.forward(logits, tgt, 0.0, torch.float32)[0])
    soft = OC.forward(logits, tgt, 0.0, torch.float32)[1]
    entry("vocab_ce_bwd", 2 * T * V * 2 + T * (8 + 12),
          lambda: OC.backward(soft, tgt, ones).to(torch.float16))
    return out


def cpu_attention_chunk(cfg, heads, lens=None):
    """The oracle's attention fwd+bwd (fp32 CPU, autograd) on one batch and `heads` heads of an
    other_attention workload; TFLOP/s count 14 * D per attended pair of the chunk."""
    from oracle import attention as OA

    threads = _use_all_cores()
    S, D, w, p = cfg["seq"], cfg["head_dim"], cfg["window"], cfg["p"]
    g = torch.Generator().manual_seed(2013)
    q, k, v, do = (torch.randn((1, S, heads, D), generator=g).to(torch.bfloat16) for _ in range(4))
    mask, n = None, S
    if lens is not None:
        n = lens[0]
        mask = torch.zeros(1, 1, 1, S)
        mask[0, 0, 0, n:] = torch.finfo(torch.bfloat16).min
    keep = (torch.rand(heads, S, S, generator=g) >= p) if p > 0 else None
    sec = _median_time(lambda: OA.attention_fwd_bwd(q, k, v, do, mask, True, w, p, keep, None,
                                                    torch.float32), reps=3)
    pairs = OA.attended_pairs(S, S, True, w, n) * heads
    return {"value": 14 * D * pairs / sec / 1e12, "unit": "TFLOP/s", "cores": threads,
            "kind": "port", "sample": f"1 of {cfg['batch']} batches, {heads} of {cfg['heads']} "
                                      f"heads, fp32 math on bf16 inputs, {sec:.2f} s per pass"}


def bench_bert_large_fp32(device, iters=10):
    """BASELINE configuration 1: BERT-large-shaped self-attention, fp32, B 4, S 512, 16 x 64, no
    mask, dropout 0, forward only.  The configuration is defined as the native CPU path, so the
    CPU time of the oracle IS its figure; the library's fp32 FMA kernel runs beside it."""
    from oracle import attention as OA
    from slapo_amd import op

    threads = _use_all_cores()
    B, S, H, D = 4, 512, 16, 64
    g = torch.Generator().manual_seed(2013)
    q, k, v = (torch.randn((B, S, H, D), generator=g) for _ in range(3))
    flops = 4 * D * S * S * B * H
    cpu_sec = _median_time(lambda: OA.xformers_ref(q, k, v, None, False,
                                                   compute_dtype=torch.float32))
    qd, kd, vd = (t.to(device) for t in (q, k, v))
    for _ in range(3):
        op.hip_attention(qd, kd, vd, None, causal=False)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        op.hip_attention(qd, kd, vd, None, causal=False)
    e1.record()
    torch.cuda.synchronize()
    gpu_sec = e0.elapsed_time(e1) / iters * 1e-3
    return {"workload": "bert-large self-attention forward, fp32, B4 S512 H16 D64, no mask",
            "flops": flops,
            "cpu": {"ms": cpu_sec * 1e3, "TFLOPs": flops / cpu_sec / 1e12, "cores": threads,
                    "kind": "port", "sample": "the whole configuration, median of 3"},
            "gpu_fp32_fma_kernel": {"ms": gpu_sec * 1e3, "TFLOPs": flops / gpu_sec / 1e12,
                                    "peak": FP32_VECTOR_PEAK_TFLOPS,
                                    "frac_of_fp32_vector_peak":
                                        flops / gpu_sec / 1e12 / FP32_VECTOR_PEAK_TFLOPS,
                                    "note": "parity kernel (1e-5 bar), not a performance target"}}


def cpu_baseline(cfg, budget_batches=8):
    """The oracle's native path (fp32 CPU, autograd) on `budget_batches` of the 8 batches."""
    from oracle import attention as OA

    threads = _use_all_cores()
    g = torch.Generator().manual_seed(cfg["seed"])
    shape = (budget_batches, cfg["seq"], cfg["heads"], cfg["head_dim"])
    q, k, v, do = (torch.randn(shape, generator=g).to(torch.float16) for _ in range(4))

    def run():
        t0 = time.perf_counter()
        OA.attention_fwd_bwd(q, k, v, do, None, cfg["causal"], compute_dtype=torch.float32)
        return time.perf_counter() - t0

    run()  # warm-up
    times = sorted(run() for _ in range(9))
    sec = times[4]
    flops = 14 * cfg["head_dim"] * _pairs(cfg["seq"], cfg["causal"]) * budget_batches * cfg["heads"]
    return {"value": flops / sec / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"{budget_batches} of {cfg['batch']} batches of the same workload "
                      f"(fp32 math on fp16 inputs, median of 9, {sec:.2f} s per pass)"}


OTHER_ATTENTION = [
    dict(name="opt-2.7b causal + key-padding attention fwd+bwd", batch=4, seq=2048, heads=32,
         head_dim=80, window=0, p=0.0, padding=True),
    dict(name="gpt-neo-1.3b global causal attention fwd+bwd, dropout 0.1", batch=4, seq=2048,
         heads=16, head_dim=128, window=0, p=0.1, padding=False),
    dict(name="gpt-neo-1.3b local causal attention (window 256) fwd+bwd, dropout 0.1", batch=4,
         seq=2048, heads=16, head_dim=128, window=256, p=0.1, padding=False),
]


def bench_other_attention(device, iters=20, with_cpu=True):
    """Forward and backward time of the other attention shapes of the benchmark set (bf16), through
    the C ABI on preallocated buffers; TFLOP/s count 14 * D FLOP per attended (query, key) pair.
    The padding mask is the compact additive [B,1,1,Sk] tensor with per-sequence valid lengths
    ~ Uniform[512, 2048]; with dropout the backward reads the keep bits the forward stored."""
    from slapo_amd import _lib
    from slapo_amd.op import _kernels as K

    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
    bf = torch.bfloat16
    out = []
    for cfg in OTHER_ATTENTION:
        B, S, H, D = cfg["batch"], cfg["seq"], cfg["heads"], cfg["head_dim"]
        g = torch.Generator().manual_seed(2013)
        q, k, v, do = (torch.randn((B, S, H, D), generator=g).to(bf).to(device) for _ in range(4))
        bias, lens = None, [S] * B
        if cfg["padding"]:
            lens = torch.randint(512, S + 1, (B,), generator=g).tolist()
            m = torch.zeros(B, 1, 1, S)
            for i, n in enumerate(lens):
                m[i, 0, 0, n:] = torch.finfo(bf).min
            bias = K.prepare_bias(m.to(device), B, H, S, S)
        w = cfg["window"]
        pairs = 0
        for n in lens:  # query i sees keys max(0, i - w + 1) .. min(i, n - 1)
            for i in range(S):
                lo = max(0, i - w + 1) if w else 0
                pairs += max(0, min(i, n - 1) - lo + 1)
        pairs *= H
        plan = K.dropout_plan(B * H * S * S, 4, q.device) if cfg["p"] > 0 else None
        scale = D ** -0.5
        o, lse, _, keep = K.attn_fwd(q, k, v, bias, True, w, scale, cfg["p"], 2013, 0, plan,
                                     save_mask=True)
        prm = K.make_attn_params(q, k, v, o, bias, True, w, scale, cfg["p"], 2013, 0, plan, keep)
        dq, dk, dv = (torch.empty_like(q) for _ in range(3))
        nbytes = lib.slapo_amd_attn_bwd_workspace_bytes(ctypes.byref(prm))
        ws = torch.empty(nbytes // 4, dtype=torch.float32, device=device)
        strides = [K._bshd_strides(t) for t in (dq, dk, dv)]

        def fwd():
            rc = lib.slapo_amd_attn_fwd(ctypes.byref(prm), P(q), P(k), P(v), P(bias), P(o), P(lse),
                                        st)
            if rc:
                raise RuntimeError(f"slapo_amd_attn_fwd failed with status {rc}")

        def bwd():
            rc = lib.slapo_amd_attn_bwd(ctypes.byref(prm), P(q), P(k), P(v), P(bias), P(o), P(do),
                                        P(lse), P(dq), P(dk), P(dv), *strides, P(ws), nbytes, st)
            if rc:
                raise RuntimeError(f"slapo_amd_attn_bwd failed with status {rc}")

        def timed(fn):
            for _ in range(3):
                fn()
            _settle(fn)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / iters * 1e-3

        tf, tb = timed(fwd), timed(bwd)
        stage_us = {}
        for name, bits in (("dq_us", _lib.BWD_PREPARE | _lib.BWD_DQ), ("dkdv_us", _lib.BWD_DKDV)):
            def one(bits=bits):
                rc = lib.slapo_amd_attn_bwd_stages(ctypes.byref(prm), P(q), P(k), P(v), P(bias),
                                                   P(o), P(do), P(lse), P(dq), P(dk), P(dv),
                                                   *strides, P(ws), nbytes, bits, st)
                if rc:
                    raise RuntimeError(f"slapo_amd_attn_bwd_stages failed with status {rc}")
            stage_us[name] = timed(one) * 1e6
        tflops = 14 * D * pairs / (tf + tb) / 1e12
        entry = {"workload": cfg["name"], "dtype": "bf16", "batch": B, "seq_len": S, "heads": H,
                 "head_dim": D, "window": w, "dropout_p": cfg["p"], "attended_pairs": pairs,
                 "fwd_us": tf * 1e6, "bwd_us": tb * 1e6, **stage_us, "TFLOPs": tflops,
                 "frac_of_mfma_peak": tflops / MFMA_PEAK_TFLOPS}
        if with_cpu:
            entry["cpu_baseline"] = cpu_attention_chunk(cfg, 16, lens if cfg["padding"] else None)
        out.append(entry)
        del q, k, v, do, o, lse, dq, dk, dv, ws, keep, bias
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--repeats", type=int, default=25,
                    help="timed loops of --steps steps; the median loop is reported")
    ap.add_argument("--settle-ms", type=float, default=30.0,
                    help="back-to-back launches for this long before each timed sub-benchmark")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-epilogues", action="store_true")
    ap.add_argument("--no-other-attention", action="store_true",
                    help="skip the other attention shapes of the benchmark set")
    ap.add_argument("--traffic-reference", action="store_true",
                    help="also run three 256 MiB device-to-device copies, the known-size kernel "
                         "against which FETCH_SIZE / WRITE_SIZE counter readings are scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU's throughput; --gpus above 1 is not supported "
                 "(no collectives are part of this hot path)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs an MI355X (no GPU visible)")

    global SETTLE_SECONDS
    SETTLE_SECONDS = max(args.settle_ms, 0.0) * 1e-3
    cfg = WORKLOAD
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)
    if args.traffic_reference:
        src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device=device).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    step = AttentionStep(cfg, device)

    for _ in range(args.warmup):
        step.step()
    torch.cuda.synchronize()
    loops = []
    for _ in range(max(1, args.repeats)):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step.step()
        torch.cuda.synchronize()
        loops.append(time.perf_counter() - t0)
    order = sorted(range(len(loops)), key=lambda i: loops[i])
    median_index = order[len(order) // 2]
    elapsed = loops[median_index]

    # Per-kernel durations: a pass of its own over the same steps, with HIP events (recorded on the
    # launching stream) around each of the three launches of every step.  An event between two
    # launches costs stream time of its own (2-3 us here), so the three intervals of a step add up
    # to more than a step of the timed loops; that excess is the events', and a third of it is
    # taken off each interval (the figures then agree with rocprofv3's kernel durations within
    # 2 %, and add up to `ms_per_step`).
    n_ev = max(args.steps, 40)
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(n_ev)]
    torch.cuda.synchronize()
    for ev in events:
        step.step(ev)
    torch.cuda.synchronize()
    seg_raw = [sum(ev[i].elapsed_time(ev[i + 1]) for ev in events) / len(events) for i in range(3)]
    event_cost_ms = max(sum(seg_raw) - elapsed / args.steps * 1e3, 0.0) / 3
    seg_ms = [max(t - event_cost_ms, 0.0) for t in seg_raw]

    n_pairs = _pairs(cfg["seq"], cfg["causal"]) * cfg["batch"] * cfg["heads"]
    d = cfg["head_dim"]
    ms_per_step = elapsed / args.steps * 1e3
    value = 14 * d * n_pairs / (elapsed / args.steps) / 1e12
    kern_ms = seg_ms[2]
    bwd_flops = 8 * d * n_pairs
    achieved = bwd_flops / (kern_ms * 1e-3) / 1e12

    def kern(name, flops, ms):
        tf = flops / (ms * 1e-3) / 1e12
        return {"kernel": name, "flops_per_launch": flops, "avg_launch_ms": ms, "TFLOPs": tf,
                "frac_of_mfma_peak": tf / MFMA_PEAK_TFLOPS}

    result = {
        "metric": "attention fwd+bwd TFLOP/s + epilogue GB/s, % of MI355X roofline, 1 GPU",
        "value": value,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "repeats": len(loops),
        "ms_per_step": ms_per_step,
        "median_loop_index": median_index,
        "ms_per_step_of_every_loop": [t / args.steps * 1e3 for t in loops],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": cfg["name"], "batch": cfg["batch"], "seq_len": cfg["seq"],
                   "heads": cfg["heads"], "head_dim": cfg["head_dim"], "causal": cfg["causal"],
                   "dropout_p": cfg["p"], "flops_per_step": 14 * d * n_pairs},
        "frac_of_mfma_peak": value / MFMA_PEAK_TFLOPS,
        "roofline": {"bound": "mfma", "kernel": "attn_bwd_kernel<f16,64,0,0,1,4> (dK/dV)",
                     "achieved": achieved,
                     "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / MFMA_PEAK_TFLOPS, "traffic": DKDV_TRAFFIC_BYTES,
                     "flops_per_launch": bwd_flops, "avg_launch_ms": kern_ms},
        "kernel_timing": {"steps_with_events": n_ev, "event_cost_ms": event_cost_ms,
                          "raw_event_intervals_ms": seg_raw,
                          "sum_of_kernels_ms": sum(seg_ms)},
    }
    result["kernels"] = [kern("attn_fwd_kernel<f16,64,0,0,0,4>", 4 * d * n_pairs, seg_ms[0]),
                         kern("attn_bwd_kernel<f16,64,0,0,1,4> (dK/dV)", bwd_flops, seg_ms[2]),
                         kern("attn_bwd_dq_kernel<f16,64,0,0,true,4>", 6 * d * n_pairs, seg_ms[1])]
    with_cpu = not args.no_cpu_baseline
    if not args.no_epilogues:
        result["epilogue"] = bench_epilogues(device)
        if with_cpu:
            for name, base in cpu_epilogue_baselines().items():
                result["epilogue"][name]["cpu_baseline"] = base
    if not args.no_other_attention:
        result["other_attention"] = bench_other_attention(device, with_cpu=with_cpu)
    if with_cpu:
        result["bert_large_fp32"] = bench_bert_large_fp32(device)
        result["cpu_baseline"] = cpu_baseline(cfg)
        result["host"] = _cpu_info()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
