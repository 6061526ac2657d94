#!/usr/bin/env python3
"""Benchmark of the tensor-parallel hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extras]

Headline (``value``): TFLOP/s of one rank's Llama-3-8B-shaped linears, forward +
backward, bf16 with fp32 accumulate, on 4096 tokens:
    QKV 4096->6144, gate/up 4096->2x14336 with fused SwiGLU, down 14336->4096.
A step is: 3 forwards (Y = X W^T, SwiGLU fused into the gate/up epilogue), the
SwiGLU backward, 3 input gradients (dX = dY W) and 3 weight gradients
(dW = dY^T X), the two gradients of a layer through the one call the layers'
backward makes (one launch where their tiles share rounds of workgroups).  FLOPs counted: 6*M*K*N per layer (4947.8 GFLOP per step); the
activation work is executed inside the timed region but not counted.

Inputs are resident in HBM before the timed region.  Timing: W warm-up steps,
then K steps between two ``torch.cuda.synchronize()`` calls.  The per-kernel
figures under ``roofline`` / ``kernels`` come from HIP events recorded on the
launch stream around each launch, inside this same process.

``secondary`` carries the other pieces of the path (cross entropy, embedding
gather, decode GEMV + argmax, the Llama-70B tp=8 shard shapes and the fp32
GPT-2 shapes) — one number each, same event timing.  ``cpu_baseline`` is the
CPU oracle (the reference's op sequence in torch fp32) on a bounded sample.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_F32_TFLOPS = 157.3     # MI355X fp32 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "hbm_traffic_fetch_write_size.txt")


def measured_traffic():
    """HBM bytes per launch from the committed rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summary: its lines
    `traffic_bytes <kernel of this file> <bytes>` and `measured_at <commit>`.  ({}, None) when the file is absent:
    the figure is a measurement of a profiler run, never a constant of this script."""
    rows, stamp = {}, None
    try:
        with open(TRAFFIC_PROFILE) as f:
            for line in f:
                t = line.split()
                if len(t) >= 3 and t[0] == "traffic_bytes":
                    rows[t[1]] = float(t[2])
                elif len(t) >= 2 and t[0] == "measured_at":
                    stamp = t[1]
    except OSError:
        pass
    return rows, stamp


LLAMA8B = [  # (name, K, N, epilogue)
    ("qkv", 4096, 6144, "none"),
    ("gate_up", 4096, 2 * 14336, "swiglu"),
    ("down", 14336, 4096, "none"),
]
LLAMA70B_TP8 = [
    ("qkv", 8192, 1280, "none"),
    ("gate_up", 8192, 2 * 3584, "swiglu"),
    ("down", 3584, 8192, "none"),
    ("o_proj", 1024, 8192, "none"),
]


def gen(seed):
    return torch.Generator().manual_seed(1234 + seed)


class Timer:
    """HIP events on the current stream (the stream every kernel here is launched on).  Every figure this script
    prints is the MEAN of the timed repetitions (what a profiler's per-kernel average is); the medians are kept
    beside them (`median`) and go into the roofline entry."""

    WARM_S = 0.03

    def __init__(self):
        self.t = {}
        self.median = {}

    def run(self, name, fn, reps):
        # untimed: first touch of the buffers, then the same launches for WARM_S seconds.  The board's power
        # management needs some milliseconds to settle on a new kernel mix (measured on the LM-head GEMV: 151 us
        # for ten launches after a change of workload, 175-185 us for the next ten, back to 152 us within
        # forty), and what is reported is the sustained rate.
        t0 = time.perf_counter()
        n = 0
        while n < 3 or time.perf_counter() - t0 < self.WARM_S:
            fn()
            n += 1
            if n % 8 == 0:
                torch.cuda.synchronize()
        torch.cuda.synchronize()
        evs = []
        for _ in range(reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            evs.append((a, b))
        torch.cuda.synchronize()
        ms = [a.elapsed_time(b) for a, b in evs]
        self.t[name] = statistics.mean(ms)      # the mean: an average launch duration, like a profiler's summary
        self.median[name] = statistics.median(ms)
        return self.t[name]


def build_linear_workload(dev, layers, M, seed):
    from merak_amd import ops
    out = []
    for i, (name, K, N, epi) in enumerate(layers):
        x = torch.randn(M, K, generator=gen(seed + 10 * i)).bfloat16().to(dev)
        w = (torch.randn(N, K, generator=gen(seed + 10 * i + 1)) * 0.02).bfloat16().to(dev)
        n_out = N // 2 if epi == "swiglu" else N
        dy = torch.randn(M, n_out, generator=gen(seed + 10 * i + 2)).bfloat16().to(dev)
        out.append(dict(name=name, K=K, N=N, M=M, epi=ops.EPI_SWIGLU if epi == "swiglu" else ops.EPI_NONE,
                        x=x, w=w, dy=dy, flops=6.0 * M * K * N))
    return out


def linear_step(work):
    """fwd + bwd of every layer; returns nothing (outputs are dropped, as a trainer's would be consumed)."""
    from merak_amd import ops
    for L in work:
        y, act = ops.linear_fwd(L["x"], L["w"], None, L["epi"], want_pre=True)
        g = L["dy"]
        if L["epi"] == ops.EPI_SWIGLU:
            g = ops.activation_bwd(g, y, ops.EPI_SWIGLU)
        ops.linear_bwd(g, L["x"], L["w"], False)     # dX and dW: one call, as the layers' backward makes it


def per_kernel(work, timer, reps):
    """Average launch duration of each GEMM launch of the step, by HIP events."""
    from merak_amd import ops
    rows = []
    for L in work:
        M, K, N = L["M"], L["K"], L["N"]
        y, act = ops.linear_fwd(L["x"], L["w"], None, L["epi"], want_pre=True)
        g = L["dy"] if L["epi"] != ops.EPI_SWIGLU else ops.activation_bwd(L["dy"], y, ops.EPI_SWIGLU)
        for kind, fn in (("fwd", lambda: ops.linear_fwd(L["x"], L["w"], None, L["epi"], want_pre=True)),
                         ("dgrad", lambda: ops.linear_dgrad(g, L["w"])),
                         ("wgrad", lambda: ops.linear_wgrad(g, L["x"], False))):
            ms = timer.run(f"{L['name']}.{kind}", fn, reps)
            rows.append(dict(kernel=f"{L['name']}.{kind}", M=M, N=N, K=K, ms=round(ms, 4),
                             tflops=round(2.0 * M * N * K / ms / 1e9, 1)))
        # both gradients through the one call the step makes (one launch where their tiles share rounds of workgroups)
        ms = timer.run(f"{L['name']}.bwd", lambda: ops.linear_bwd(g, L["x"], L["w"], False), reps)
        rows.append(dict(kernel=f"{L['name']}.dgrad+wgrad", M=M, N=N, K=K, ms=round(ms, 4),
                         tflops_both=round(4.0 * M * N * K / ms / 1e9, 1)))
        if L["epi"] == ops.EPI_SWIGLU:
            ms = timer.run(f"{L['name']}.swiglu_bwd", lambda: ops.activation_bwd(L["dy"], y, ops.EPI_SWIGLU), reps)
            rows.append(dict(kernel=f"{L['name']}.swiglu_bwd", ms=round(ms, 4),
                             gbs=round((M * N // 2 * 2 + 2 * M * N * 2) / ms / 1e6, 1)))
    return rows


def cpu_baseline(sample_tokens):
    """The oracle (reference op order, torch fp32) on `sample_tokens` tokens of the Llama-3-8B workload."""
    from oracle import tp_reference as R
    # threads: this process's CPU share (affinity), not more than the OpenMP setting of the environment
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        cores = os.cpu_count() or 1
    if os.environ.get("OMP_NUM_THREADS", "").isdigit():
        cores = max(1, min(cores, int(os.environ["OMP_NUM_THREADS"])))
    torch.set_num_threads(cores)
    M = sample_tokens
    flops = 0.0
    layers = []
    for i, (name, K, N, epi) in enumerate(LLAMA8B):
        x = torch.randn(M, K, generator=gen(20 + 10 * i))
        w = torch.randn(N, K, generator=gen(21 + 10 * i)) * 0.02
        dy = torch.randn(M, N // 2 if epi == "swiglu" else N, generator=gen(22 + 10 * i))
        layers.append((x, w, dy, epi))
        flops += 6.0 * M * K * N

    def step():
        for x, w, dy, epi in layers:
            y, _ = R.column_parallel_linear_forward(x, w, None)
            g = dy
            if epi == "swiglu":
                R.swiglu(y)
                g = R.swiglu_backward(dy, y)
            R.linear_backward(x, w, g, False)

    step()
    ts = []
    for _ in range(3):
        t0 = time.perf_counter()
        step()
        ts.append(time.perf_counter() - t0)
    sec = statistics.median(ts)
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"value": round(flops / sec / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"llama3-8b QKV+gate/up(SwiGLU)+down fwd+bwd on {M} of 4096 tokens, fp32 torch CPU ops in the "
                      f"reference's order, median of 3 ({sec:.2f} s/step); cpu: {model}"}


def kv_cache_decode(dev, timer, reps, table):
    """Attention over the cache alone (algorithmic bytes: the K and V rows of every cached token, once), and
    whole-model steps (32 blocks + LM head with fused argmax; bytes: all weights + the cached rows)."""
    from merak_amd import ops, _lib
    from merak_amd.inference import LlamaBlockWeights, LlamaDecoder
    n_q, n_kv, d, H, I, layers = 32, 8, 128, 4096, 14336, 32
    res = {}
    st = torch.cuda.current_stream().cuda_stream
    att = {}
    for B, L in ((32, 8192), (8, 8192), (1, 8192)):
        kc = torch.empty(B, n_kv, L, d, dtype=torch.bfloat16, device=dev).normal_()
        vc = torch.empty(B, n_kv, L, d, dtype=torch.bfloat16, device=dev).normal_()
        q = torch.randn(B, n_q, d, device=dev).bfloat16()
        lens = torch.full((B,), L, dtype=torch.int64, device=dev)
        ws = ops.attn_workspace(B, n_q, n_kv, L, dev)
        o = torch.empty_like(q)
        fn = lambda: _lib.check(_lib.lib().mtp_attn_decode(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), lens.data_ptr(),
                                                           o.data_ptr(), ws.data_ptr(), ws.numel(), B, n_q, n_kv, d, L,
                                                           L, d ** -0.5, 1, st), "attn")
        # ten launches per timed region: one launch is shorter than the host's launch path at the small sizes
        ms = timer.run(f"attn.b{B}", lambda: [fn() for _ in range(10)], max(3, reps // 2)) / 10
        by = 2.0 * B * n_kv * L * d * 2
        att[f"B{B}_L{L}"] = {"us": round(ms * 1e3, 1), "GBs": round(by / ms / 1e6, 1),
                             "frac_hbm_peak": round(by / ms / 1e6 / PEAK_HBM_GBS, 4)}
        del kc, vc
    res["attention"] = att
    mk = lambda *shape: torch.empty(*shape, device=dev).normal_(0, 0.02).bfloat16()
    ones = torch.ones(H, device=dev).bfloat16()
    blocks = [LlamaBlockWeights(ones, mk((n_q + 2 * n_kv) * d, H), mk(H, n_q * d), ones, mk(2 * I, H), mk(H, I))
              for _ in range(layers)]
    wbytes = sum(t.numel() * 2 for b in blocks for t in (b.qkv, b.o, b.gate_up, b.down)) + table.numel() * 2
    for B, L in ((1, 2048), (8, 2048), (32, 2048), (32, 8192)):
        dec = LlamaDecoder(table, blocks, ones, table, n_q, n_kv, d, 1e-5, 500000.0, None, L + 8, B)
        for c in dec.k_cache + dec.v_cache:
            c.normal_()
        tok = torch.randint(0, table.shape[0], (B,), device=dev)

        def one():
            dec.lens.fill_(L)
            dec.host_len_bound = L
            dec.step(tok)

        ms = timer.run(f"kvdecode.b{B}.l{L}", one, max(3, reps // 4))
        by = wbytes + 2.0 * layers * B * n_kv * L * d * 2
        res[f"model_B{B}_L{L}"] = {"ms_per_token_step": round(ms, 3), "tokens_per_s": round(B / ms * 1e3, 1),
                                   "GBs": round(by / ms / 1e6, 1), "frac_hbm_peak": round(by / ms / 1e6 / PEAK_HBM_GBS, 4)}
        if B == 1:
            # host wall clock per token, launches from Python against one HIP graph replay
            def wall(n=20):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(n):
                    one()
                torch.cuda.synchronize()
                return (time.perf_counter() - t0) / n * 1e3
            eager_ms = wall()
            dec.lens.fill_(L)
            dec.host_len_bound = L
            dec.capture()
            graph_ms = wall()
            res[f"model_B{B}_L{L}"].update({"wall_ms_python_launches": round(eager_ms, 3),
                                            "wall_ms_hip_graph": round(graph_ms, 3),
                                            "tokens_per_s_hip_graph_wall": round(B / graph_ms * 1e3, 1)})
        del dec
    return res


def secondary(dev, timer, reps, with_cpu):
    from merak_amd import ops, _lib
    from oracle import tp_reference as R
    out = {}
    # --- vocab cross entropy, Llama-3 vocabulary, 8192 tokens, bf16, 5% labels = -100
    n, v = 8192, 128256
    g = torch.Generator(device=dev).manual_seed(1238)
    logits = torch.empty(n, v, dtype=torch.bfloat16, device=dev).normal_(generator=g)
    tgt = torch.randint(0, v, (n,), generator=gen(4))
    tgt[torch.randperm(n, generator=gen(5))[: n // 20]] = -100
    tgt = tgt.to(dev)
    go = torch.full((n,), 1.0 / n, device=dev)
    f_ms = timer.run("ce.fwd", lambda: ops.vocab_ce_fwd(logits, tgt, 0), reps)
    loss, m, s, _ = ops.vocab_ce_fwd(logits, tgt, 0)
    work = logits.clone()
    b_ms = timer.run("ce.bwd", lambda: ops.vocab_ce_bwd_(work, tgt, m, s, go, 0), reps)
    nbytes = n * v * 2
    # Algorithmic traffic of forward + backward: three passes over the logits (read; read + write).  The two-launch
    # path (the reference's own API: forward, later backward) moves exactly those; the one-launch kernel moves two
    # (one read, one write), so its rate is quoted by the bytes it moves and never divided into the three-pass count.
    out["vocab_ce_c4"] = {
        "shape": [n, v], "dtype": "bf16", "fwd_us": round(f_ms * 1e3, 1), "bwd_us": round(b_ms * 1e3, 1),
        "fwd_GBs": round(nbytes / f_ms / 1e6, 1), "bwd_GBs": round(2 * nbytes / b_ms / 1e6, 1),
        "fwd_bwd_GBs": round(3 * nbytes / (f_ms + b_ms) / 1e6, 1),
        "frac_hbm_peak": round(3 * nbytes / (f_ms + b_ms) / 1e6 / PEAK_HBM_GBS, 4)}
    # forward+backward in one launch (what mpu.vocab_loss_fn runs): one read + one write of the logits
    o_ms = timer.run("ce.fwd_bwd", lambda: ops.vocab_ce_fwd_bwd_(work, tgt, 0, None, 1.0 / n), reps)
    out["vocab_ce_c4"].update({
        "one_launch_us": round(o_ms * 1e3, 1), "one_launch_hbm_GBs": round(2 * nbytes / o_ms / 1e6, 1),
        "one_launch_frac_hbm_peak": round(2 * nbytes / o_ms / 1e6 / PEAK_HBM_GBS, 4),
        "one_launch_speedup_over_two_launches": round((f_ms + b_ms) / o_ms, 3),
        "note": "fwd_bwd_GBs / frac_hbm_peak: the two launches of the reference's own API, three passes moved and "
                "counted; one_launch_*: forward+backward in one kernel, two passes moved and counted"})
    # What this board moves when a plain copy kernel reads and rewrites the same 2.1 GB in place (the backward's
    # memory pattern with no arithmetic), and when it copies them to a second buffer: the ceiling the backward and
    # the one-launch kernel stand against.
    st = torch.cuda.current_stream().cuda_stream
    nb16 = nbytes // 16 * 16
    ip_ms = timer.run("ce.copy_in_place", lambda: _lib.check(_lib.lib().mtp_stream_copy(work.data_ptr(), work.data_ptr(), nb16, st), "copy"), reps)
    other = torch.empty_like(work)
    cp_ms = timer.run("ce.copy", lambda: _lib.check(_lib.lib().mtp_stream_copy(work.data_ptr(), other.data_ptr(), nb16, st), "copy"), reps)
    del other
    out["vocab_ce_c4"].update({
        "copy_in_place_same_bytes_us": round(ip_ms * 1e3, 1), "copy_in_place_GBs": round(2 * nb16 / ip_ms / 1e6, 1),
        "copy_to_second_buffer_us": round(cp_ms * 1e3, 1), "copy_to_second_buffer_GBs": round(2 * nb16 / cp_ms / 1e6, 1),
        "bwd_rate_over_copy_in_place": round(ip_ms / b_ms, 4)})
    cpu_rows = 64
    cpu_sample = (logits[:cpu_rows].cpu(), tgt[:cpu_rows].cpu(), go[:cpu_rows].cpu()) if with_cpu else None
    del work
    # --- GPT-2 vocabulary fp32 (config 1)
    n1, v1 = 8192, 50257
    lg1 = torch.empty(n1, v1, device=dev).normal_(generator=g)
    t1 = torch.randint(0, v1, (n1,), generator=gen(6)).to(dev)
    f1 = timer.run("ce1.fwd", lambda: ops.vocab_ce_fwd(lg1, t1, 0), reps)
    _, m1, s1, _ = ops.vocab_ce_fwd(lg1, t1, 0)
    b1 = timer.run("ce1.bwd", lambda: ops.vocab_ce_bwd_(lg1, t1, m1, s1, go, 0), reps)
    o1 = timer.run("ce1.fwd_bwd", lambda: ops.vocab_ce_fwd_bwd_(lg1, t1, 0, None, 1.0 / n1), reps)
    out["vocab_ce_c1"] = {"shape": [n1, v1], "dtype": "f32", "fwd_us": round(f1 * 1e3, 1), "bwd_us": round(b1 * 1e3, 1),
                          "fwd_bwd_GBs": round(3 * n1 * v1 * 4 / (f1 + b1) / 1e6, 1),
                          "frac_hbm_peak": round(3 * n1 * v1 * 4 / (f1 + b1) / 1e6 / PEAK_HBM_GBS, 4),
                          "one_launch_us": round(o1 * 1e3, 1), "one_launch_hbm_GBs": round(2 * n1 * v1 * 4 / o1 / 1e6, 1)}
    del lg1
    # --- embedding gather
    h = 4096
    table = torch.empty(v, h, dtype=torch.bfloat16, device=dev).normal_(0, 0.02, generator=g)
    ids = torch.randint(0, v, (n,), generator=gen(7)).to(dev)
    e_ms = timer.run("emb", lambda: ops.embedding_gather(ids, table, 0, v), reps)
    out["embedding_c4"] = {"rows": n, "dim": h, "us": round(e_ms * 1e3, 1),
                           "GBs": round((2 * n * h * 2 + n * 8) / e_ms / 1e6, 1)}
    # dense gradient: the scatter itself (into an existing table) and with the zero fill of the [V, H] table
    dout = torch.empty(n, h, dtype=torch.bfloat16, device=dev).normal_(generator=g)
    dtab = torch.zeros(v, h, dtype=torch.bfloat16, device=dev)
    eb_ms = timer.run("emb.bwd", lambda: ops.embedding_bwd(ids, dout, v, 0, v, out=dtab), reps)
    ebz_ms = timer.run("emb.bwd0", lambda: ops.embedding_bwd(ids, dout, v, 0, v), max(3, reps // 4))
    out["embedding_c4"].update({"bwd_scatter_us": round(eb_ms * 1e3, 1), "bwd_with_zero_fill_us": round(ebz_ms * 1e3, 1)})
    # the same scatter when half of the batch is one padding id, and when every id is the same
    ids_pad = ids.clone()
    ids_pad[torch.randperm(n, generator=gen(13))[: n // 2].to(dev)] = 2
    ids_one = torch.full_like(ids, 7)
    for nm, ii in (("bwd_scatter_half_padded_us", ids_pad), ("bwd_scatter_one_id_us", ids_one)):
        out["embedding_c4"][nm] = round(timer.run("emb." + nm, lambda: ops.embedding_bwd(ii, dout, v, 0, v, out=dtab), reps) * 1e3, 1)
    del dout, dtab
    # --- LM head + cross entropy at the C4 shape: full logits vs one chunk of rows at a time
    from merak_amd import mpu
    hid = torch.empty(n, h, dtype=torch.bfloat16, device=dev).normal_(generator=g)
    def head_ce_unfused():
        lg, _ = ops.linear_fwd(hid, table, None, ops.EPI_NONE)
        ops.vocab_ce_fwd_bwd_(lg, tgt, 0, None, 1.0 / n)
        ops.linear_dgrad(lg, table)
        ops.linear_wgrad(lg, hid, False)
    def head_ce_chunked():
        hh = hid.detach().requires_grad_(True)
        ww = table.detach().requires_grad_(True)
        mpu.lm_head_cross_entropy(hh, ww, tgt, chunk_rows=4096).mean().backward()
    hc = {}
    for nm, fn in (("full_logits", head_ce_unfused), ("chunks_of_4096_rows", head_ce_chunked)):
        torch.cuda.synchronize(); torch.cuda.empty_cache(); torch.cuda.reset_peak_memory_stats()
        base = torch.cuda.memory_allocated()
        ms = timer.run(f"headce.{nm}", fn, max(3, reps // 4))
        hc[nm] = {"ms": round(ms, 3), "peak_extra_GB": round((torch.cuda.max_memory_allocated() - base) / 1e9, 2),
                  "tflops": round(6.0 * n * h * v / ms / 1e9, 1)}
    out["lm_head_plus_ce_c4"] = hc
    del hid
    # --- decode step: QKV, gate/up+SwiGLU, down, LM head + argmax (the table doubles as the LM head)
    mk = lambda nn, kk: torch.empty(nn, kk, device=dev).normal_(0, 0.02, generator=g).bfloat16()
    wq, wg, wd = mk(6144, 4096), mk(2 * 14336, 4096), mk(4096, 14336)
    wbytes = (wq.numel() + wg.numel() + wd.numel() + table.numel()) * 2
    from merak_amd.inference import DecodeStep
    step = DecodeStep(wq, wg, wd, table)
    dec = {}
    for b in (1, 8, 32):
        x = torch.randn(b, 4096, generator=gen(8)).bfloat16().to(dev)
        ms = timer.run(f"decode.b{b}", lambda: step(x), reps)
        lm = timer.run(f"lmhead.b{b}", lambda: ops.gemv_argmax(x, table, step.workspace), reps)
        dec[f"B{b}"] = {"us_per_step": round(ms * 1e3, 1), "tokens_per_s": round(b / ms * 1e3, 1),
                        "GBs": round(wbytes / ms / 1e6, 1), "frac_hbm_peak": round(wbytes / ms / 1e6 / PEAK_HBM_GBS, 4),
                        "lm_head_argmax_us": round(lm * 1e3, 1), "lm_head_GBs": round(table.numel() * 2 / lm / 1e6, 1)}
    # sampling tail on materialised LM-head logits (temperature 0.8, top-k 50, top-p 0.95), kernel only
    smp = {}
    for b in (1, 8, 32):
        lg = torch.empty(b, v, device=dev).normal_(0, 2.5, generator=g).bfloat16()
        u = torch.rand(b, device=dev)
        tok = torch.empty(b, dtype=torch.int64, device=dev)
        st = torch.cuda.current_stream().cuda_stream
        ws = torch.empty(int(_lib.lib().mtp_sample_workspace_bytes(b)), dtype=torch.uint8, device=dev)
        fn = lambda: _lib.check(_lib.lib().mtp_sample_top_k_top_p(lg.data_ptr(), 1, b, v, 0.8, 50, 0.95, u.data_ptr(),
                                                                  tok.data_ptr(), None, ws.data_ptr(), ws.numel(), st),
                                "sample")
        smp[f"B{b}_us"] = round(timer.run(f"sample.b{b}", fn, reps) * 1e3, 1)
    dec["sample_top_k_top_p"] = smp
    out["decode_c5"] = dec
    del wq, wg, wd, step
    # --- the same step with attention over a key/value cache: one Llama-3-8B position per sequence
    out["decode_with_kv_cache_llama8b"] = kv_cache_decode(dev, timer, reps, table)
    del table
    # --- Llama-70B tp=8 shard shapes
    w3 = build_linear_workload(dev, LLAMA70B_TP8, 8192, 100)
    ms3 = timer.run("c3.step", lambda: linear_step(w3), max(3, reps // 2))
    fl3 = sum(L["flops"] for L in w3)
    out["linear_c3_llama70b_tp8"] = {"ms_per_step": round(ms3, 4), "tflops": round(fl3 / ms3 / 1e9, 1),
                                     "frac_bf16_peak": round(fl3 / ms3 / 1e9 / PEAK_BF16_TFLOPS, 4),
                                     "tokens": 8192, "kernels": per_kernel(w3, timer, max(3, reps // 2))}
    del w3
    # --- GPT-2-small fp32 (config 1): Column 768->3072 bias+GeLU, Row 3072->768 bias
    M1 = 8192
    x1 = torch.randn(M1, 768, generator=gen(9)).to(dev)
    wc = (torch.randn(3072, 768, generator=gen(10)) * 0.02).to(dev)
    wr = (torch.randn(768, 3072, generator=gen(11)) * 0.02).to(dev)
    bc, br = torch.zeros(3072, device=dev), torch.zeros(768, device=dev)
    dy1 = torch.randn(M1, 768, generator=gen(12)).to(dev)

    def c1_step():
        y, a = ops.linear_fwd(x1, wc, bc, ops.EPI_BIAS_GELU)
        o, _ = ops.linear_fwd(a, wr, br, ops.EPI_BIAS)
        da = ops.linear_dgrad(dy1, wr)
        ops.linear_wgrad(dy1, a, True)
        dpre = ops.activation_bwd(da, y, ops.EPI_BIAS_GELU)
        ops.linear_dgrad(dpre, wc)
        ops.linear_wgrad(dpre, x1, True)

    ms1 = timer.run("c1.step", c1_step, max(3, reps // 2))
    fl1 = 2 * 6.0 * M1 * 768 * 3072
    out["linear_c1_gpt2_fp32"] = {"ms_per_step": round(ms1, 4), "tflops": round(fl1 / ms1 / 1e9, 1),
                                  "frac_f32_peak": round(fl1 / ms1 / 1e9 / PEAK_F32_TFLOPS, 4)}
    # --- what this GPU does on a plain copy and on a register-resident MFMA loop
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    st = torch.cuda.current_stream().cuda_stream
    c_ms = timer.run("copy", lambda: _lib.check(_lib.lib().mtp_stream_copy(src.data_ptr(), dst.data_ptr(), src.numel(), st), "copy"), reps)
    src_bytes = src.numel()
    sink = torch.empty(64 * 4096, device=dev)
    iters = 8192
    # register-resident MFMA loop, no memory traffic at all: what the matrix cores sustain under the power
    # limit with smooth operands and with operands of random sign and mantissa (what N(0,1) data looks like)
    p_ms = timer.run("mfma", lambda: _lib.check(_lib.lib().mtp_mfma_peak(sink.data_ptr(), 4096, iters, 0, st), "peak"), 3)
    r_ms = timer.run("mfma_r", lambda: _lib.check(_lib.lib().mtp_mfma_peak(sink.data_ptr(), 4096, iters, 1, st), "peak"), 3)
    del src, dst
    out["vendor_blas_same_gemms"] = vendor_compare(dev, reps)
    gi = 128 * 1024
    g0 = timer.run("mfma_g0", lambda: _lib.check(_lib.lib().mtp_mfma_peak_gemm_loop(sink.data_ptr(), 1024, gi, 0, st), "peak"), 3)
    g1 = timer.run("mfma_g1", lambda: _lib.check(_lib.lib().mtp_mfma_peak_gemm_loop(sink.data_ptr(), 1024, gi, 1, st), "peak"), 3)
    out["device_reference"] = {"copy_1GiB_GBs_read_plus_write": round(2 * src_bytes / c_ms / 1e6, 1),
                               "mfma_32x32x16_4acc_tflops_smooth_operands": round(4096 * iters * 32 * 32 * 16 * 2 / p_ms / 1e9, 1),
                               "mfma_32x32x16_4acc_tflops_random_operands": round(4096 * iters * 32 * 32 * 16 * 2 / r_ms / 1e9, 1),
                               "mfma_16x16x32_gemm_loop_tflops_smooth_operands": round(1024 * gi * 16 * 16 * 32 * 2 / g0 / 1e9, 1),
                               "mfma_16x16x32_gemm_loop_tflops_random_operands": round(1024 * gi * 16 * 16 * 32 * 2 / g1 / 1e9, 1)}
    # The CPU leg comes last: it sets the host thread count and builds a process group, and with those in place the
    # host side of the autograd-driven measurements above (LM head + cross entropy in chunks) runs 25 % slower.
    if with_cpu:
        # the reference's multi-pass algorithm with its three all-reduces on a 1-rank gloo group (CPU tensors)
        import torch.distributed as dist
        rows = cpu_rows
        xs, ts, gs = cpu_sample
        cores = os.cpu_count() or 1
        try:
            cores = len(os.sched_getaffinity(0))
        except AttributeError:
            pass
        torch.set_num_threads(cores)
        made = False
        # gloo announces its connections on stdout, which carries this script's one JSON line: send the
        # process's stdout to stderr while the group is built
        sys.stdout.flush()
        keep = os.dup(1)
        os.dup2(2, 1)
        try:
            if not dist.is_initialized():
                dist.init_process_group("gloo", init_method="tcp://127.0.0.1:29577", rank=0, world_size=1)
                made = True
            grp = dist.new_group([0], backend="gloo")
        finally:
            os.dup2(keep, 1)
            os.close(keep)
        t0 = time.perf_counter()
        for _ in range(3):
            xx = xs.float().clone()
            loss_c, sm, mask, mt = R.vocab_parallel_cross_entropy_forward(xx, ts, 0, v, group=grp)
            R.vocab_parallel_cross_entropy_backward(sm, mask, mt, gs)
        sec = (time.perf_counter() - t0) / 3
        if made:
            dist.destroy_process_group()
        out["vocab_ce_c4"]["cpu_port_GBs"] = round(3 * rows * v * 2 / sec / 1e9, 2)
        out["vocab_ce_c4"]["cpu_cores"] = cores
        out["vocab_ce_c4"]["cpu_sample"] = (f"{rows} of {n} rows, the reference's multi-pass algorithm in fp32 with its "
                                            f"three all-reduces on a 1-rank gloo group, {cores} cores")
    return out


def vendor_compare(dev, reps, kinds=("fwd", "dgrad", "wgrad")):
    """The plain GEMMs of the headline step through the vendor library (torch.matmul, i.e. hipBLASLt) and through
    this library on the same operands, launch by launch in turn so that both see the same clocks: what the
    board's power management grants depends on what ran in the milliseconds before."""
    from merak_amd import ops
    w2 = build_linear_workload(dev, LLAMA8B, 4096, 100)
    rows, v_sum, o_sum, fl_sum = {}, 0.0, 0.0, 0.0
    for L in w2:
        gdy = torch.randn(L["M"], L["N"], device=dev).bfloat16()
        pairs = (("fwd", lambda: torch.nn.functional.linear(L["x"], L["w"]), lambda: ops.linear_fwd(L["x"], L["w"], None, ops.EPI_NONE)),
                 ("dgrad", lambda: gdy @ L["w"], lambda: ops.linear_dgrad(gdy, L["w"])),
                 ("wgrad", lambda: gdy.t() @ L["x"], lambda: ops.linear_wgrad(gdy, L["x"], False)))
        for kind, vendor_fn, own_fn in pairs:
            if kind not in kinds:
                continue
            vendor_fn(), own_fn()
            torch.cuda.synchronize()
            ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(2 * reps)]
            for e0, e1, e2 in ev:
                e0.record(); vendor_fn(); e1.record(); own_fn(); e2.record()
            torch.cuda.synchronize()
            v_ms = statistics.mean(e0.elapsed_time(e1) for e0, e1, _ in ev)
            o_ms = statistics.mean(e1.elapsed_time(e2) for _, e1, e2 in ev)
            fl = 2.0 * L["M"] * L["N"] * L["K"]
            rows[f"{L['name']}.{kind}"] = {"M": L["M"], "N": L["N"], "K": L["K"], "vendor_ms": round(v_ms, 4),
                                           "this_library_ms": round(o_ms, 4), "vendor_tflops": round(fl / v_ms / 1e9, 1),
                                           "this_library_tflops": round(fl / o_ms / 1e9, 1)}
            v_sum, o_sum, fl_sum = v_sum + v_ms, o_sum + o_ms, fl_sum + fl
        del gdy
    return {"vendor_sum_ms": round(v_sum, 4), "vendor_tflops": round(fl_sum / v_sum / 1e9, 1),
            "this_library_sum_ms": round(o_sum, 4), "this_library_tflops": round(fl_sum / o_sum / 1e9, 1),
            "note": "plain GEMMs, alternating launches; the headline step also fuses SwiGLU into gate_up.fwd",
            "per_gemm": rows}


def gemm_loop_parts(dev, reps):
    """Where the time of the 64-deep GEMM loop goes: the gate/up forward launch of the headline step (with the SwiGLU
    epilogue, and as a plain product) timed whole, with its DMA requests answered out of range (instructions issued,
    LDS written, no memory traffic), with no DMA requests at all, with no fragment reads from LDS, and with neither.
    Needs the measurement build of the library (python -m merak_amd.build --measure; MERAK_AMD_LIB points at it):
    the switched-off forms compute wrong results and do not exist in the library that ships."""
    from merak_amd import ops, _lib
    lib = _lib.lib()
    L = build_linear_workload(dev, LLAMA8B, 4096, 20)[1]
    flops = 2.0 * L["M"] * L["N"] * L["K"]
    variants = (("whole", 0), ("dma_answered_out_of_range", 4), ("no_dma_requests", 16), ("no_lds_fragment_reads", 32),
                ("no_dma_requests_no_lds_reads", 48))
    forms = (("swiglu", ops.EPI_SWIGLU), ("plain", ops.EPI_NONE))
    acc = {(f, v): [] for f, _ in forms for v, _ in variants}
    timer = Timer()
    try:
        for _ in range(3):                      # the variants in turn, three times: all see the same clocks
            for v, bits in variants:
                os.environ["MTP_GEMM_DEBUG"] = str(bits)
                lib.mtp_reload_tuning()
                for f, epi in forms:
                    acc[(f, v)].append(timer.run(f"{f}.{v}", lambda: ops.linear_fwd(L["x"], L["w"], None, epi, want_pre=True), reps))
    finally:
        os.environ.pop("MTP_GEMM_DEBUG", None)
        lib.mtp_reload_tuning()
    out = {}
    for f, _ in forms:
        whole = statistics.mean(acc[(f, "whole")])
        out[f] = {v: {"ms": round(statistics.mean(acc[(f, v)]), 4), "tflops_equivalent": round(flops / statistics.mean(acc[(f, v)]) / 1e9, 1),
                      "share_of_whole": round(statistics.mean(acc[(f, v)]) / whole, 4)} for v, _ in variants}
    sink = torch.empty(64 * 1024, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    gi = 128 * 1024
    g1 = timer.run("mfma_g1", lambda: _lib.check(lib.mtp_mfma_peak_gemm_loop(sink.data_ptr(), 1024, gi, 1, st), "peak"), 5)
    out["mfma_16x16x32_gemm_loop_tflops_random_operands"] = round(1024 * gi * 16 * 16 * 32 * 2 / g1 / 1e9, 1)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="headline only (no secondary figures)")
    ap.add_argument("--cpu-tokens", type=int, default=4096,
                    help="tokens of the workload the CPU baseline runs (default: all 4096, about 13 s on 16 cores)")
    ap.add_argument("--only", choices=["gemm-fwd-vs-vendor", "gemm-vs-vendor", "gemm-loop-parts"], default=None,
                    help="launch nothing but the forward GEMMs (or all nine plain GEMMs) of the headline step, each "
                         "through the vendor library and through this one in turn, and print their times: the "
                         "program to put behind `rocprofv3 --pmc ... --` or `--kernel-trace` for a counter comparison; "
                         "gemm-loop-parts: the gate/up forward launch with parts of its main loop switched off "
                         "(measurement build of the library only)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (no collectives, one rank's share "
              "of the tensor-parallel layers per process). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs an MI355X (gfx950) device", file=sys.stderr)
        sys.exit(2)
    from merak_amd import _lib
    _lib.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.only == "gemm-loop-parts":
        if "measure" not in os.environ.get("MERAK_AMD_LIB", ""):
            print("gemm-loop-parts needs the measurement build: python -m merak_amd.build --measure, then "
                  "MERAK_AMD_LIB=merak_amd/lib/libmerak_tp_gfx950_measure.so", file=sys.stderr)
            sys.exit(2)
        print(json.dumps({"mode": args.only, **gemm_loop_parts(dev, max(3, args.steps))}))
        return
    if args.only:
        kinds = ("fwd",) if args.only == "gemm-fwd-vs-vendor" else ("fwd", "dgrad", "wgrad")
        res = vendor_compare(dev, max(3, args.steps), kinds)
        print(json.dumps({"mode": args.only, "launches_per_gemm_and_library": 2 * max(3, args.steps) + 1, **res}))
        return

    M = 4096
    work = build_linear_workload(dev, LLAMA8B, M, 20)
    flops = sum(L["flops"] for L in work)
    for _ in range(args.warmup):
        linear_step(work)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        linear_step(work)
    torch.cuda.synchronize()
    sec = time.perf_counter() - t0
    ms_per_step = sec / args.steps * 1e3
    tflops = flops / (ms_per_step * 1e-3) / 1e12

    timer = Timer()
    reps = max(5, min(20, args.steps))
    kernels = per_kernel(work, timer, reps)
    gemms = [k for k in kernels if "tflops" in k]
    dom = max(gemms, key=lambda k: k["ms"])
    traffic, stamp = measured_traffic()
    roofline = {"bound": "mfma", "kernel": dom["kernel"], "achieved": dom["tflops"], "peak": PEAK_BF16_TFLOPS,
                "unit": "TFLOP/s", "frac": round(dom["tflops"] / PEAK_BF16_TFLOPS, 4),
                "traffic": traffic.get(dom["kernel"]),
                "traffic_source": (f"profiles/hbm_traffic_fetch_write_size.txt, measured at commit {stamp}"
                                   if dom["kernel"] in traffic else None),
                "launch_ms": dom["ms"], "flops_per_launch": 2.0 * dom["M"] * dom["N"] * dom["K"]}
    # what the matrix cores sustain on this board with no memory traffic at all (register-resident MFMA loop on
    # operands of random sign and mantissa): the chip runs against its power limit well below the published peak
    # The ceiling probe is the GEMM's own instruction stream: v_mfma_f32_16x16x32_bf16 on 64 accumulator quads, 32
    # operand fragments walked in the loop's quadrant order, one wave per SIMD, 128 MFMAs per pass, nothing else.
    sink = torch.empty(64 * 4096, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    g_iters = 128 * 1024
    r_ms = timer.run("mfma_g", lambda: _lib.check(_lib.lib().mtp_mfma_peak_gemm_loop(sink.data_ptr(), 1024, g_iters, 1, st),
                                                  "peak"), 12)
    roofline["mfma_loop_random_operands"] = round(1024 * g_iters * 16 * 16 * 32 * 2 / r_ms / 1e9, 1)
    roofline["mfma_loop"] = "v_mfma_f32_16x16x32_bf16, 64 accumulator quads, 1024 waves, register-resident"
    roofline["frac_of_mfma_loop"] = round(dom["tflops"] / roofline["mfma_loop_random_operands"], 4)
    roofline["launch_ms_median"] = round(timer.median[dom["kernel"]], 4)
    del work, sink
    result = {
        "metric": "TP-shard linear fwd+bwd TFLOP/s (% bf16 peak); vocab-CE HBM GB/s",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "llama3-8b single-rank (tp=1) QKV 4096->6144 + gate/up 4096->2x14336 (fused SwiGLU) + "
                               "down 14336->4096, fwd+bwd on 4096 tokens, bf16 / fp32 accumulate",
                   "tokens": M, "flops_per_step": flops},
        "frac_bf16_peak": round(tflops / PEAK_BF16_TFLOPS, 4),
        "roofline": roofline,
        "kernels": kernels,
    }
    if not args.no_extras:
        result["secondary"] = secondary(dev, timer, reps, not args.no_cpu)
        ce = result["secondary"]["vocab_ce_c4"]
        result["vocab_ce_GBs"] = ce["fwd_bwd_GBs"]
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(args.cpu_tokens)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
