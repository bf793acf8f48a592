#!/usr/bin/env python3
"""Benchmark of the calibration-time quantization hot path on one MI355X.

Workload (the fourth of the benchmark configurations, one decoder layer per step): GPTQ W4A16 g128,
activation ordering "static", of the seven Linears of a random-init
Llama-3-8B-shaped decoder layer.  A step is

  Hessian phase : 256 calibration batches x 2048 tokens through GPTQModifier's forward
                  hook for each Linear (q/k/v/o/gate/up on the 4096-wide input, down on
                  the 14336-wide one); the hook stages batches and launches H += 2 X^T X
                  once per --stage-tokens tokens -- 3.21e14 algorithmic FLOP per step
  quantize phase: per Linear  min-max observer -> scales -> diag argsort ->
                  damped Cholesky chain -> GPTQ column loop -> int4 packing

All inputs are resident in HBM before the timed region: one activation stream per distinct
Linear input of the layer (q/k/v share theirs, o_proj has its own, gate/up share theirs, down_proj
has its own).  `value` is the Hessian phase's algorithmic TFLOP/s (2*T*K^2 per Linear per batch)
with one Hessian accumulated per Linear, as the reference does; `quantize_weight_ms_per_linear` is
the second half of the metric.  `shared_input_hessians` repeats the step with
GPTQModifier(share_identical_inputs=True), where q/k/v and gate/up accumulate one Hessian per
shared input (identical results, 3 of the 6 narrow products removed) -- same algorithmic FLOP
count over the shorter time.  Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "llm-compressor_amd"))

HIDDEN, INTER, KV = 4096, 14336, 1024
LINEARS = [  # name, out_features, in_features
    ("q_proj", HIDDEN, HIDDEN),
    ("k_proj", KV, HIDDEN),
    ("v_proj", KV, HIDDEN),
    ("o_proj", HIDDEN, HIDDEN),
    ("gate_proj", INTER, HIDDEN),
    ("up_proj", INTER, HIDDEN),
    ("down_proj", HIDDEN, INTER),
]
GROUP = 128
MFMA_BF16_PEAK_TFLOPS = 2500.0


def dominant_traffic_bytes(tokens_per_launch: int):
    """HBM bytes per launch of the dominant kernel, from the FETCH_SIZE / WRITE_SIZE counter runs whose raw
    averages and calibration are kept next to their summary (profiles/hessian_syrk_k14336_t65536_hbm_traffic.json);
    None when no counter run exists for this launch size or the kernel's source has changed since that run."""
    path = os.path.join(ROOT, "profiles", "hessian_syrk_k14336_t65536_hbm_traffic.json")
    try:
        with open(path) as f:
            rec = json.load(f)
    except OSError:
        return None
    if int(rec.get("tokens_per_launch", -1)) != int(tokens_per_launch) or int(rec.get("K", -1)) != INTER:
        return None
    # the counters were read on one build of the kernel: a figure taken on other source is not reported
    import hashlib

    try:
        with open(os.path.join(ROOT, rec.get("kernel_source", "")), "rb") as f:
            if hashlib.sha256(f.read()).hexdigest() != rec.get("kernel_source_sha256"):
                return None
    except OSError:
        return None
    return float(rec["FETCH_SIZE_avg_per_dispatch"]) * rec["FETCH_SIZE_unit_bytes"] + \
        float(rec["WRITE_SIZE_avg_per_dispatch"]) * rec["WRITE_SIZE_unit_bytes"]


def cpu_baseline(tokens: int):
    """The oracle (a port of the reference's torch CPU path) on a bounded sample of the same workload: one
    warm-up, then the median of three timings for each half of the metric.  Threads: the host's CPU count,
    capped at the 16 cores one GPU's share of the box provides."""
    import statistics

    import torch

    from oracle import gptq as G
    from oracle import observers as O
    from oracle import qformat as F

    host_cpus = os.cpu_count() or 1
    cores = min(host_cpus, 16)
    torch.set_num_threads(cores)
    torch.manual_seed(0)
    K = HIDDEN
    calls = 4
    x = torch.randn(calls, 1, tokens, K).bfloat16()
    H = G.make_empty_hessian(K)
    n = torch.zeros(())
    G.accumulate_hessian(x[0], H, n)  # warm-up
    t_hs = []
    for _ in range(3):
        t0 = time.perf_counter()
        for i in range(calls):
            G.accumulate_hessian(x[i], H, n)
        t_hs.append((time.perf_counter() - t0) / calls)
    t_h = statistics.median(t_hs)
    w = (torch.randn(HIDDEN, K) * 0.02).bfloat16()
    args = F.QArgs(num_bits=4, strategy="group", group_size=GROUP, actorder="weight")
    t_qs = []
    for rep in range(4):  # the first one is the warm-up
        obs = O.Observer("memoryless_minmax", "weight", args)
        t0 = time.perf_counter()
        obs(w)
        G.quantize_weight(w, obs, args, H / n)
        t_qs.append(time.perf_counter() - t0)
    t_q = statistics.median(t_qs[1:])
    return {
        "value": round(2.0 * tokens * K * K / t_h / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": cores,
        "host_cpus": host_cpus,
        "kind": "port",
        "sample": f"median of 3 x ({calls} accumulate_hessian calls of [1,{tokens},{K}] bf16, fp32 GEMM) and median of 3 "
        f"quantize_weight of a {HIDDEN}x{K} Linear (W4A16 g128, actorder static), one warm-up each, {cores} torch threads",
        "quantize_weight_ms_per_linear": round(t_q * 1e3, 1),
    }


def probe_bandwidth(rows_filter=None, reps=20, stack=8):
    """Observer / quantize / pack kernels on a 114688 x 4096 bf16 weight (eight gate/up projections stacked,
    0.94 GB) and the per-token activation kernel on 65536 x 4096 inputs (0.54 GB): algorithmic bytes (one read
    of the input plus one write of the output) over the event-timed launch, against the 8 TB/s HBM peak.

    Cold cache: one launch streams several times the 256 MB last-level cache, consecutive launches read a
    different one of 3 distinct inputs and write an output buffer of their own (the last 3 results are kept
    alive), and a launch lasts 150 us or more, so the host's launch overhead hides behind the queue.
    `rows_filter` (substrings) selects rows, so that a counter run can hold one row per kernel name.
    `stack` = 1 runs the single-Linear size instead (14336 x 4096 weights, 8192 x 4096 activations, 12 distinct
    inputs in rotation): launches of 20-40 us whose event timing includes the host's launch overhead, so their
    durations are read from a kernel trace.  Prints a table."""
    import torch

    from llmcompressor_amd import ops

    NW = 3 if stack > 1 else 12

    def timed(fn, n=reps):
        keep = [None] * NW
        for i in range(3):
            keep[i % NW] = fn(i % NW)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(n):
            keep[i % NW] = fn((i + 3) % NW)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n * 1e-3

    R, K = stack * INTER, HIDDEN
    n = R * K
    NT = 8192 * stack
    ws = [(torch.randn(R, K, device="cuda") * 0.02).bfloat16() for _ in range(NW)]
    xs = [torch.randn(NT, HIDDEN, device="cuda").bfloat16() for _ in range(NW)]
    nx = xs[0].numel()
    rows = []

    def want(name):
        return not rows_filter or any(f in name for f in rows_filter)

    def rep(name, fn, nbytes, n_launch=reps, note=None):
        if not want(name):
            return
        t = timed(fn, n_launch)
        rows.append((name if note is None else name + note(t), t * 1e6, nbytes / t / 1e9, nbytes / t / 8e12))

    dsts = [torch.empty_like(ws[0]) for _ in range(NW)]
    rep("copy (reference), 4 B/elem", lambda i: dsts[i].copy_(ws[i]), 4 * n)
    for g in (16, 32, 128, K):
        rep(f"min-max observer g={g}, 2 B/elem", lambda i, g=g: ops.minmax_groups(ws[i], g), 2 * n)

    def scales(g, fmt, bits, mode=ops.SCALE_PLAIN, with_gs=False):
        out = []
        for w in ws:
            mn, mx = ops.minmax_groups(w, g)
            gs = ops.global_scale_from_stats([(mn, mx)]) if with_gs else None
            sc, _, codes = ops.calculate_qparams(mn, mx, fmt, bits, True, mode, gs, want_codes=mode == ops.SCALE_MXFP4)
            out.append((sc, gs))
        return out

    grp = (1, K // 128, 128)
    if want("int4 g128"):
        sc = scales(128, ops.FMT_INT, 4)
        rep("int4 g128 -> packed int32, 2.5 B/elem",
            lambda i: ops.quantize(ws[i], sc[i][0], None, ops.FMT_INT, 4, *grp, out_mode=ops.OUT_PACKED), 2.5 * n)
        rep("int4 g128 fake-quant, 4 B/elem", lambda i: ops.quantize(ws[i], sc[i][0], None, ops.FMT_INT, 4, *grp), 4 * n)
    if want("fp8 e4m3 per-channel"):
        s8 = scales(K, ops.FMT_FP8, 8)
        rep("fp8 e4m3 per-channel -> bytes, 3 B/elem",
            lambda i: ops.quantize(ws[i], s8[i][0], None, ops.FMT_FP8, 8, 1, 1, 1 << 40, out_mode=ops.OUT_PACKED), 3 * n)
    if want("nvfp4 g16"):
        s4 = scales(16, ops.FMT_FP4, 4, ops.SCALE_NVFP4, with_gs=True)
        rep("nvfp4 g16 -> packed nibbles, 2.5625 B/elem",
            lambda i: ops.quantize(ws[i], s4[i][0], None, ops.FMT_FP4, 4, 1, K // 16, 16, out_mode=ops.OUT_PACKED,
                                   global_scale=s4[i][1]), 2.5625 * n)
    if want("mxfp4 g32"):
        sm = scales(32, ops.FMT_FP4, 4, ops.SCALE_MXFP4)
        rep("mxfp4 g32 -> packed nibbles, 2.53125 B/elem",
            lambda i: ops.quantize(ws[i], sm[i][0], None, ops.FMT_FP4, 4, 1, K // 32, 32, out_mode=ops.OUT_PACKED),
            2.53125 * n)
    rep(f"fp8 dynamic per-token fake-quant [{NT}x4096], 4 B/elem", lambda i: ops.dynamic_per_token_quantize(xs[i]), 4 * nx)
    rep(f"fp8 dynamic per-token -> bytes [{NT}x4096], 3 B/elem",
        lambda i: ops.dynamic_per_token_quantize(xs[i], out_mode=ops.OUT_CODES), 3 * nx)
    # the MSE grid search is arithmetic-bound (every candidate scale re-quantises the group): its figure
    # of merit is candidate evaluations per second; the GB/s column is its one read of the weight
    for name, kw, fmt, bits, g in (("mse observer int4 g128, 20 candidates", {}, ops.FMT_INT, 4, 128),
                                   ("mse observer fp4 g16, 20 candidates", {}, ops.FMT_FP4, 4, 16),
                                   ("mse observer fp4 g16, 80 candidates (maxshrink 0.8, no early stop)",
                                    dict(maxshrink=0.8, patience=100), ops.FMT_FP4, 4, 16)):
        cands = 80 if kw else 20
        rep(name, lambda i, g=g, fmt=fmt, bits=bits, kw=kw: ops.mse_observe_groups(ws[i], g, fmt, bits, True,
                                                                                   ops.SCALE_PLAIN, **kw),
            2 * n, n_launch=5, note=lambda t, c=cands: f": {n * c / t / 1e12:.2f} T element-candidates/s")
    tot = torch.zeros(HIDDEN, dtype=torch.float32, device="cuda")
    rep(f"imatrix hook: sum of squares per channel [{NT}x4096], 2 B/elem", lambda i: ops.sumsq_accumulate_(tot, xs[i]),
        2 * nx)
    imp = torch.rand(K, device="cuda") + 0.1
    rep("imatrix observer int4 g128, 20 candidates, fp32 weighted error",
        lambda i: ops.imatrix_observe_groups(ws[i], 128, ops.FMT_INT, 4, True, importance=imp), 2 * n, n_launch=5,
        note=lambda t: f": {n * 20 / t / 1e12:.2f} T element-candidates/s")
    print(f"| kernel ({R} x {K} bf16 unless noted), cold cache | us | GB/s | of 8 TB/s |")
    print("|---|---|---|---|")
    for name, us, gbs, frac in rows:
        print(f"| {name} | {us:.1f} | {gbs:.0f} | {frac * 100:.1f}% |")


def probe_sparsegpt():
    """SparseGPT on the layer's three Linear shapes (Hessian from 8192 tokens): event-timed factorisation and
    pruning loop per Linear, unstructured 50 % and 2:4, and the CPU oracle on the 4096 x 4096 one.  Prints a table."""
    import torch

    from llmcompressor_amd import ops
    from oracle import sparsegpt as S

    def timed(fn, n=3):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n

    print("| Linear (rows x columns) | factorisation ms | unstructured 50% ms | 2:4 ms | zeros (unstructured) |")
    print("|---|---|---|---|---|")
    keep = None
    for R, K in ((HIDDEN, HIDDEN), (INTER, HIDDEN), (HIDDEN, INTER)):
        torch.manual_seed(0)
        x = torch.randn(8192, K, device="cuda").bfloat16()
        W = (torch.randn(R, K, device="cuda") * 0.02).bfloat16()
        H0 = torch.zeros(K, K, device="cuda")
        ops.hessian_accumulate_(H0, x)
        form = ops.gptq_factor_form(K, 128)  # what sparsify_weight picks at this width
        t_f = timed(lambda: ops.gptq_hinv_(H0.clone(), None, divisor=4.0, form=form))
        U, dead, _ = ops.gptq_hinv_(H0.clone(), None, divisor=4.0, form=form)
        t_u = timed(lambda: ops.sparsegpt_sparsify(W, U, 0.5, dead=dead, form=form))
        t_s = timed(lambda: ops.sparsegpt_sparsify(W, U, 0.5, prune_n=2, prune_m=4, dead=dead, form=form))
        Q, _ = ops.sparsegpt_sparsify(W, U, 0.5, dead=dead, form=form)
        print(f"| {R} x {K} | {t_f:.2f} | {t_u:.2f} | {t_s:.2f} | {(Q == 0).float().mean().item():.4f} |")
        if keep is None:
            keep = (x.cpu(), W.cpu())
    x, W = keep
    torch.set_num_threads(min(os.cpu_count() or 1, 16))
    H, n = S.make_empty_hessian(HIDDEN), 0
    for chunk in x.reshape(4, 2048, HIDDEN):
        H, n = S.accumulate_hessian(chunk, H, n)
    t0 = time.perf_counter()
    S.sparsify_weight(W, H, 0.5)
    print(f"\nCPU oracle, 4096 x 4096 unstructured 50% (factorisation + loop, {torch.get_num_threads()} threads): "
          f"{(time.perf_counter() - t0) * 1e3:.0f} ms")


def probe_chain():
    """The quantize phase's pieces run alone, event-timed: the damped Cholesky chain and the column loop for the
    layer's three Linear shapes (W4A16 g128, static activation ordering), and the fp32 products they are made
    of, through `llmc_sgemm`, at the shapes the K = 14336 chain and the down_proj loop use.  Prints two tables."""
    import torch

    from llmcompressor_amd import ops

    def timed(fn, n=5):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n

    print("| Linear (rows x columns) | Cholesky chain ms | column loop ms | chain, full inverse factor ms | loop on it ms |")
    print("|---|---|---|---|---|")
    for R, K in ((HIDDEN, HIDDEN), (INTER, HIDDEN), (HIDDEN, INTER)):
        torch.manual_seed(0)
        x = torch.randn(16384, K, device="cuda").bfloat16()
        W = (torch.randn(R, K, device="cuda") * 0.02).bfloat16()
        H0 = torch.zeros(K, K, device="cuda")
        ops.hessian_accumulate_(H0, x)
        del x
        perm = torch.argsort(torch.diagonal(H0), descending=True, stable=True).to(torch.int32)
        work = torch.empty_like(H0)

        mn, mx = ops.minmax_groups(W, 128)
        scale, _, _ = ops.calculate_qparams(mn, mx, ops.FMT_INT, 4, True)
        g_idx = (torch.arange(K, dtype=torch.int32, device="cuda") // 128)[perm.long()]
        t_copy = timed(lambda: work.copy_(H0))
        cells = []
        # the form quantize_weight uses at this width (the factor of H outside 512-column diagonal blocks), then the
        # reference's full inverse factor
        for form in (ops.gptq_factor_form(K, 128), ops.FACTOR_INVERSE):
            def chain():
                work.copy_(H0)
                return ops.gptq_hinv_(work, perm, divisor=8.0, form=form)

            t_chain = timed(chain) - t_copy
            U, dead, _ = ops.gptq_hinv_(H0.clone(), perm, divisor=8.0, form=form)
            t_loop = timed(lambda: ops.gptq_quantize(W, U, scale, None, ops.FMT_INT, 4, 1, K // 128, g_idx=g_idx,
                                                     perm=perm, dead=dead, form=form))
            cells += [f"{t_chain:.2f}", f"{t_loop:.2f}"]
            del U
        print(f"| {R} x {K} | " + " | ".join(cells) + " |")
        del H0, work

    print()
    print("| fp32 product C -= A B (llmc_sgemm) | M | N | K | us | TFLOP/s of the non-zero part |")
    print("|---|---|---|---|---|---|")
    cases = [
        ("square", 8192, 8192, 8192, False, 0, 1.0),
        ("inversion, 8192-wide level: L21 X11 (X11 lower triangular)", 6144, 8192, 8192, False, ops.SGEMM_B_LOWER_TRI, 0.5),
        ("inversion, 8192-wide level: X22 T (X22 lower triangular)", 6144, 8192, 6144, False, ops.SGEMM_A_LOWER_TRI, 0.5),
        ("inversion, 4096-wide level: L21 X11", 4096, 4096, 4096, False, ops.SGEMM_B_LOWER_TRI, 0.5),
        ("trailing SYRK of the first 512-wide panel (lower triangle)", 13824, 13824, 512, True, ops.SGEMM_C_LOWER, 0.5),
        ("trailing SYRK, half way", 7168, 7168, 512, True, ops.SGEMM_C_LOWER, 0.5),
        ("column loop: far product of the first group", 4096, 13824, 512, False, 0, 1.0),
        ("column loop: far product, half way", 4096, 7168, 512, False, 0, 1.0),
        ("column loop: product inside a group", 4096, 384, 128, False, 0, 1.0),
    ]
    for name, M, N, Kc, trans_b, flags, frac in cases:
        A = torch.randn(M, Kc, device="cuda")
        B = torch.randn(N, Kc, device="cuda") if trans_b else torch.randn(Kc, N, device="cuda")
        C = torch.zeros(M, N, device="cuda")
        ms = timed(lambda: ops.sgemm_(C, A, B, -1.0, 1.0, trans_b, flags))
        print(f"| {name} | {M} | {N} | {Kc} | {ms * 1e3:.1f} | {2.0 * M * N * Kc * frac / ms / 1e9:.0f} |")
        del A, B, C


def probe_vendor_gemm(tokens=65536):
    """The dominant launch beside the vendor library's bf16 GEMM (through ``torch.matmul``) on the same operands:
    the full product X^T X in the hook's layout (tokens strided), the same with all-zero data (matrix instructions
    on constant operands draw less power, so the chip clocks higher), and a product of the same size whose operands
    are stored with the contraction index contiguous.  Event-timed, mean of 6 launches after 2."""
    import torch

    from llmcompressor_amd import ops

    def timed(fn, n=6):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n

    T, K = tokens, INTER
    x = torch.randn(T, K, device="cuda").bfloat16()
    out = torch.empty(K, K, device="cuda", dtype=torch.bfloat16)
    H = torch.zeros(K, K, device="cuda")
    full = 2.0 * T * K * K
    tiles = (K // 256) * (K // 256 + 1) // 2
    executed = 2.0 * T * tiles * 256 * 256
    rows = []
    for data in ("random", "zero"):
        if data == "zero":
            x.zero_()
        ms = timed(lambda: ops.hessian_accumulate_(H, x))
        rows.append((f"hessian_syrk_kernel, X [{T} x {K}] {data} data (upper-triangular tiles only)", ms, executed))
        ms = timed(lambda: torch.matmul(x.t(), x, out=out))
        rows.append((f"vendor GEMM X^T X on the same tensor, {data} data (all of the product)", ms, full))
    del x, out, H
    K2 = 8192
    xt = torch.randn(K2, T, device="cuda").bfloat16()
    out = torch.empty(K2, K2, device="cuda", dtype=torch.bfloat16)
    ms = timed(lambda: torch.matmul(xt, xt.t(), out=out))
    rows.append((f"vendor GEMM A A^T, A [{K2} x {T}] random data (contraction index contiguous in both operands)",
                 ms, 2.0 * T * K2 * K2))
    x2 = xt.t().contiguous()
    ms = timed(lambda: torch.matmul(x2.t(), x2, out=out))
    rows.append((f"vendor GEMM X^T X, X [{T} x {K2}] random data (the hook's layout)", ms, 2.0 * T * K2 * K2))
    print("| launch | ms | executed bf16 matrix TFLOP/s |")
    print("|---|---|---|")
    for name, ms, flop in rows:
        print(f"| {name} | {ms:.2f} | {flop / ms / 1e9:.0f} |")


def probe_moe(mode="both"):
    """One MoE expert layer (128 experts, hidden 2048, intermediate 768, top-8 routing of 4096 tokens: 384 expert
    Linears) through GPTQModifier W4A16 and NVFP4A16: time of the calibration forward (grouped Hessian launches from
    the hooks) and of the quantisation of the 384 Linears, with lock-step groups and with the per-module path.
    Prints a table."""
    import torch

    from llmcompressor_amd.core import LifecycleCallbacks, active_session
    from llmcompressor_amd.modeling.moe import LinearExperts2D
    from llmcompressor_amd.modifiers.gptq import GPTQModifier

    E, H, I, T, TOPK = 128, 2048, 768, 4096, 8
    torch.manual_seed(0)

    class Layer(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.experts = LinearExperts2D(E, H, I, torch.bfloat16, "cuda")

        def forward(self, x, idx, w):
            return self.experts(x, idx, w)

    class Wrap(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.layers = torch.nn.ModuleList([Layer()])

    model = Wrap()
    x = torch.randn(T, H, device="cuda").bfloat16()
    # a skewed router, as trained ones are: expert e is about e^-1.1 as likely as expert 1
    logits = torch.randn(T, E, device="cuda") + torch.log(1.0 / torch.arange(1, E + 1, device="cuda").float() ** 1.1)
    w, idx = torch.topk(torch.softmax(logits, -1), TOPK, -1)
    from llmcompressor_amd.modeling import moe as moe_module

    with torch.no_grad():  # the propagation pass: nothing observes the experts
        for grouped in (False, True):
            moe_module.GROUPED_FORWARD = grouped
            for _ in range(2):
                model.layers[0](x, idx, w.to(x.dtype))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(5):
                model.layers[0](x, idx, w.to(x.dtype))
            torch.cuda.synchronize()
            print(f"propagation forward, {'grouped launches' if grouped else 'per-expert calls'}: "
                  f"{(time.perf_counter() - t0) / 5 * 1e3:.2f} ms per batch")
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        model.layers[0](x, idx, w.to(x.dtype))
        e0.record()
        model.layers[0](x, idx, w.to(x.dtype))
        e1.record()
        torch.cuda.synchronize()
        print(f"propagation forward, grouped launches, device time between events: {e0.elapsed_time(e1):.2f} ms")
    print("| quantisation of the 384 expert Linears | forward + Hessians ms per batch | quantise ms | ms per Linear |")
    print("|---|---|---|---|")
    from llmcompressor_amd.modeling.moe import moe_calibration_context

    variants = (("W4A16, lock-step groups (default)", 8, "lockstep", "W4A16", False, False),
                ("W4A16, one module at a time, 4 streams", 0, "permodule", "W4A16", False, False),
                ("NVFP4A16, lock-step groups (default)", 8, "lockstep", "NVFP4A16", False, False),
                ("W4A16, lock-step groups, every expert calibrated on all tokens (`moe_calibrate_all_experts`, the "
                 "`oneshot` default)", 8, "lockstep", "W4A16", True, False),
                ("W4A16, lock-step groups, grouped launches in the observed pass too (`moe_grouped_calibration`)",
                 8, "lockstep", "W4A16", False, True),
                ("W4A16, lock-step groups, every expert on all tokens, grouped launches in the observed pass too",
                 8, "lockstep", "W4A16", True, True))
    for label, gmin, key, scheme, all_experts, grouped_cal in variants:
        if mode not in ("both", key):
            continue
        best = None
        for _ in range(3):
            for p in model.parameters():
                if p.dtype == torch.bfloat16:
                    p.data.normal_(0, 0.02)
            mod = GPTQModifier(targets="Linear", scheme=scheme, group_min_modules=gmin)
            s = active_session()
            s.reset()
            s.initialize(model=model, recipe=mod)
            LifecycleCallbacks.calibration_start()
            with torch.no_grad(), moe_calibration_context(all_experts, grouped=grouped_cal):
                model.layers[0](x, idx, w.to(x.dtype))  # first batch: the Hessians are allocated here
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(3):
                    model.layers[0](x, idx, w.to(x.dtype))
            torch.cuda.synchronize()
            t0 = time.perf_counter() - (time.perf_counter() - t0) / 3
            t1 = time.perf_counter()
            LifecycleCallbacks.sequential_epoch_end(modules=list(model.modules()))
            torch.cuda.synchronize()
            t2 = time.perf_counter()
            LifecycleCallbacks.calibration_end()
            s.finalize()
            if best is None or t2 - t1 < best[1]:
                best = (t1 - t0, t2 - t1)
        print(f"| {label} | {best[0] * 1e3:.1f} | {best[1] * 1e3:.1f} | {best[1] * 1e3 / (3 * E):.2f} |")


def probe_oneshot_moe(batches=16, tokens=2048, layers=2, vocab=32000):
    """oneshot() on a transformers Qwen3MoeForCausalLM with `layers` decoder layers of the Qwen3-30B-A3B shape
    (hidden 2048, 32 query and 4 key / value heads of 128, 128 experts of intermediate size 768, top-8 routing,
    random weights, fused expert tensors that oneshot replaces by per-expert Linears), GPTQ W4A16 on attention and
    expert Linears, in the four ways the experts can be calibrated.  Wall time around oneshot."""
    import torch
    import transformers

    from llmcompressor_amd import oneshot
    from llmcompressor_amd.core import active_session
    from llmcompressor_amd.modifiers.gptq import GPTQModifier

    cfg = transformers.Qwen3MoeConfig(hidden_size=2048, intermediate_size=6144, moe_intermediate_size=768,
                                      num_hidden_layers=layers, num_attention_heads=32, num_key_value_heads=4,
                                      head_dim=128, vocab_size=vocab, max_position_embeddings=4096, num_experts=128,
                                      num_experts_per_tok=8, decoder_sparse_step=1, mlp_only_layers=[])
    data = [{"input_ids": torch.randint(0, vocab, (1, tokens))} for _ in range(batches)]
    print(f"| oneshot GPTQ W4A16, {layers} Qwen3-30B-A3B-shaped layers, {batches} x {tokens} tokens | s | "
          "ms per layer and batch | peak GiB |")
    print("|---|---|---|---|")
    for label, kw in (
            ("every expert on every token, per-expert calls (default)", {}),
            ("every expert on every token, `moe_grouped_calibration=True`", {"moe_grouped_calibration": True}),
            ("routed tokens only (`moe_calibrate_all_experts=False`), per-expert calls",
             {"moe_calibrate_all_experts": False}),
            ("routed tokens only, `moe_grouped_calibration=True`",
             {"moe_calibrate_all_experts": False, "moe_grouped_calibration": True})):
        best = None
        for _ in range(2 if layers <= 8 else 1):
            torch.manual_seed(0)
            with torch.device("cuda"):
                model = transformers.Qwen3MoeForCausalLM(cfg).to(torch.bfloat16)
            torch.cuda.synchronize()
            torch.cuda.reset_peak_memory_stats()
            t0 = time.perf_counter()
            oneshot(model=model, dataset=data, recipe=GPTQModifier(targets="Linear", scheme="W4A16",
                                                                   ignore=["lm_head", "re:.*mlp.gate$"]), **kw)
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            peak = torch.cuda.max_memory_allocated() / 2 ** 30
            del model
            active_session().reset()  # the session still refers to the model it compressed
            torch.cuda.empty_cache()
            if best is None or dt < best[0]:
                best = (dt, peak)
        print(f"| {label} | {best[0]:.2f} | {best[0] / layers / batches * 1e3:.1f} | {best[1]:.1f} |")


def probe_oneshot(batches, tokens, layers=2, vocab=32000):
    """oneshot() on a transformers LlamaForCausalLM with `layers` Llama-3-8B-shaped decoder layers (random
    weights), GPTQ W4A16 with the modifier's defaults, `batches` x `tokens` calibration tokens: wall time per layer
    with both passes of the sequential pipeline, the time inside the epoch-end events (observers + quantize_weight),
    peak device memory, and the model's own forward for comparison.  With more than 4 layers (the whole-model run:
    --layers 32 --vocab 128256) only the default configuration runs, once.  Prints a table."""
    import torch
    from transformers import LlamaConfig, LlamaForCausalLM

    from llmcompressor_amd import oneshot
    from llmcompressor_amd.core import LifecycleCallbacks
    from llmcompressor_amd.modifiers.gptq import GPTQModifier

    whole = layers > 4
    cfg = LlamaConfig(hidden_size=HIDDEN, intermediate_size=INTER, num_hidden_layers=layers, num_attention_heads=32,
                      num_key_value_heads=8, vocab_size=vocab, max_position_embeddings=max(4096, tokens))
    torch.manual_seed(0)
    data = [{"input_ids": torch.randint(0, vocab, (1, tokens))} for _ in range(batches)]

    def make():
        with torch.device("cuda"):
            return LlamaForCausalLM(cfg).to(torch.bfloat16)

    model = make()
    with torch.no_grad():
        for rep in range(1 if whole else 2):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for d in data:
                model(d["input_ids"].cuda(), use_cache=False, logits_to_keep=1)
            torch.cuda.synchronize()
            fwd = time.perf_counter() - t0
    del model
    torch.cuda.empty_cache()
    print(f"| oneshot GPTQ W4A16, {layers} layers of 4096/14336, vocabulary {vocab}, {batches} x {tokens} tokens | s | "
          "ms per layer | s inside epoch-end events | peak GiB |")
    print("|---|---|---|---|---|")
    print(f"| model forward alone, one pass over the data (embedding included, lm_head on the last token) | {fwd:.2f} | "
          f"{fwd / layers * 1e3:.0f} | | |")
    variants = [("Hessian launches of 65536 staged tokens (default)", 65536, True),
                ("the same with `propagate_error=False`: the next layer calibrated on the uncompressed layer's "
                 "outputs, one pass per layer", 65536, False)]
    if not whole:
        variants.append(("one Hessian launch per hook call", 0, True))
    raw_end = LifecycleCallbacks.sequential_epoch_end
    for label, stage, propagate in variants:
        best = None
        for rep in range(1 if whole else 2):
            model = make()
            spent = [0.0]

            def timed_end(*args, **kw):
                torch.cuda.synchronize()
                t = time.perf_counter()
                out = raw_end(*args, **kw)
                torch.cuda.synchronize()
                spent[0] += time.perf_counter() - t
                return out

            LifecycleCallbacks.sequential_epoch_end = staticmethod(timed_end)
            torch.cuda.reset_peak_memory_stats()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            try:
                oneshot(model=model, dataset=data, propagate_error=propagate,
                        recipe=GPTQModifier(targets="Linear", scheme="W4A16", ignore=["lm_head"],
                                            hessian_batch_tokens=stage))
            finally:
                LifecycleCallbacks.sequential_epoch_end = raw_end
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            peak = torch.cuda.max_memory_allocated() / 2 ** 30
            if best is None or dt < best[0]:
                best = (dt, spent[0], peak)
            del model
            torch.cuda.empty_cache()
        print(f"| {label} | {best[0]:.2f} | {best[0] / layers * 1e3:.0f} | {best[1]:.2f} | {best[2]:.1f} |")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--batches", type=int, default=256, help="calibration batches per step (config: 256)")
    ap.add_argument("--tokens", type=int, default=2048, help="tokens per batch (config: 2048)")
    ap.add_argument("--stage-tokens", type=int, default=65536,
                    help="tokens staged per Hessian launch (GPTQModifier.hessian_batch_tokens; 0 = one launch per batch)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--group-min-modules", type=int, default=None,
                    help="GPTQModifier.group_min_modules of the step (default: the modifier's own)")
    ap.add_argument("--compress-concurrency", type=int, default=None,
                    help="GPTQModifier.compress_concurrency of the step (default: the modifier's own)")
    ap.add_argument("--probe-dominant", type=int, default=0, metavar="N",
                    help="counter runs: launch only the dominant kernel N times (14336-wide Hessian, --stage-tokens "
                    "tokens) and N plain copies of a 1 GiB buffer (the known-size kernel the HBM counters are scaled by)")
    ap.add_argument("--probe-bandwidth", action="store_true",
                    help="print achieved GB/s of the observer / quantize / pack kernels instead of the bench line")
    ap.add_argument("--probe-rows", default="", help="comma-separated substrings: the rows --probe-bandwidth runs")
    ap.add_argument("--probe-reps", type=int, default=20, help="timed launches per row of --probe-bandwidth")
    ap.add_argument("--probe-stack", type=int, default=8,
                    help="--probe-bandwidth: gate/up projections stacked into one weight (1 = the single-Linear size)")
    ap.add_argument("--probe-sparsegpt", action="store_true",
                    help="print SparseGPT timings per Linear shape instead of the bench line")
    ap.add_argument("--moe-mode", choices=("both", "lockstep", "permodule"), default="both",
                    help="which quantisation path --probe-moe runs (one path alone gives a clean kernel profile)")
    ap.add_argument("--probe-oneshot", action="store_true",
                    help="print end-to-end oneshot timings on a transformers Llama with two 8B-shaped layers "
                    "(--batches x --tokens calibration tokens) instead of the bench line")
    ap.add_argument("--layers", type=int, default=2, help="--probe-oneshot: decoder layers of the model (config: 32)")
    ap.add_argument("--vocab", type=int, default=32000, help="--probe-oneshot: vocabulary size (config: 128256)")
    ap.add_argument("--probe-chain", action="store_true",
                    help="time the Cholesky chain, the column loop and their fp32 products alone, print tables")
    ap.add_argument("--probe-oneshot-moe", action="store_true",
                    help="print end-to-end oneshot timings on a transformers Qwen3-MoE with two 30B-A3B-shaped layers "
                    "for the four ways of calibrating the experts")
    ap.add_argument("--moe-batches", type=int, default=16, help="--probe-oneshot-moe: calibration batches of --tokens tokens")
    ap.add_argument("--probe-vendor-gemm", action="store_true",
                    help="time the dominant launch beside the vendor library's bf16 GEMM on the same operands")
    ap.add_argument("--probe-product", type=int, default=0, metavar="N",
                    help="counter runs: launch only the split fp32 product C -= A B of 8192^3 N times through "
                    "llmc_sgemm (with --probe-trans-b: C -= A B^T)")
    ap.add_argument("--probe-trans-b", action="store_true", help="--probe-product: B is stored transposed")
    ap.add_argument("--probe-moe", action="store_true",
                    help="print the timings of one 128-expert MoE layer through GPTQModifier instead of the bench line")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus must be 1 (no multi-GPU figure is produced)", file=sys.stderr)
        sys.exit(2)

    import torch

    from llmcompressor_amd import ops
    from llmcompressor_amd.compressors import compress_module
    from llmcompressor_amd.core import LifecycleCallbacks, active_session
    from llmcompressor_amd.modifiers.gptq import GPTQModifier

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if a.probe_bandwidth:
        probe_bandwidth([r for r in a.probe_rows.split(",") if r], a.probe_reps, a.probe_stack)
        return
    if a.probe_sparsegpt:
        probe_sparsegpt()
        return
    if a.probe_chain:
        probe_chain()
        return
    if a.probe_moe:
        probe_moe(a.moe_mode)
        return
    if a.probe_oneshot_moe:
        probe_oneshot_moe(a.moe_batches, a.tokens, a.layers, a.vocab)
        return
    if a.probe_vendor_gemm:
        probe_vendor_gemm(a.stage_tokens or 65536)
        return
    if a.probe_product:
        n = 8192
        A, Bm = torch.randn(n, n, device=dev), torch.randn(n, n, device=dev)
        C = torch.zeros(n, n, device=dev)
        for _ in range(a.probe_product):
            ops.sgemm_(C, A, Bm, -1.0, 1.0, a.probe_trans_b, 0)
        torch.cuda.synchronize()
        print(f"probe: {a.probe_product} x llmc_sgemm {n}^3, B {'transposed' if a.probe_trans_b else 'as stored'}")
        return
    if a.probe_oneshot:
        probe_oneshot(a.batches, a.tokens, a.layers, a.vocab)
        return
    if a.probe_dominant:
        from llmcompressor_amd import ops

        # the launch the bench's hook path makes: the batches of one staging period, each in its own buffer
        nseg = max(1, (a.stage_tokens or a.tokens) // a.tokens)
        x = torch.randn(nseg, a.tokens, INTER, device=dev).bfloat16()
        H = torch.zeros(INTER, INTER, device=dev)
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(a.probe_dominant):
            ops.hessian_accumulate_segments_(H, [x[i] for i in range(nseg)])
            dst.copy_(src)
        torch.cuda.synchronize()
        print(f"probe: {a.probe_dominant} x hessian [{nseg}x{a.tokens}x{INTER}] + {a.probe_dominant} x copy of {src.numel() * 4} bytes")
        return
    B, T = a.batches, a.tokens
    gen = torch.Generator(device=dev).manual_seed(0)

    class Layer(torch.nn.Module):  # the seven Linears of one decoder layer (no forward needed here)
        def __init__(self):
            super().__init__()
            for name, r, k in LINEARS:
                setattr(self, name, torch.nn.Linear(k, r, bias=False, dtype=torch.bfloat16, device=dev))

    layer = Layer()
    originals = {}
    for name, r, k in LINEARS:
        w = (torch.randn(r, k, device=dev, generator=gen) * 0.02).bfloat16()
        getattr(layer, name).weight.data.copy_(w)
        originals[name] = w
    # calibration activations, resident in HBM: one stream per distinct Linear input
    streams = {"attn_in": HIDDEN, "attn_out": HIDDEN, "mlp_in": HIDDEN, "mlp_mid": INTER}
    xs = {k: torch.empty(B, T, w, dtype=torch.bfloat16, device=dev) for k, w in streams.items()}
    for b in range(B):
        for k, w in streams.items():
            xs[k][b] = torch.randn(T, w, device=dev, generator=gen).bfloat16()
    input_of = {"q_proj": "attn_in", "k_proj": "attn_in", "v_proj": "attn_in", "o_proj": "attn_out",
                "gate_proj": "mlp_in", "up_proj": "mlp_in", "down_proj": "mlp_mid"}

    # time every launch of the dominant kernel (the 14336-wide Hessian) with events on the launch stream
    dom_events = []
    dom_tokens = []
    recording = [False]
    raw_accumulate = ops.hessian_accumulate_

    def timed_accumulate(H, x, **kw):
        if recording[0] and H.shape[0] == INTER:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            out = raw_accumulate(H, x, **kw)
            e1.record()
            dom_events.append((e0, e1))
            dom_tokens.append(x.shape[0])
            return out
        return raw_accumulate(H, x, **kw)

    ops.hessian_accumulate_ = timed_accumulate
    raw_segments = ops.hessian_accumulate_segments_

    def timed_segments(H, xs_, **kw):  # the same kernel, fed the hook's buffers in place (no staging copy)
        if recording[0] and H.shape[0] == INTER and len(xs_) <= ops.SEGMENTS_MAX:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            out = raw_segments(H, xs_, **kw)
            e1.record()
            dom_events.append((e0, e1))
            dom_tokens.append(sum(x.shape[0] for x in xs_))
            return out
        return raw_segments(H, xs_, **kw)

    ops.hessian_accumulate_segments_ = timed_segments

    def step(record: bool, share: bool = False):  # the headline step accumulates one Hessian per module, as the reference does
        for name, r, k in LINEARS:
            getattr(layer, name).weight.data.copy_(originals[name])
        recording[0] = record
        tuning = {}
        if a.group_min_modules is not None:
            tuning["group_min_modules"] = a.group_min_modules
        if a.compress_concurrency is not None:
            tuning["compress_concurrency"] = a.compress_concurrency
        modifier = GPTQModifier(targets="Linear", scheme="W4A16", actorder="static", block_size=128,
                                dampening_frac=0.01, hessian_batch_tokens=a.stage_tokens,
                                share_identical_inputs=share, **tuning)
        session = active_session()
        session.reset()
        session.initialize(model=layer, recipe=modifier)
        LifecycleCallbacks.calibration_start()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        # what the forward hooks do during the calibration pass of this layer
        mods = [(getattr(layer, name), input_of[name]) for name, _, _ in LINEARS]
        for b in range(B):
            args_of = {k: (x[b:b + 1],) for k, x in xs.items()}
            for mod, stream in mods:
                modifier.calibrate_module(mod, args_of[stream], None)
        for m in list(modifier._num_samples):
            modifier._flush(m)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        # epoch end: observers -> qparams -> Cholesky chain -> column loop, then pack
        LifecycleCallbacks.sequential_epoch_end(modules=list(layer.modules()))
        out = {name: compress_module(getattr(layer, name)) for name, _, _ in LINEARS}
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        LifecycleCallbacks.calibration_end()
        session.finalize()
        recording[0] = False
        return t1 - t0, t2 - t1, out

    for _ in range(a.warmup):
        step(False)
    th = tq = 0.0
    torch.cuda.synchronize()
    wall0 = time.perf_counter()
    for _ in range(a.steps):
        h, q, out = step(True)
        th += h
        tq += q
    torch.cuda.synchronize()
    wall = time.perf_counter() - wall0

    # the same step with one Hessian per shared input (results identical, checked below)
    sh_h = sh_q = 0.0
    for _ in range(a.steps):
        h, q, out_shared = step(False, share=True)
        sh_h += h
        sh_q += q
    same = all(torch.equal(out[n][k], out_shared[n][k]) for n in out for k in out[n])

    flop_step = sum(2.0 * T * k * k for _, _, k in LINEARS) * B
    value = flop_step * a.steps / th / 1e12
    dom_ms = sum(e0.elapsed_time(e1) for e0, e1 in dom_events) / max(1, len(dom_events))
    dom_T = sum(dom_tokens) / max(1, len(dom_tokens))
    dom_flop = 2.0 * dom_T * INTER * INTER
    achieved = dom_flop / (dom_ms * 1e-3) / 1e12
    nb = (INTER + 255) // 256
    dom_exec_flop = 2.0 * dom_T * 256 * 256 * (nb * (nb + 1) // 2)
    rec = {
        "metric": "GPTQ quantize_weight ms/Linear + Hessian TFLOP/s, Llama-3-8B shapes, W4A16 g128",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": round(wall / a.steps * 1e3, 2),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "configs[3]: sequential GPTQ W4A16 g128 actorder=static, one Llama-3-8B-shaped decoder layer "
            f"per step ({B} batches x {T} tokens, 7 Linears: Hessians 6x4096^2 + 14336^2, then quantize_weight + pack)",
            "batches": B,
            "tokens": T,
            "hessian_tokens_per_launch": int(dom_T),
        },
        "quantize_weight_ms_per_linear": round(tq / a.steps / len(LINEARS) * 1e3, 3),
        "hessian_phase_ms_per_step": round(th / a.steps * 1e3, 2),
        "hessian_algorithmic_flop_per_step": flop_step,
        "shared_input_hessians": {
            "value": round(flop_step * a.steps / sh_h / 1e12, 2),
            "unit": "TFLOP/s",
            "hessian_phase_ms_per_step": round(sh_h / a.steps * 1e3, 2),
            "quantize_weight_ms_per_linear": round(sh_q / a.steps / len(LINEARS) * 1e3, 3),
            "packed_weights_identical": bool(same),
        },
        "roofline": {
            "kernel": "hessian_syrk_kernel<256> (down_proj Hessian, %d tokens per launch, K=%d)" % (int(dom_T), INTER),
            "bound": "mfma",
            "achieved": round(achieved, 2),
            "peak": MFMA_BF16_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 4),
            # the kernel executes the upper-triangular 256-wide tiles only and mirrors them: what the matrix
            # cores actually do per launch, next to the algorithmic figure of the reference's full GEMM
            "executed_tflops": round(dom_exec_flop / (dom_ms * 1e-3) / 1e12, 2),
            "executed_frac": round(dom_exec_flop / (dom_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
            "traffic": dominant_traffic_bytes(int(dom_T)),
            "algorithmic_hbm_bytes": 2.0 * dom_T * INTER + 8.0 * INTER * INTER,
            "avg_launch_ms": round(dom_ms, 4),
            "launches_timed": len(dom_events),
        },
    }
    if not a.no_cpu_baseline:
        rec["cpu_baseline"] = cpu_baseline(T)
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
