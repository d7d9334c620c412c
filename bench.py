#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X: beam-12 decoding of the 4+4-layer, 1000-hidden,
30k-vocabulary encoder-decoder with local-p attention and input feeding (BASELINE.json configs[2]).

One "step" = one pass of the hot path over 64 synthetic source sentences: encoder, every decoder
step with on-device top-k / merge / state gather, hypothesis read-back.  The sentences of all
`steps` are handed over as ONE list and decoded 64 at a time with every one of the 768 beam columns
busy in every step of the search (a finished sentence's columns go to the next sentence of the
list: lnmt_decode_stream, the driver Dispatcher::Decoding uses).  Prints ONE JSON line: metric /
value / unit (whole-job target tokens per second), ms_per_step, the workload in `config`,
`roofline` for the dominant kernel (live HIP-event timing of its launches against the fp32 MFMA
peak, measured HBM traffic), `step` (the matrix-product flop of one step of 768 hypotheses over the
measured time per step, against the same peak), `hbm_kernels`, `cpu_baseline` (the CPU restatement
on the host cores, same sentences), `parity` (every sentence's search against the oracle's), and
beside them `batch` (the same sentences one batch after the other, lnmt_decode_batch) and
`split_products` (the opt-in arithmetic).

  python bench.py --gpus 1 --steps K --warmup W

Only one GPU is used; --gpus N with N > 1 exits with a message.
"""
import argparse
import gc
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

SEED = 20161030
HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
MFMA_FP32_PEAK_TFLOPS = 157.3
MFMA_BF16_PEAK_TFLOPS = 2500.0  # dense bf16 MFMA, MI355X
# HBM-side bytes per launch of the dominant kernel (fetched + written beyond L2), measured with
# `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` over this script (KiB per dispatch at the
# grid of 768 live columns; FETCH_SIZE x 2.0 and WRITE_SIZE x 1.0, the factors a device copy of
# known size gives).  A counter run cannot happen inside the timed run, so the figure is carried
# here, from the counter runs whose summary is kept under profiles/ (the decode kernel profile's
# traffic section names the commands); its algorithmic counterpart is 30000*1000*4 + 768*1000*4
# read + 30000*768*4 written.
MEASURED_TRAFFIC_BYTES = {
    "gemm_kernel<64, 64, 2, 2, 1, 16, false, false>": int((238145 + 94004) * 1024),
    "gemm_kernel<128, 96, 4, 1, 1, 16, false, false>": int((240671 + 89778) * 1024),
    "gemm_kernel<128, 64, 2, 2, 1, 16, false, false>": int((232112 + 101329) * 1024),
}


def make_params(rng, layers, H, Vs, Vt, scale=0.08, E=None, fast=False):
    """uniform[-0.08, 0.08], forget-gate bias 1 (reference initialisation)."""
    P = {}
    E = H if E is None else E
    if fast:  # float32 generator: the 0.8 G parameters of the training workload in seconds
        u = lambda *s: ((rng.random(size=s, dtype=np.float32) * 2 - 1) * np.float32(scale))
    else:
        u = lambda *s: rng.uniform(-scale, scale, size=s).astype(np.float32)
    for side, V in (("src", Vs), ("tgt", Vt)):
        for l in range(layers):
            pfx = f"{side}.{l}."
            for g in "ifco":
                P[pfx + "W_h" + g] = u(H, H)
                P[pfx + "M_" + g] = u(H, E if l == 0 else H)
                P[pfx + "b_" + g] = u(H)
                if side == "tgt" and l == 0:
                    P[pfx + "Q_" + g] = u(H, H)
            P[pfx + "b_f"] = np.ones(H, np.float32)
            if l == 0:
                P[pfx + "W"] = u(E, V)
    for n in ("W_a", "W_p", "W_c1", "W_c2"):
        P["attn." + n] = u(H, H)
    P["attn.v_p"] = u(H)
    P["attn.b_out"] = u(H)
    P["softmax.D"] = u(Vt, H)
    P["softmax.b_d"] = u(Vt)
    return P


def zipf_ids(rng, n, V, s=1.1, lo=0):
    """Zipf(s) over the ids lo..V-1 (rank 1 = id lo)."""
    ranks = np.arange(1, V - lo + 1, dtype=np.float64)
    p = ranks ** (-s)
    p /= p.sum()
    return (rng.choice(V - lo, size=n, p=p) + lo).astype(np.int32)


def make_sentences(rng, n_sent, V, lo_len=10, hi_len=60):
    lens = rng.integers(lo_len, hi_len + 1, size=n_sent)
    return [zipf_ids(rng, int(L), V) for L in lens]


def near_tie_epsilon(score, score_deviation):
    """Gap below which two fp32 implementations of the same search may order two candidates of a
    step differently, given how far their path scores were apart when the step began: twice that
    deviation (either candidate's score may be off by it, in opposite directions) plus 8 units in
    the last place of the score for the step's own log-probability and addition."""
    return 2.0 * float(score_deviation) + 8.0 * float(np.spacing(np.float32(abs(score))))


# A local-p attention window is cut at (int)p_t with p_t = S * sigmoid(.) (LowerUpperKernel,
# src/deep_rnn_kernel.h:1095-1098).  Two fp32 evaluations of the sigmoid agree to the absolute
# tolerance of an fp32 state, 1e-5, so a p_t within S * 1e-5 of an integer may give them windows
# one source position apart -- a discrete change of the context vector that moves the step's
# log-probabilities by ~1e-2.
WINDOW_TIE_PER_SOURCE_POSITION = 1e-5


def classify_beam_parity(gpu_best, gpu_tok, gpu_bp, gpu_score, trace, source_len=0):
    """Compares one sentence's GPU search (1-best; beam tokens, back-pointers and path scores per
    expansion step) with the oracle's traced search.  Returns (class, step, epsilon):
      "identical"            every step's beam and the 1-best are the same;
      "diverged_at_near_tie" the first step that differs is one whose closest decision in the
                             oracle was nearer than near_tie_epsilon, with the score deviation
                             MEASURED on the identical beams of the step before (everything before
                             it equal);
      "diverged_at_window_tie" (source_len given) the first step that differs is one where a live
                             column's window position was within source_len * 1e-5 of an integer
                             in the oracle (trace["window_margin"]);
      "diverged_other"       a difference that neither explains (a bug)."""
    n = min(len(gpu_tok), len(trace["tok"]))
    dev = 0.0  # largest |GPU score - oracle score| over the beam entries of the steps so far
    for t in range(n):
        if (gpu_tok[t].tolist() != trace["tok"][t].tolist()
                or gpu_bp[t].tolist() != trace["backptr"][t].tolist()):
            eps = near_tie_epsilon(float(np.abs(trace["score"][t]).max()), dev)
            if trace["margin"][t] < eps:
                return "diverged_at_near_tie", t, eps
            if (source_len > 0 and "window_margin" in trace
                    and trace["window_margin"][t] < WINDOW_TIE_PER_SOURCE_POSITION * source_len):
                return "diverged_at_window_tie", t, eps
            return "diverged_other", t, eps
        live = trace["score"][t] > -1e30  # slots filled with -FLT_MAX when candidates ran out
        if live.any():
            dev = max(dev, float(np.abs(gpu_score[t][live] - trace["score"][t][live]).max()))
    if len(gpu_tok) != len(trace["tok"]) or list(gpu_best) != list(trace["best"]):
        return "diverged_other", n, 0.0
    return "identical", -1, 0.0


# HBM-side bytes per launch of the attention kernels at the decode step's size (768 columns, 12 per
# sentence, S=60, D=10), from `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` over
# `bench.py --kernels` (FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 KiB per dispatch).  Their algorithmic
# byte count charges every beam column its own window, but the 12 columns of a sentence share one
# in L2, so the rate against the HBM peak is quoted on the measured bytes.
MEASURED_ATTN_BYTES = {
    ("attn_core_fwd (local-p)", 768): int((21146 + 3195) * 1024),
    ("attn_core_projected_fwd (local-p, decoding)", 768): int((37725 + 3195) * 1024),
}


def bench_fused_kernels(torch, steps, warmup, quick=False):
    from linmt_amd import lib as lh
    lh.load()
    steps = max(steps, 20)
    dev = "cuda"
    # quick: the subset that goes into the default run's `hbm_kernels` field (a second or two)
    big = (lambda full, small: small) if quick else (lambda full, small: full)

    def timed(fn):
        for _ in range(max(warmup, 3)):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / steps  # us

    out = []
    ceiling = {}  # what this GPU sustains: "rw" = the plain copy, "ro" = the faster read-only pass

    def add(name, shape, nbytes, fn, columns=None, kind=None):
        """kind: "rw" for a kernel that writes about as much as it reads, "ro" for one that only
        reads: its rate is also quoted against the calibration pass of that kind."""
        us = timed(fn)
        gbs = nbytes / us / 1e3
        row = {"kernel": name, "shape": shape, "alg_bytes": int(nbytes), "us": round(us, 2),
               "GB/s": round(gbs, 1), "frac_of_8TBs": round(gbs / HBM_PEAK_GBS, 4)}
        if kind == "rw":
            row["frac_of_copy_rate"] = round(gbs / ceiling["rw"], 4)
        elif kind == "ro":
            row["frac_of_read_only_ceiling"] = round(gbs / ceiling["ro"], 4)
        hbm = MEASURED_ATTN_BYTES.get((name, columns))
        if hbm:  # L2 serves most of the algorithmic bytes: quote the HBM rate on measured traffic
            row.update({"hbm_bytes_measured": hbm, "hbm_GB/s": round(hbm / us / 1e3, 1),
                        "hbm_frac_of_8TBs": round(hbm / us / 1e3 / HBM_PEAK_GBS, 4)})
        out.append(row)

    f = (lambda n: torch.rand(n, device=dev) * 2 - 1) if quick else (lambda n: torch.randn(n, device=dev))
    # calibration: plain copy, n floats read + n floats written
    n = 256 * 1024 * 1024  # 1 GiB: far beyond the 256 MB memory-side cache, in the quick subset as well
    src, dst = f(n), torch.empty(n, device=dev)
    add("device copy (calibration)", f"{n} floats", 8.0 * n, lambda: dst.copy_(src))
    ceiling["rw"] = out[-1]["GB/s"]
    # calibration for the kernels that only read (log-softmax + loss, beam top-k): n floats read,
    # nothing written -- the library's sum and this library's own sum of squares (lh_grad_sumsq_f32)
    add("read-only pass (calibration, library sum)", f"{n} floats", 4.0 * n, lambda: torch.sum(src))
    ws = torch.zeros(lh.LH_SUMSQ_WORKSPACE, dtype=torch.float64, device=dev)
    acc = torch.zeros(1, dtype=torch.float64, device=dev)
    add("read-only pass (calibration, lh_grad_sumsq_f32)", f"{n} floats", 4.0 * n,
        lambda: lh.grad_sumsq(src, n, 1, n, 1.0, ws, acc))
    read_ceiling = max(r["GB/s"] for r in out if r["kernel"].startswith("read-only pass"))
    ceiling["ro"] = read_ceiling
    del src, dst
    for H, B in big(((1000, 768), (1000, 768 * 64), (2048, 256 * 32)), ((1000, 768), (1000, 768 * 16))):
        pre, bias, cp = f(4 * H * B), f(4 * H), f(H * B)
        m = torch.ones(B, dtype=torch.int32, device=dev)
        c, h = torch.empty(H * B, device=dev), torch.empty(H * B, device=dev)
        gates = torch.empty(4 * H * B, device=dev)
        add("lstm_cell_fwd (inference)", f"H={H} B={B}", 28.0 * H * B,
            lambda: lh.lstm_cell_fwd(H, B, pre, bias, cp, m, c, h), kind="rw")
        if not quick:
            add("lstm_cell_fwd (gates kept)", f"H={H} B={B}", 44.0 * H * B,
                lambda: lh.lstm_cell_fwd(H, B, pre, bias, cp, m, c, h, gates=gates), kind="rw")
        del pre, cp, c, h, gates
    for V, B in big(((30000, 768), (30000, 768 * 8), (50000, 256 * 16)), ((30000, 768), (30000, 768 * 4))):
        z, p = f(V * B), torch.empty(V * B, device=dev)
        K = 13
        cl = torch.empty(K * B, device=dev)
        ci = torch.empty(K * B, dtype=torch.int32, device=dev)
        le = torch.empty(B, device=dev)
        tgt = torch.randint(0, V, (B,), dtype=torch.int32, device=dev)
        m = torch.ones(B, dtype=torch.int32, device=dev)
        lp = torch.zeros(B, dtype=torch.float64, device=dev)
        loss = torch.zeros(1, dtype=torch.float64, device=dev)
        add("softmax_fwd (probabilities out)", f"V={V} B={B}", 8.0 * V * B,
            lambda: lh.softmax_fwd(z, V, None, V, B, p, V), kind="rw")
        add("logsoftmax_xent (double)", f"V={V} B={B}", 4.0 * V * B,
            lambda: lh.logsoftmax_xent(z, V, None, V, B, tgt, m, lp, loss), kind="ro")
        add("beam_topk (log-softmax + top-13)", f"V={V} B={B}", 4.0 * V * B,
            lambda: lh.beam_topk(z, V, None, V, B, K, 1, cl, ci, le), kind="ro")
        if B == 768 and not quick:
            # an ensemble of two models: both distributions are read once
            p2 = torch.empty(V * B, device=dev)
            lh.softmax_fwd(f(V * B), V, None, V, B, p2, V)
            add("beam_topk_ensemble (2 models, mean + top-13)", f"V={V} B={B}", 8.0 * V * B,
                lambda: lh.beam_topk_ensemble([p, p2], V, V, B, K, 1, cl, ci, le), kind="ro")
            del p2
        del z, p
    for H, B, S, D, per in big(((1000, 768, 60, 10, 12), (1000, 768 * 16, 60, 10, 1)),
                               ((1000, 768, 60, 10, 12), (1000, 768 * 8, 60, 10, 1))):
        ncol = B // per
        hs = f(S * ncol * H)
        tanh1, v_p, wa = torch.tanh(f(H * B)), f(H) * 0.1, f(H * B) * 0.1
        col = (torch.arange(B, device=dev, dtype=torch.int32) // per).contiguous()
        bi = torch.cat([torch.full((B,), S, dtype=torch.int32, device=dev),
                        torch.zeros(B, dtype=torch.int32, device=dev)])
        m = torch.ones(B, dtype=torch.int32, device=dev)
        W = 2 * D + 1
        o = [torch.empty(B, device=dev), torch.empty(B, device=dev),
             torch.empty(B * W, dtype=torch.int32, device=dev), torch.empty(B * W, device=dev),
             torch.empty(B * W, device=dev), torch.empty(H * B, device=dev)]
        add("attn_core_fwd (local-p)", f"H={H} B={B} S={S} D={D} ({per} columns/sentence)",
            4.0 * B * (W * H + 2 * H + 2 * W),
            lambda: lh.attn_core_fwd(H, B, D, 0, S, tanh1, v_p, wa, hs, ncol * H, H, col, bi, m,
                                     o[0], o[1], o[2], o[3], o[4], o[5]), columns=B)
        # the decoding form: scores against W_a*hs, context sum over W_c1*hs, h~ out
        hs2, both, b_out = f(S * ncol * H), f(2 * H * B), f(H) * 0.1
        add("attn_core_projected_fwd (local-p, decoding)",
            f"H={H} B={B} S={S} D={D} ({per} columns/sentence)",
            4.0 * B * (2 * W * H + 4 * H + 2 * W),
            lambda: lh.attn_core_projected_fwd(H, B, D, S, both, 2 * H, v_p, wa, H, hs, hs2, ncol * H,
                                               H, col, bi, m, both[H:], 2 * H, b_out, o[0], o[1],
                                               o[2], o[3], o[4], o[5]), columns=B)
        del hs, hs2, both, tanh1, wa
    for H, B, n_t in big(((1000, 768, 9), (1000, 768 * 16, 9)), ((1000, 768, 9), (1000, 768 * 8, 9))):
        srcs = [f(H * B) for _ in range(n_t)]
        dsts = [torch.empty(H * B, device=dev) for _ in range(n_t)]
        bp = torch.randint(0, B, (B,), dtype=torch.int32, device=dev)
        add("beam_gather", f"H={H} B={B} tensors={n_t}", 8.0 * n_t * H * B,
            lambda: lh.beam_gather(srcs, dsts, H, B, bp), kind="rw")
        del srcs, dsts
    for E, V, B in big(((1000, 30000, 768), (1000, 30000, 768 * 64)), ()):
        Wm = f(E * V)
        idx = torch.randint(0, V, (B,), dtype=torch.int32, device=dev)
        o = torch.empty(E * B, device=dev)
        add("embed_lookup", f"E={E} V={V} B={B}", 8.0 * E * B,
            lambda: lh.embed_lookup(Wm, E, V, idx, B, o), kind="rw")
        del Wm, o
    return {"metric": "fused-kernel HBM GB/s % of peak", "unit": "GB/s", "peak": HBM_PEAK_GBS,
            "copy_rate_GB/s": ceiling["rw"], "read_only_ceiling_GB/s": read_ceiling,
            "launches_timed": steps, "kernels": out}


def bench_mfma_kernels(torch, steps, warmup):
    """The decode step's two MFMA kernels alone, at the size one step of the benchmark gives them
    (768 columns): the output projection D*h~ + b_d and one layer's gate product with the fused
    LSTM cell, next to a plain 1 GiB copy (the calibration point for clock counters)."""
    import ctypes as C
    from linmt_amd import lib as lh
    lh.load()
    steps = max(steps, 20)
    dev = "cuda"
    f = lambda n: (torch.rand(n, device=dev) - 0.5) * 0.16

    def timed(fn):
        for _ in range(max(warmup, 3)):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / steps  # us

    out = []
    n = 256 * 1024 * 1024
    src, dst = f(n), torch.empty(n, device=dev)
    us = timed(lambda: dst.copy_(src))
    out.append({"kernel": "device copy (calibration)", "shape": f"{n} floats", "us": round(us, 2),
                "GB/s": round(8.0 * n / us / 1e3, 1)})
    del src, dst
    H, V, B = 1000, 30000, 768
    D, bd, x, logits = f(V * H), f(V), f(H * B), torch.empty(V * B, device=dev)
    us = timed(lambda: lh.gemm(V, B, [(D, V, x, H, H)], logits, V, bias=bd))
    flop = 2.0 * V * B * H
    out.append({"kernel": "logits_gemm", "shape": f"M={V} N={B} K={H}", "flop": flop, "us": round(us, 2),
                "TFLOP/s": round(flop / us / 1e6, 2),
                "frac_of_peak": round(flop / us / 1e6 / MFMA_FP32_PEAK_TFLOPS, 4)})
    del D, logits
    W, M4, hb, hp = f(4 * H * H), f(4 * H * H), f(H * B), f(H * B)
    b4, cp = f(4 * H), f(H * B)
    m = torch.ones(B, dtype=torch.int32, device=dev)
    c, h = torch.empty(H * B, device=dev), torch.empty(H * B, device=dev)
    segs = [(M4, 4 * H, hb, H, H), (W, 4 * H, hp, H, H)]
    fusable, name = lh.gate_gemm_lstm_cell_plan(H, B, segs)
    us = timed(lambda: lh.gate_gemm_lstm_cell(H, B, segs, b4, cp, m, c, h))
    flop = 2.0 * 4 * H * B * 2 * H
    out.append({"kernel": "gate_gemm + lstm cell", "instance": name, "fused": fusable,
                "shape": f"M={4 * H} N={B} K={H}+{H}", "flop": flop, "us": round(us, 2),
                "TFLOP/s": round(flop / us / 1e6, 2),
                "frac_of_peak": round(flop / us / 1e6 / MFMA_FP32_PEAK_TFLOPS, 4)})
    del W, M4
    # calibration: the vendor library's fp32 product (torch.mm, TF32 off) at the same shapes, best
    # of its operand layouts; it has no cell epilogue, so the gate line is the bare product
    torch.backends.cuda.matmul.allow_tf32 = False
    for label, M_, N_, K_ in (("logits_gemm", V, B, H), ("gate_gemm", 4 * H, B, 2 * H),
                              ("square (what the part sustains on a large product)", 4096, 4096, 4096)):
        A_, X_ = f(M_ * K_).view(M_, K_), f(K_ * N_).view(K_, N_)
        At_, Xt_ = A_.t().contiguous(), X_.t().contiguous()
        o_ = torch.empty(M_, N_, device=dev)
        us = min(timed(lambda: torch.mm(A_, X_, out=o_)), timed(lambda: torch.mm(At_.t(), X_, out=o_)),
                 timed(lambda: torch.mm(A_, Xt_.t(), out=o_)), timed(lambda: torch.mm(At_.t(), Xt_.t(), out=o_)))
        flop = 2.0 * M_ * N_ * K_
        out.append({"kernel": f"vendor library product (calibration): {label}", "shape": f"M={M_} N={N_} K={K_}",
                    "flop": flop, "us": round(us, 2), "TFLOP/s": round(flop / us / 1e6, 2),
                    "frac_of_peak": round(flop / us / 1e6 / MFMA_FP32_PEAK_TFLOPS, 4)})
        del A_, X_, At_, Xt_, o_
    W, M4 = f(4 * H * H), f(4 * H * H)
    # the same two products from three-way bf16 splits (six bf16 MFMAs per fp32 one): operands packed
    # ahead, as the decoder does (weights once, the step's inputs per step)
    L = lh.load()
    kg = lh.split_kgroups_padded(lh.split_kgroups(H))
    D = f(V * H)
    Dp = torch.empty(lh.split_bytes(V, kg) // 4, dtype=torch.int32, device=dev)
    xp = torch.empty(lh.split_bytes(B, kg) // 4, dtype=torch.int32, device=dev)
    logits = torch.empty(V * B, device=dev)
    lh.split_pack([dict(src=D, ld=V, k_contiguous=False, D=V, K=H, planes=Dp, kgroups_total=kg, kgroups=kg)])
    src_x = [dict(src=x, ld=H, k_contiguous=True, D=B, K=H, planes=xp, kgroups_total=kg, kgroups=kg)]
    us_pack = timed(lambda: lh.split_pack(src_x))
    us = timed(lambda: lh.gemm_split(V, B, kg, Dp, xp, logits, V, bias=bd))
    flop = 2.0 * V * B * H
    name = C.create_string_buffer(160)
    L.lh_gemm_split_kernel_name(0, V, B, name, 160)
    out.append({"kernel": "logits_gemm, split products", "instance": name.value.decode(),
                "shape": f"M={V} N={B} K={H}", "flop": flop, "us": round(us, 2),
                "TFLOP/s": round(flop / us / 1e6, 2), "bf16_TFLOP/s_issued": round(6 * flop / us / 1e6, 1),
                "frac_of_bf16_peak": round(6 * flop / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4),
                "packing_h_us": round(us_pack, 2)})
    del D, Dp, logits
    g1 = lh.split_kgroups(H)
    KG = lh.split_kgroups_padded(2 * g1)
    Wp = torch.empty(lh.split_bytes(L.lh_split_gate_rows(H), KG) // 4, dtype=torch.int32, device=dev)
    Xp = torch.empty(lh.split_bytes(B, KG) // 4, dtype=torch.int32, device=dev)
    lh.split_pack([dict(src=M4, ld=4 * H, k_contiguous=False, D=4 * H, K=H, gate_H=H, planes=Wp,
                        kgroups_total=KG, kg_offset=0, kgroups=g1),
                   dict(src=W, ld=4 * H, k_contiguous=False, D=4 * H, K=H, gate_H=H, planes=Wp,
                        kgroups_total=KG, kg_offset=g1, kgroups=KG - g1)])
    src_g = [dict(src=hb, ld=H, k_contiguous=True, D=B, K=H, planes=Xp, kgroups_total=KG, kg_offset=0, kgroups=g1),
             dict(src=hp, ld=H, k_contiguous=True, D=B, K=H, planes=Xp, kgroups_total=KG, kg_offset=g1,
                  kgroups=KG - g1)]
    lh.split_pack(src_g)
    us = timed(lambda: lh.gate_gemm_split_lstm_cell(H, B, KG, Wp, Xp, b4, cp, m, c, h))
    flop = 2.0 * 4 * H * B * 2 * H
    L.lh_gemm_split_kernel_name(1, H, B, name, 160)
    out.append({"kernel": "gate_gemm + lstm cell, split products", "instance": name.value.decode(),
                "shape": f"M={4 * H} N={B} K={H}+{H}", "flop": flop, "us": round(us, 2),
                "TFLOP/s": round(flop / us / 1e6, 2), "bf16_TFLOP/s_issued": round(6 * flop / us / 1e6, 1),
                "frac_of_bf16_peak": round(6 * flop / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)})
    return {"metric": "MFMA kernels alone, fp32 TFLOP/s", "unit": "TFLOP/s",
            "peak": MFMA_FP32_PEAK_TFLOPS, "bf16_peak": MFMA_BF16_PEAK_TFLOPS, "launches_timed": steps,
            "kernels": out}


def bench_training(torch, host, steps, warmup, small, split=False):
    """One training minibatch (forward with stored activations, backward, global-norm clip at 5,
    SGD update) of the 8+8-layer, 2048-hidden, 1024-embedding, 50k-vocabulary model with local-p
    attention and input feeding, batch 256, lengths uniform in [20,80], dropout 0.2
    (BASELINE.json configs[4]).  Prints target tokens/s and the per-kernel-site table."""
    rng = np.random.default_rng(SEED)
    if small:
        L, H, E, V, B, lo, hi = 2, 512, 256, 8000, 64, 10, 30
    else:
        L, H, E, V, B, lo, hi = 8, 2048, 1024, 50000, 256, 20, 80
    longest = hi + 4
    t0 = time.time()
    m = host.Model(L, H, V, V, longest_sentence=longest, attention_mode=1, attention_width=10,
                   feed_input=True, minibatch_size=B, embedding_size=E,
                   training=dict(learning_rate=0.1, grad_clip_mode=2, norm_clip=5.0, dropout_keep=0.8,
                                 dropout_seed=SEED))
    m.set_params(make_params(rng, L, H, V, V, E=E, fast=True))
    m.set_split_products(bool(split))
    t_init = time.time() - t0
    ls = rng.integers(lo, hi + 1, size=B)
    lt = rng.integers(lo, hi + 1, size=B)
    S, T = int(ls.max()), int(lt.max())
    src = np.full((B, S), -1, np.int32)
    tin = np.full((B, T), -1, np.int32)
    tout = np.full((B, T), -1, np.int32)
    for b in range(B):
        src[b, S - ls[b]:] = zipf_ids(rng, ls[b], V)
        t = zipf_ids(rng, lt[b] - 1, V, lo=3)
        tin[b, :lt[b]] = np.concatenate([[0], t])
        tout[b, :lt[b]] = np.concatenate([t, [1]])
    bi = np.concatenate([ls, S - ls]).astype(np.int32)
    su = np.unique(src[src >= 0]).astype(np.int32)
    tu = np.unique(tin[tin >= 0]).astype(np.int32)
    n_tgt, n_src = int(lt.sum()), int(ls.sum())

    def step():
        ll = m.compute_gradients(src, tin, tout, bi, su, tu)
        return ll, m.update_weights()

    for _ in range(warmup):
        step()
    m.profile(0)
    torch.cuda.synchronize()
    t0 = time.time()
    for _ in range(steps):
        ll, nrm = step()
    torch.cuda.synchronize()
    dt = (time.time() - t0) / steps
    # the per-site table comes from further, untimed minibatches with every launch bracketed by
    # events (the brackets cost about 10 us of idle GPU per launch, 6-8% of such a minibatch)
    m.profile(2)
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    tot = m.profile_totals()
    m.profile(0)
    rows = []
    for k, v in sorted(tot.items(), key=lambda kv: -kv[1]["ms"]):
        is_gemm = "|" in k
        us = v["ms"] * 1e3 / max(v["launches"], 1)
        rate = v["work"] / max(v["ms"], 1e-9) / 1e9 if is_gemm else v["work"] / max(v["ms"], 1e-9) / 1e6
        rows.append({"site": k, "ms_per_step": round(v["ms"] / steps, 3),
                     "launches_per_step": v["launches"] // steps, "us_per_launch": round(us, 1),
                     ("TFLOP/s" if is_gemm else "GB/s"): round(rate, 1)})
    out = {"metric": "target tokens/sec (training step: forward + backward + clip + SGD)",
           "value": round(n_tgt / dt, 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps,
           "warmup": warmup, "ms_per_step": round(dt * 1e3, 2), "higher_is_better": True,
           "dtype": "f32", "data": "synthetic",
           "config": {"workload": ("configs[4]" if not small else "reduced smoke size")
                      + f": {L}+{L} layers, H={H}, E={E}, V={V}, batch {B}, S={S}, T={T}, "
                      f"dropout keep 0.8, {n_src} source + {n_tgt} target tokens"},
           "loglik_per_target_token": round(ll / n_tgt, 4), "global_grad_norm": round(nrm, 4),
           "kernel_ms_per_step": round(sum(v["ms"] for v in tot.values()) / steps, 2),
           "model_build_s": round(t_init, 1), "kernels": rows}
    m.close()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--cpu-sentences", type=int, default=64,
                    help="sentences of the same workload decoded by the CPU oracle for cpu_baseline")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-hbm-kernels", action="store_true",
                    help="skip the stand-alone timing of the HBM-bound kernels (hbm_kernels field)")
    ap.add_argument("--no-batch", action="store_true",
                    help="skip the extra leg that decodes the same sentences one batch after the "
                         "other (lnmt_decode_batch; reported beside `value`, never as it)")
    ap.add_argument("--no-split-products", action="store_true",
                    help="skip the second timing of the same batch with the opt-in arithmetic "
                         "(lnmt_set_split_products; reported beside `value`, never as it)")
    ap.add_argument("--split-products-only", action="store_true",
                    help="profiling aid: the whole run (timed steps, kernel table, parity) with the "
                         "opt-in arithmetic switched on; the JSON line's metric and dtype say so")
    ap.add_argument("--profile-level", type=int, default=1,
                    help="1: HIP events around the output projection (the dominant kernel) during "
                         "the timed steps; "
                         "2: one extra untimed pass with every launch bracketed (kernel table)")
    ap.add_argument("--kernels", action="store_true",
                    help="instead of the decode benchmark, time the fused HBM-bound kernels alone "
                         "(at the benchmark's size and at a size that saturates HBM) and print "
                         "one JSON line with their achieved GB/s")
    ap.add_argument("--mfma-kernels", action="store_true",
                    help="instead of the decode benchmark, time the decode step's two MFMA kernels "
                         "alone (output projection, gate product + cell) at 768 columns")
    ap.add_argument("--train", action="store_true",
                    help="instead of the decode benchmark, time one training minibatch of "
                         "BASELINE.json configs[4] and print one JSON line")
    ap.add_argument("--train-small", action="store_true", help="--train at a reduced size")
    ap.add_argument("--train-split-products", action="store_true",
                    help="--train with the opt-in arithmetic for the large batched products")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on ONE GPU (the path shards over sentences with no "
              f"communication; no multi-GPU run is part of it); --gpus {args.gpus} is not supported",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from linmt_amd import host

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    host.load()
    if args.kernels:
        print(json.dumps(bench_fused_kernels(torch, args.steps, args.warmup)))
        return
    if args.mfma_kernels:
        print(json.dumps(bench_mfma_kernels(torch, args.steps, args.warmup)))
        return
    if args.train or args.train_small or args.train_split_products:
        print(json.dumps(bench_training(torch, host, args.steps, args.warmup, args.train_small,
                                        args.train_split_products)))
        return

    layers, H, V, D, beam, n_sent, longest = 4, 1000, 30000, 10, 12, 64, 104
    rng = np.random.default_rng(SEED)
    P = make_params(rng, layers, H, V, V)
    sents = make_sentences(rng, n_sent, V)
    model = host.Model(layers, H, V, V, longest_sentence=longest, attention_mode=1,
                       attention_width=D, feed_input=True, decoding=(n_sent, beam))
    model.set_params(P)
    # `value` is the fp32 MFMA path whatever the environment says (unless the run is asked to be
    # about the opt-in arithmetic, which its metric then names)
    model.set_split_products(bool(args.split_products_only))

    def gemm_roofline(totals, site_prefix="logits_gemm"):
        """The GEMM kernel instance that carries the most algorithmic work among the bracketed
        launches of a call site: achieved = sum of flop / sum of launch durations."""
        by_kernel = {}
        for key, t in totals.items():
            if "|" not in key or not key.startswith(site_prefix):
                continue
            site, kern = key.split("|", 1)
            e = by_kernel.setdefault(kern, dict(ms=0.0, work=0.0, launches=0, sites=set()))
            e["ms"] += t["ms"]
            e["work"] += t["work"]
            e["launches"] += t["launches"]
            e["sites"].add(site)
        if not by_kernel:
            return None
        kern, g = max(by_kernel.items(), key=lambda kv: kv[1]["work"])
        achieved = g["work"] / (g["ms"] * 1e-3) / 1e12
        r = {"kernel": kern, "call_sites": sorted(g["sites"]), "bound": "mfma",
             "achieved": round(achieved, 2), "peak": MFMA_FP32_PEAK_TFLOPS,
             "unit": "TFLOP/s", "frac": round(achieved / MFMA_FP32_PEAK_TFLOPS, 4),
             "traffic": MEASURED_TRAFFIC_BYTES.get(kern), "launches": g["launches"],
             "avg_launch_us": round(g["ms"] * 1e3 / g["launches"], 2)}
        if kern.startswith("gemm_split_kernel"):  # six bf16 products issued per algorithmic product
            r.update({"algorithmic_TFLOP/s": round(achieved, 2), "achieved": round(6 * achieved, 1),
                      "peak": MFMA_BF16_PEAK_TFLOPS,
                      "unit": "TFLOP/s (bf16 products issued = 6 x algorithmic)",
                      "frac": round(6 * achieved / MFMA_BF16_PEAK_TFLOPS, 4)})
        return r

    def kernel_table(totals):
        out = {}
        for name, t in sorted(totals.items()):
            rate = t["work"] / (t["ms"] * 1e-3)
            is_gemm = "|" in name
            out[name] = {"ms": round(t["ms"], 3), "launches": t["launches"],
                         "rate": round(rate / (1e12 if is_gemm else 1e9), 2),
                         "unit": "TFLOP/s" if is_gemm else "GB/s",
                         "frac": round(rate / ((MFMA_FP32_PEAK_TFLOPS * 1e12) if is_gemm
                                               else (HBM_PEAK_GBS * 1e9)), 4)}
        return out

    # ---- the measured hot path: the sentences of `steps` batches as ONE list through the 64 slots ----
    # One "step" = 64 source sentences through the decoder.  A sentence that has taken its last
    # step hands its 12 beam columns to the next sentence of the list (lnmt_decode_stream, what
    # Dispatcher::Decoding runs), so every step of the search runs all 768 hypotheses: encoder in
    # groups of 64, one read-back at the end, the whole call inside the timed region.
    B = n_sent * beam
    model.profile(0)
    model.decode_stream(sents * max(args.warmup, 1), beam=beam)
    model.profile(1 if args.profile_level >= 1 else 0)
    # the interpreter's cyclic collector stays out of the timed regions, as in the standard
    # library's timeit: with torch imported one full collection is tens of milliseconds
    gc.collect()
    gc.disable()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    res_all = model.decode_stream(sents * args.steps, beam=beam)  # ends with a stream synchronisation
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    prof1 = model.profile_totals()
    ticks = model.stream_ticks
    tokens = sum(len(r["best"]) for r in res_all)
    ms_per_step = dt * 1e3 / args.steps
    value = tokens / dt
    res = res_all[:n_sent]
    histories = [model.decode_history(i, beam) for i in range(n_sent)]
    copies_same = all(res_all[i]["best"].tolist() == res_all[i % n_sent]["best"].tolist()
                      for i in range(len(res_all)))
    roofline = gemm_roofline(prof1)
    # The whole step against the MFMA roofline: the matrix products of one tick of 768 hypotheses
    # (gate products of every layer, the attention projections, the output projection) over the
    # measured time per tick -- everything else the tick does (attention, top-k, merge, state
    # gather, the encoder of the coming groups, admissions) counts as time and not as work.
    flop_per_column = layers * 2.0 * 4 * H * 2 * H + 2.0 * 2 * H * H + 2.0 * V * H
    tick_us = dt * 1e6 / ticks
    step_tflops = flop_per_column * B / tick_us / 1e6
    # the encoder's matrix products run inside the same timed region, beside the steps (layers'
    # gate products and the two projected attention memories, per source word)
    enc_flop = (layers * 2.0 * 4 * H * 2 * H + 2 * 2.0 * H * H) * sum(len(s_) for s_ in sents) * args.steps
    with_encoder = (flop_per_column * B * ticks + enc_flop) / (dt * 1e6) / 1e6
    step = {"ticks": ticks, "hypotheses_per_tick": B, "tick_us": round(tick_us, 1),
            "mfma_flop_per_tick": flop_per_column * B, "achieved": round(step_tflops, 2),
            "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(step_tflops / MFMA_FP32_PEAK_TFLOPS, 4),
            "encoder_flop_per_tick": round(enc_flop / ticks),
            "achieved_with_encoder": round(with_encoder, 2),
            "frac_with_encoder": round(with_encoder / MFMA_FP32_PEAK_TFLOPS, 4)}

    kernels = {}
    if args.profile_level >= 2:
        model.profile(2)
        model.decode_stream(sents * min(args.steps, 2), beam=beam)
        kernels = kernel_table(model.profile_totals())
    model.profile(0)

    # ---- beside it: one batch after the other (DecodeBatch), the batch's live hypotheses falling ----
    # from 768 to 12 as its sentences end
    batch, batch_hist, batch_res = None, None, None
    if not args.no_batch:
        for _ in range(args.warmup):
            model.decode_batch(sents, beam=beam)
        model.profile(1 if args.profile_level >= 1 else 0)
        torch.cuda.synchronize()
        b0 = time.perf_counter()
        btok = 0
        for _ in range(args.steps):
            batch_res = model.decode_batch(sents, beam=beam)  # ends with a stream synchronisation
            btok += sum(len(r["best"]) for r in batch_res)
        torch.cuda.synchronize()
        bdt = time.perf_counter() - b0
        batch_hist = [model.decode_history(i, beam) for i in range(n_sent)]
        batch = {"value": round(btok / bdt, 1), "unit": "target tokens/s",
                 "ms_per_batch": round(bdt * 1e3 / args.steps, 2),
                 "ratio_to_value": round(btok / bdt / value, 3),
                 "how": "lnmt_decode_batch on the same 64 sentences, one batch after the other",
                 "roofline": gemm_roofline(model.profile_totals()),
                 "one_best_same_as_value": int(sum(a["best"].tolist() == b["best"].tolist()
                                                   for a, b in zip(res, batch_res)))}
        if args.profile_level >= 2:
            model.profile(2)
            model.decode_batch(sents, beam=beam)
            batch["kernels"] = kernel_table(model.profile_totals())
        model.profile(0)

    # The same list with the opt-in arithmetic: gate products and output projection from three-way
    # bf16 splits of their fp32 operands (six exact products per term, fp32 accumulation).  Reported
    # beside `value`; `value` stays the fp32 MFMA path.
    split, split_res, split_hist = None, None, None
    if not args.no_split_products and not args.split_products_only:
        model.set_split_products(True)
        # Warm-up: the first call packs the weights; the GPU's power management takes ~150 ms to
        # settle on the other matrix pipe, so the warm-up list is at least three batches long.
        model.profile(0)
        model.decode_stream(sents * (max(args.warmup, 1) + 2), beam=beam)
        model.profile(1)
        torch.cuda.synchronize()
        s0 = time.perf_counter()
        ss_all = model.decode_stream(sents * args.steps, beam=beam)  # ends with a stream synchronisation
        torch.cuda.synchronize()
        sdt = time.perf_counter() - s0
        stok = sum(len(r["best"]) for r in ss_all)
        split_res = ss_all[:n_sent]
        split_hist = [model.decode_history(i, beam) for i in range(n_sent)]
        sroof = gemm_roofline(model.profile_totals())
        split = {"value": round(stok / sdt, 1), "unit": "target tokens/s",
                 "ms_per_step": round(sdt * 1e3 / args.steps, 2),
                 "tick_us": round(sdt * 1e6 / model.stream_ticks, 1),
                 "speedup_over_value": round(stok / sdt / value, 3),
                 "arithmetic": "fp32 operands held as three bf16 terms; every product = six exact "
                               "bf16 x bf16 products (v_mfma_f32_32x32x16_bf16) added in fp32; what "
                               "is left out is below 2^-23 per product; used for the gate products "
                               "and the output projection of steps with >= 84 live hypotheses",
                 "one_best_same_as_fp32_path": int(sum(a["best"].tolist() == b["best"].tolist()
                                                       for a, b in zip(res, split_res)))}
        if sroof:
            split["roofline"] = sroof
        if args.profile_level >= 2:
            model.profile(2)
            model.decode_stream(sents * min(args.steps, 2), beam=beam)
            split["kernels"] = kernel_table(model.profile_totals())
        model.profile(0)
        if not args.no_batch:
            model.decode_batch(sents, beam=beam)
            torch.cuda.synchronize()
            b0 = time.perf_counter()
            sbtok = 0
            for _ in range(args.steps):
                sbtok += sum(len(r["best"]) for r in model.decode_batch(sents, beam=beam))
            sbdt = time.perf_counter() - b0
            split["batch"] = {"value": round(sbtok / sbdt, 1), "unit": "target tokens/s",
                              "ms_per_batch": round(sbdt * 1e3 / args.steps, 2)}
        model.set_split_products(False)

    # the metric's second half: the fused HBM-bound kernels alone (outside the timed region), each
    # at the size one decode step gives it (768 columns) and at a size that saturates HBM, next to
    # a plain device copy and a read-only pass, the practical ceilings of this GPU
    hbm_kernels = None
    if not args.no_hbm_kernels:
        k = bench_fused_kernels(torch, 20, 2, quick=True)
        hbm_kernels = {"peak_GB/s": HBM_PEAK_GBS, "copy_rate_GB/s": k["copy_rate_GB/s"],
                       "read_only_ceiling_GB/s": k["read_only_ceiling_GB/s"],
                       "launches_timed": k["launches_timed"],
                       "kernels": [{a: r[a] for a in ("kernel", "shape", "us", "GB/s", "frac_of_8TBs",
                                                      "frac_of_copy_rate", "frac_of_read_only_ceiling",
                                                      "hbm_GB/s", "hbm_frac_of_8TBs") if a in r}
                                   for r in k["kernels"]]}

    gc.enable()
    cpu_baseline = None
    parity = None
    if not args.no_cpu_baseline and args.cpu_sentences > 0:
        from oracle import orc  # the checker / reported baseline, never the measured path
        # every host core this process may use: OMP_NUM_THREADS when the environment sets it (a GPU
        # box gives a job a share of its cores), else all of them
        host_cores = os.cpu_count() or 1
        env_threads = int(os.environ.get("OMP_NUM_THREADS", "0") or 0)
        cores = min(host_cores, env_threads) if env_threads > 0 else host_cores
        om = orc.Model(layers, H, V, V, attention=1, D=D, feed_input=1, longest_sent=longest)
        om.set_params(P)
        # bounded sample: every k-th sentence of the batch by length (all 64 by default, about
        # 10-30 s of CPU work), each decoded on its own by the CPU restatement
        by_len = np.argsort([len(s) for s in sents], kind="stable")
        pick = by_len[np.unique(np.linspace(0, n_sent - 1, min(args.cpu_sentences, n_sent)).round().astype(int))]
        om.decode_sentence(sents[by_len[0]][:3], beam=beam, num_threads=cores)  # warm-up
        cpu_tokens, cdt = 0, 0.0
        classes = {"identical": 0, "diverged_at_near_tie": 0, "diverged_at_window_tie": 0, "diverged_other": 0}
        sclasses, bclasses = dict(classes), dict(classes)
        same, ssame, bsame, detail = 0, 0, 0, []
        for i in pick:
            c0 = time.perf_counter()
            tr = om.decode_sentence_trace(sents[i], beam=beam, num_threads=cores)
            cdt += time.perf_counter() - c0
            cpu_tokens += len(tr["best"])
            gtok, gbp, gsc = histories[int(i)]
            cls, at, eps = classify_beam_parity(res[i]["best"], gtok, gbp, gsc, tr, len(sents[i]))
            classes[cls] += 1
            same += int(tr["best"].tolist() == res[i]["best"].tolist())
            if batch is not None:
                qtok, qbp, qsc = batch_hist[int(i)]
                bclasses[classify_beam_parity(batch_res[i]["best"], qtok, qbp, qsc, tr, len(sents[i]))[0]] += 1
                bsame += int(tr["best"].tolist() == batch_res[i]["best"].tolist())
            if split is not None:
                stok_h, sbp_h, ssc_h = split_hist[int(i)]
                sclasses[classify_beam_parity(split_res[i]["best"], stok_h, sbp_h, ssc_h, tr, len(sents[i]))[0]] += 1
                ssame += int(tr["best"].tolist() == split_res[i]["best"].tolist())
            if tr["best"].tolist() != res[i]["best"].tolist() or cls == "diverged_other":
                detail.append({"sentence": int(i), "source_len": int(len(sents[i])), "class": cls,
                               "first_differing_step": int(at),
                               "oracle_margin": float(tr["margin"][at]) if 0 <= at < len(tr["margin"]) else None,
                               "oracle_window_margin": float(tr["window_margin"][at]) if 0 <= at < len(tr["margin"]) else None,
                               "epsilon": eps})
        cpu_baseline = {"value": round(cpu_tokens / cdt, 2), "unit": "target tokens/s",
                        "cores": cores, "host_cores": host_cores, "kind": "port",
                        "sample": f"{len(pick)} of the 64 benchmark sentences, spread over the "
                                  f"length distribution ({cpu_tokens} target tokens, {cdt:.1f} s), "
                                  f"decoded one at a time by the CPU restatement (oracle/) with "
                                  f"OpenMP on {cores} threads (the host shows {host_cores} cores; "
                                  f"OMP_NUM_THREADS={os.environ.get('OMP_NUM_THREADS', 'unset')})"}
        parity = {"sentences_checked": int(len(pick)), "one_best_identical": int(same),
                  "beam_steps": classes, "parity_ok": classes["diverged_other"] == 0,
                  "repeated_sentences_decode_identically": bool(copies_same),
                  "near_tie_rule": "first differing step has an oracle margin below 2 x the largest "
                                   "|GPU - oracle| path score measured on the (identical) beams "
                                   "before it + 8 ulp of the score",
                  "window_tie_rule": "first differing step has a local-p window position within "
                                     "1e-5 x source length of an integer in the oracle (the window "
                                     "is cut at (int)p_t)",
                  "one_best_differs_or_unexplained": detail}
        if split is not None:
            split["parity"] = {"sentences_checked": int(len(pick)), "one_best_identical": int(ssame),
                               "beam_steps": sclasses, "parity_ok": sclasses["diverged_other"] == 0}
        if batch is not None:
            batch["parity"] = {"sentences_checked": int(len(pick)), "one_best_identical": int(bsame),
                               "beam_steps": bclasses, "parity_ok": bclasses["diverged_other"] == 0}

    out = {
        "metric": "target tokens/sec (beam-12 decode, 1 GPU)" +
                  (" with split bf16 products (opt-in arithmetic)" if args.split_products_only else ""),
        "value": round(value, 1),
        "unit": "target tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 2),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32 operands as three bf16 terms, f32 accumulation" if args.split_products_only else "f32",
        "data": "synthetic",
        "config": {"workload": "configs[2]: beam-12 decode, 64 sentences at a time (768 live "
                               "hypotheses in every step: a finished sentence's 12 beam columns go "
                               "to the next sentence of the list, lnmt_decode_stream), 4+4 LSTM "
                               "layers, hidden=emb=1000, vocab 30k/30k, local-p attention D=10 + "
                               "input feeding, source len U[10,60] Zipf ids, max target 1.5x "
                               "source, random-init uniform[-0.08,0.08]; one step = 64 sentences",
                   "sentences": n_sent * args.steps, "slots": n_sent,
                   "tokens_per_step": tokens // max(args.steps, 1),
                   "seed": SEED},
        "roofline": roofline,
        "step": step,
        "hbm_kernels": hbm_kernels,
        "cpu_baseline": cpu_baseline,
    }
    if batch:
        out["batch"] = batch
    if split:
        out["split_products"] = split
    if kernels:
        out["kernels"] = kernels
    if parity:
        out["parity"] = parity
    print(json.dumps(out))
    bad = []
    if parity and not parity["parity_ok"]:
        bad.append("the GPU search")
    if batch and "parity" in batch and not batch["parity"]["parity_ok"]:
        bad.append("the batch-after-batch search")
    if split and "parity" in split and not split["parity"]["parity_ok"]:
        bad.append("the search with split products")
    if not copies_same:
        bad.append("(repeated sentences decode differently)")
    if bad:
        print("bench.py: " + ", ".join(bad) + " differs from the oracle's where no near-tie "
              "explains it", file=sys.stderr)
        sys.exit(1)


if __name__ == "__main__":
    main()
