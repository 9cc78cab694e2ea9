#!/usr/bin/env python3
"""Benchmark of the INT8 hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extra]

One step = one pass of the OPT-6.7B-shaped W8A8 linear set at M = 2048 tokens (batch 4 x seq 512,
hidden 4096): q/k/v/out W8A8B8O8 4096x4096, fc1 4096->16384 with the GELU-quant epilogue, fc2
16384->4096 with fp32 output — six GEMMs through the package's launchers, inputs resident in HBM.
Prints ONE JSON line: whole-step int8 TOPS, the roofline of the dominant GEMM kernel (timed with
events on the launch stream), the CPU emulation baseline on a bounded row sample, and — under
"extra" — GB/s of the row kernels and the attention BMMs.

Set-up (untimed, before the W warm-up steps) runs the step for --settle-ms (default 40 ms) and reports what
those steps took under "cold_start": the first ~15 ms of heavy work of a process are a transient of the
chip's power management (a few steps at the boost clock, then ~25 steps well below the level it settles on).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "int8 GEMM TOPS (% MFMA peak), LN/GELU GB/s, W8A8 OPT-13B layer ms"
# Bytes that crossed the L2 <-> fabric boundary per launch of the dominant kernel on this workload come from
# rocprofv3 FETCH_SIZE / WRITE_SIZE passes taken outside bench.py; their summary under profiles/ holds the
# readings (KiB per dispatch) and the factors that scale them (from a 256 MiB device copy).  bench.py reads the
# figure from that file's table row, so it is as fresh as the file and cannot drift from it.
TRAFFIC_PROFILE = {
    "ws_256x128x128_w2x2_s1_p3_l4/int8": ("profiles/gemm_ws_opt67b_linear_set_counters.md", "average of the 5 launches of a step"),
}


def traffic_from_profile(kernel):
    """(bytes per launch, source description) for `kernel`, or (None, None): parses the row
    '| <label> | FETCH_SIZE KiB | .. | WRITE_SIZE KiB = .. |' and the two 'factor' figures of the summary."""
    import re

    if kernel not in TRAFFIC_PROFILE:
        return None, None
    rel, label = TRAFFIC_PROFILE[kernel]
    try:
        text = open(os.path.join(ROOT, rel)).read()
    except OSError:
        return None, None
    num = r"(\d[\d ]*(?:\.\d+)?)"
    ff = re.search(r"FETCH_SIZE reads[^\n]*?factor " + num, text)
    wf = re.search(r"WRITE_SIZE reads[^\n]*?factor " + num, text)
    row = re.search(r"\|\s*" + re.escape(label) + r"\s*\|\s*" + num + r"\s*\|[^|]*\|\s*" + num + r"\s*KiB", text)
    if not (ff and wf and row):
        return None, None
    val = lambda m, i=1: float(m.group(i).replace(" ", ""))
    fetch_kib, write_kib = val(row, 1), val(row, 2)
    total = (val(ff) * fetch_kib + val(wf) * write_kib) * 1024
    return total, f"{rel}, row '{label}': FETCH_SIZE {fetch_kib:.0f} KiB x {val(ff)} + WRITE_SIZE {write_kib:.0f} KiB x {val(wf)}"


INT8_PEAK_TOPS = 5000.0   # MI355X dense INT8 MFMA, published
HBM_PEAK_GBPS = 8000.0    # MI355X HBM3E, published


def build_linear_set(torch, dev, seed=1234):
    """OPT-6.7B linear set, M=2048: int8 activations/weights uniform in [-127,127], per-tensor fp32
    scales uniform in [1e-3, 1e-2]."""
    from triton_int_amd.nn.fused import W8A8BFP32OFP32_GeLu_Q
    from triton_int_amd.nn.linear import W8A8B8O8Linear, W8A8BFP32OFP32Linear

    g = torch.Generator(device="cpu").manual_seed(seed)
    M, H, F = 2048, 4096, 16384

    def i8(*shape):
        return torch.randint(-127, 128, shape, dtype=torch.int8, generator=g)

    def scale():
        return float(torch.empty(1).uniform_(1e-3, 1e-2, generator=g))

    layers = []
    for name in ("q_proj", "k_proj", "v_proj", "out_proj"):
        m = W8A8B8O8Linear(H, H, alpha=scale(), beta=scale())
        m.weight, m.bias = i8(H, H), i8(H)
        layers.append((name, m.to(dev), i8(M, H).to(dev)))
    m = W8A8BFP32OFP32_GeLu_Q(H, F, alpha=scale(), beta=scale())
    m.weight, m.bias = i8(F, H), torch.randn(F, generator=g)
    layers.append(("fc1_gelu_q", m.to(dev), i8(M, H).to(dev)))
    m = W8A8BFP32OFP32Linear(F, H, alpha=scale())
    m.weight, m.bias = i8(H, F), torch.randn(H, generator=g)
    layers.append(("fc2", m.to(dev), i8(M, F).to(dev)))
    return layers


def cpu_baseline(torch, layers, budget_s=12.0):
    """The PyTorch CPU emulation path (int32 matmul + the same scaling) on the first rows of each
    activation, chunk by chunk until about `budget_s` seconds of CPU work have been done."""
    from oracle import cpu_emulation as E

    torch.set_num_threads(min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16"))))
    host = []
    for name, m, x in layers:
        host.append((name, m.weight.cpu(), m.bias.cpu(), float(m.a), float(m.b), x.cpu()))
    chunk, rows_done, ops, elapsed = 16, 0, 0.0, 0.0
    M = host[0][5].shape[0]
    while rows_done < M and elapsed < budget_s:
        sl = slice(rows_done, rows_done + chunk)
        t0 = time.perf_counter()
        for name, w, b, a, bb, x in host:
            if name == "fc1_gelu_q":
                E.linear_gelu_q(x[sl], w, b, a, bb)
            elif name == "fc2":
                E.linear_ofp32(x[sl], w, b, a)
            else:
                E.linear_o8(x[sl], w, b, a, bb)
            ops += 2.0 * chunk * w.shape[0] * w.shape[1]
        elapsed += time.perf_counter() - t0
        rows_done += chunk
    return {
        "value": ops / elapsed / 1e12, "unit": "TOPS", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"first {rows_done} of {M} token rows through all six linears "
                  f"(torch int32 matmul + fp32 scaling, {elapsed:.1f} s of CPU work)",
    }


SETTLE_MS = 25.0  # every timed region is preceded by this much of the same work (see "cold_start" in main)


def time_region(torch, fn, iters, warm):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    # a burst of work that follows a lighter phase starts with a transient of the chip's power management (some
    # 15 ms: boost, over-correction, then the level it holds); the timed iterations come after it
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < SETTLE_MS:
        for _ in range(max(1, warm)):
            fn()
        torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) / iters  # ms


def mfma_issue_peak(torch, lib, random_operands):
    """TOPS of back-to-back int8 MFMAs on register operands (no memory traffic) at the clock the chip
    sustains; with random operand bytes this is the ceiling a GEMM on random int8 data can approach."""
    import ctypes

    ops = ctypes.c_double(0.0)
    stream = torch.cuda.current_stream().cuda_stream
    lib.ti_mfma_i8_probe(2000, random_operands, stream, ctypes.byref(ops))  # warm-up
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    rc = lib.ti_mfma_i8_probe(20000, random_operands, stream, ctypes.byref(ops))
    e.record()
    torch.cuda.synchronize()
    assert rc == 0
    return ops.value / (s.elapsed_time(e) * 1e-3) / 1e12


def _find_sclk_file(torch, glob):
    """pp_dpm_sclk of the GPU torch uses (matched by PCI address), or of the only AMD GPU in sysfs."""
    cands = sorted(glob.glob("/sys/bus/pci/devices/*/pp_dpm_sclk"))
    try:
        pr = torch.cuda.get_device_properties(0)
        addr = f"{pr.pci_domain_id:04x}:{pr.pci_bus_id:02x}:{pr.pci_device_id:02x}.0"
        for c in cands:
            if addr in c:
                return c
    except Exception:
        pass
    return cands[0] if len(cands) == 1 else None


def _read_sclk_mhz(path):
    """Current shader clock: the line of pp_dpm_sclk marked with '*'."""
    import re

    if not path:
        return None
    try:
        with open(path) as f:
            for line in f:
                if "*" in line:
                    m = re.search(r"(\d+)\s*Mhz", line, re.I)
                    return int(m.group(1)) if m else None
    except OSError:
        return None
    return None


def sustained_clock(torch, dev, seconds=2.5):
    """fc2-shaped GEMM (2048 x 4096 x 16384, fp32 out) looped for `seconds` while the driver's
    pp_dpm_sclk file is sampled from a thread: sustained TOPS and the shader clock the chip holds under that load, once with
    uniform random int8 operands and once with all-zero operands (same instruction stream, no
    operand toggling).  The difference is the power limit, not the kernel."""
    import glob
    import re
    import threading

    from triton_int_amd.kernels import linear

    M, N, K = 2048, 4096, 16384
    out = {}
    sclk_file = _find_sclk_file(torch, glob)
    for kind in ("uniform", "zeros"):
        if kind == "uniform":
            ws = [torch.randint(-127, 128, (N, K), dtype=torch.int8, device=dev) for _ in range(8)]
            x = torch.randint(-127, 128, (M, K), dtype=torch.int8, device=dev)
        else:
            ws = [torch.zeros((N, K), dtype=torch.int8, device=dev) for _ in range(8)]
            x = torch.zeros((M, K), dtype=torch.int8, device=dev)
        y = torch.empty((M, N), dtype=torch.float32, device=dev)
        clocks = []

        def sample():
            # the driver's sysfs file, read in-process (no child process is started once the GPU is in use)
            for _ in range(int(seconds / 0.5)):
                time.sleep(0.4)
                mhz = _read_sclk_mhz(sclk_file)
                if mhz:
                    clocks.append(mhz)

        th = threading.Thread(target=sample)
        th.start()
        t0, n = time.perf_counter(), 0
        while time.perf_counter() - t0 < seconds:
            for i in range(50):
                linear.linear_a8_w8_ofp32(x, ws[i % 8], 0.002, out=y)
            torch.cuda.synchronize()
            n += 50
        el = time.perf_counter() - t0
        th.join()
        out[kind] = {"TOPS": 2.0 * M * N * K * n / el / 1e12, "us_per_gemm": el / n * 1e6,
                     "sclk_mhz": (sorted(clocks)[len(clocks) // 2] if clocks else None)}
        if out[kind]["sclk_mhz"]:
            # MFMA peak at the clock actually held: 256 CUs x 8192 int8 ops per clock
            out[kind]["frac_of_peak_at_held_clock"] = out[kind]["TOPS"] * 1e12 / (256 * 8192 * out[kind]["sclk_mhz"] * 1e6)
        del ws, x, y
    return out


def extras(torch, dev):
    """GB/s of the HBM-bound kernels at the baseline's shapes (algorithmic bytes / time)."""
    from triton_int_amd.kernels import bmm, fused

    out = {}
    rows, cols = 8192, 5120
    gam, bet = torch.randn(cols, device=dev) * 2 + 20, torch.randn(cols, device=dev) * 2
    # config 3: dequant + residual add + LayerNormQ, 13 B/element (545 MB per call > 256 MB MALL)
    acc = torch.randint(-2**20, 2**20 + 1, (rows, cols), dtype=torch.int32, device=dev)
    res = torch.randn(rows, cols, device=dev)
    ms = time_region(torch, lambda: fused.dq_add_layernorm_q(acc, 1e-5, res, gam, bet, 1e-5), 20, 3)
    out["dq_add_layernorm_q_8192x5120"] = {"ms": ms, "GBps": rows * cols * 13 / ms / 1e6}
    # LayerNormQ alone, 5 B/element; two input sets are alternated so the 168 MB input is not MALL-resident
    xs = [res, torch.randn(rows, cols, device=dev)]
    state = {"i": 0}

    def lnq():
        state["i"] ^= 1
        fused.layer_norm_fwd_fused_single_pass_q(xs[state["i"]], gam, bet, 1e-5)

    ms = time_region(torch, lnq, 20, 4)
    out["layernorm_q_8192x5120"] = {"ms": ms, "GBps": rows * cols * 5 / ms / 1e6}
    del acc, res, xs
    # GELU-quant alone, 5 B/element
    xg = torch.randn(8192, 20480, device=dev)
    ms = time_region(torch, lambda: fused.gelu_q(xg, 20.0), 10, 2)
    out["gelu_q_8192x20480"] = {"ms": ms, "GBps": xg.numel() * 5 / ms / 1e6}
    # per-token dynamic quantisation, fp32 in: 5 B/element; fp16 in: 3 B/element
    ms = time_region(torch, lambda: fused.quantize_per_token_absmax(xg), 10, 2)
    out["quantize_per_token_f32_8192x20480"] = {"ms": ms, "GBps": xg.numel() * 5 / ms / 1e6}
    xh = xg.half()
    ms = time_region(torch, lambda: fused.quantize_per_token_absmax(xh), 10, 2)
    out["quantize_per_token_f16_8192x20480"] = {"ms": ms, "GBps": xh.numel() * 3 / ms / 1e6}
    del xg, xh
    # floating-point LayerNorm and the skip variant with both outputs (fp16: 4 and 8 B/element;
    # fp32: 8 and 16 B/element), 16384 x 5120 so that the fp16 tensors exceed the MALL as well
    for dt, name, eb in ((torch.float16, "f16", 2), (torch.float32, "f32", 4)):
        xl = torch.randn(16384, 5120, device=dev).to(dt)
        sk = torch.randn(16384, 5120, device=dev).to(dt)
        gl, bl = (torch.randn(5120, device=dev) * 0.1 + 1).to(dt), (torch.randn(5120, device=dev) * 0.1).to(dt)
        ms = time_region(torch, lambda: fused.layer_norm_fwd_fused_single_pass(xl, gl, bl, 1e-5), 10, 2)
        out[f"layer_norm_{name}_16384x5120"] = {"ms": ms, "GBps": xl.numel() * 2 * eb / ms / 1e6}
        ms = time_region(torch, lambda: fused.skip_layer_norm_fwd_fused_single_pass2(xl, sk, gl, bl, 1e-5), 10, 2)
        out[f"skip_layer_norm2_{name}_16384x5120"] = {"ms": ms, "GBps": xl.numel() * 4 * eb / ms / 1e6}
        del xl, sk
    # config 4: attention BMMs, 160 x (2048 x 2048 x 128); HBM-bound (755 MB / 881 MB per call)
    B, S, D = 160, 2048, 128
    q = torch.randint(-127, 128, (B, S, D), dtype=torch.int8, device=dev)
    k = torch.randint(-127, 128, (B, S, D), dtype=torch.int8, device=dev)
    sc = torch.empty((B, S, S), dtype=torch.int8, device=dev)
    ms = time_region(torch, lambda: bmm.bmm_s8t_s8n_s8t(q, k, 1e-3, out=sc), 10, 2)
    out["bmm_qk_s8_160x2048x2048x128"] = {"ms": ms, "GBps": 755.0e6 / ms / 1e6, "TOPS": 171.8e9 / ms / 1e9}
    # the same launch on all-zero operands: same instructions and bytes, less switching in the MFMAs
    # and data paths, so the chip holds a higher clock (what the kernel does when power is not the limit)
    qz, kz = torch.zeros_like(q), torch.zeros_like(k)
    ms = time_region(torch, lambda: bmm.bmm_s8t_s8n_s8t(qz, kz, 1e-3, out=sc), 10, 2)
    out["bmm_qk_s8_160x2048x2048x128_zero_operands"] = {"ms": ms, "GBps": 755.0e6 / ms / 1e6, "TOPS": 171.8e9 / ms / 1e9}
    del qz, kz
    # probabilities as the baseline prescribes them: round(127 * softmax(N(0,1) * s)), here from this
    # library's own softmax-quantise kernel on int8 scores round(32 * N(0,1)) with scale 0.05 (logit std 1.6)
    p = fused.softmax_q(torch.randn((B, S, S), device=dev).mul_(32).round_().clamp_(-127, 127).to(torch.int8), 0.05)
    vt = torch.randint(-127, 128, (B, D, S), dtype=torch.int8, device=dev)
    of = torch.empty((B, S, D), dtype=torch.float32, device=dev)
    ms = time_region(torch, lambda: bmm.bmm_s8t_s8n_f32t(p, vt, 1.0 / 16129, out=of), 10, 2)
    out["bmm_pv_f32_160x2048x128x2048"] = {"ms": ms, "GBps": 880.8e6 / ms / 1e6, "TOPS": 171.8e9 / ms / 1e9}
    del sc, of
    # int8 scores -> int8 probabilities (softmax + quantise), 2 B/element
    ms = time_region(torch, lambda: fused.softmax_q(p, 0.05), 10, 2)
    out["softmax_q_160x2048x2048"] = {"ms": ms, "GBps": p.numel() * 2 / ms / 1e6}
    del p
    for v in out.values():
        v["frac_hbm_peak"] = v["GBps"] / HBM_PEAK_GBPS
    # the same three steps (Q.K^T -> softmax-quantise -> P.V, int8 out) as one kernel: scores and
    # probabilities stay in registers, so its bound is the VALU work per score, not HBM
    ctx = torch.empty((B, S, D), dtype=torch.int8, device=dev)
    for name, q_len in (("full", 0), ("causal", S)):
        ms = time_region(torch, lambda: fused.attention_i8(q, k, vt, 1e-3, 0.05, 1.0 / 127.0, causal_q_len=q_len, out=ctx), 10, 2)
        out[f"attention_i8_fused_{name}_160x2048x2048x128"] = {"ms": ms, "scores_per_us": B * S * S / (2 if q_len else 1) / ms / 1e3}
    # decode-sized block: 16 query rows per head against 2048 keys (one pass, one to four workgroups per head)
    qd, ctxd = q[:40, :16].contiguous(), torch.empty((40, 16, D), dtype=torch.int8, device=dev)
    ms = time_region(torch, lambda: fused.attention_i8(qd, k[:40], vt[:40], 1e-3, 0.05, 1.0 / 127.0, causal_q_len=16, out=ctxd), 50, 5)
    out["attention_i8_decode_40x16x2048x128"] = {"ms": ms, "GBps": 2 * 40 * S * D / ms / 1e6}
    del q, k, vt, ctx, qd, ctxd
    # config 1: one W8A8B8O8Linear 512 x 768 x 768 (launch-latency sized: no roofline claim).  Eager
    # time includes the Python launch path; the graph replay is the kernel alone.
    from triton_int_amd.kernels import linear

    x1 = torch.randint(-127, 128, (512, 768), dtype=torch.int8, device=dev)
    w1 = torch.randint(-127, 128, (768, 768), dtype=torch.int8, device=dev)
    b1 = torch.randint(-127, 128, (768,), dtype=torch.int8, device=dev)
    al, be = torch.tensor(0.0021, device=dev), torch.tensor(0.013, device=dev)
    o1 = torch.empty((512, 768), dtype=torch.int8, device=dev)
    eager_ms = time_region(torch, lambda: linear.linear_a8_w8_b8_o8(x1, w1, b1, al, be, out=o1), 200, 20)
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    with torch.cuda.stream(side):
        linear.linear_a8_w8_b8_o8(x1, w1, b1, al, be, out=o1)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(20):
                linear.linear_a8_w8_b8_o8(x1, w1, b1, al, be, out=o1)
    torch.cuda.synchronize()
    graph_ms = time_region(torch, graph.replay, 20, 3) / 20
    out["single_linear_512x768x768"] = {"eager_us": eager_ms * 1e3, "graph_us": graph_ms * 1e3,
                                        "TOPS_graph": 2.0 * 512 * 768 * 768 / (graph_ms * 1e-3) / 1e12}
    del x1, w1, b1, o1
    # q/k/v of the linear set as three launches on one input and as one grouped launch (what the decoder
    # layer does): 768 tiles in one launch instead of three single-round launches
    xq = torch.randint(-127, 128, (2048, 4096), dtype=torch.int8, device=dev)
    w3 = torch.randint(-127, 128, (3 * 4096, 4096), dtype=torch.int8, device=dev)
    b3 = torch.randint(-127, 128, (3 * 4096,), dtype=torch.int8, device=dev)
    al3, be3 = torch.rand(3, device=dev) * 9e-3 + 1e-3, torch.rand(3, device=dev) * 9e-3 + 1e-3
    o3 = torch.empty((2048, 3 * 4096), dtype=torch.int8, device=dev)
    outs = [torch.empty((2048, 4096), dtype=torch.int8, device=dev) for _ in range(3)]

    def three():
        for i in range(3):
            linear.linear_a8_w8_b8_o8(xq, w3[i * 4096:(i + 1) * 4096], b3[i * 4096:(i + 1) * 4096], al3[i], be3[i], out=outs[i])

    # the two variants alternate, four rounds of 50 iterations, medians: a single short reading right after a
    # different workload depends on the clock and cache state that workload left (it once showed the grouped
    # launch 4 % slower; under equal conditions it is 8-10 % faster, kernel time and launch gaps)
    def grouped():
        linear.linear_group_a8_w8_b8_o8(xq, w3, b3, al3, be3, 3, out=o3)

    t3s, tgs = [], []
    for rnd in range(4):
        for fn, acc in (((three, t3s), (grouped, tgs)) if rnd % 2 == 0 else ((grouped, tgs), (three, t3s))):
            acc.append(time_region(torch, fn, 50, 5))
    t3, tg = sorted(t3s)[len(t3s) // 2], sorted(tgs)[len(tgs) // 2]
    ops3 = 3 * 2.0 * 2048 * 4096 * 4096
    out["qkv_2048x3x4096x4096"] = {"three_launches_ms": t3, "three_launches_TOPS": ops3 / t3 / 1e9,
                                   "grouped_launch_ms": tg, "grouped_launch_TOPS": ops3 / tg / 1e9,
                                   "three_launches_ms_rounds": t3s, "grouped_launch_ms_rounds": tgs}
    del xq, w3, b3, o3, outs
    # the control for "what bounds a short launch": the 2048 x 4096 x 4096 int8 GEMM of the linear set on uniform
    # random and on all-zero operands (same instructions, same bytes, less switching), back to back
    xu, wu = torch.randint(-127, 128, (2048, 4096), dtype=torch.int8, device=dev), torch.randint(-127, 128, (4096, 4096), dtype=torch.int8, device=dev)
    xz, wz = torch.zeros_like(xu), torch.zeros_like(wu)
    bq = torch.randint(-127, 128, (4096,), dtype=torch.int8, device=dev)
    alq, beq, oq = torch.tensor(0.002, device=dev), torch.tensor(0.01, device=dev), torch.empty((2048, 4096), dtype=torch.int8, device=dev)
    rec = {}
    for rnd in range(3):
        for name, (xx, ww) in (("uniform", (xu, wu)), ("zeros", (xz, wz))):
            rec.setdefault(name, []).append(time_region(torch, lambda: linear.linear_a8_w8_b8_o8(xx, ww, bq, alq, beq, out=oq), 50, 5))
    out["gemm_2048x4096x4096_uniform_vs_zero_operands"] = {
        k: {"us": sorted(v)[1] * 1e3, "TOPS": 2.0 * 2048 * 4096 * 4096 / sorted(v)[1] / 1e9} for k, v in rec.items()}
    del xu, wu, xz, wz, oq
    # a yardstick, not part of the path: the vendor library's int8 GEMM (torch._int_mm, int32 out) on
    # the fc1 shape with the same kind of operands, next to this library's int32-output linear
    try:
        M, N, K = 2048, 20480, 5120
        xa = torch.randint(-127, 128, (M, K), dtype=torch.int8, device=dev)
        wa = torch.randint(-127, 128, (N, K), dtype=torch.int8, device=dev)
        ba = torch.zeros(N, dtype=torch.int32, device=dev)
        ours = time_region(torch, lambda: linear.linear_a8_w8_b32_o32(xa, wa, ba), 20, 3)
        theirs = time_region(torch, lambda: torch._int_mm(xa, wa.t()), 20, 3)
        out["int32_out_gemm_2048x20480x5120"] = {"this_library_TOPS": 2.0 * M * N * K / ours / 1e9,
                                                 "torch_int_mm_TOPS": 2.0 * M * N * K / theirs / 1e9}
    except Exception as ex:  # torch._int_mm is a private API: absent or different elsewhere
        out["int32_out_gemm_2048x20480x5120"] = {"error": repr(ex)[:120]}
    return out


def m_sweep(torch, dev, N, K, lib, full=True):
    """The reference's own benchmark (kernels/linear.py:960-1070): int8 x int8 -> fp32 linear with an
    fp32 bias over M in {32, 64, 128, 256} and 1024 * {1..16}, weights [N, K] = [6848, 10240]; operands made
    like the reference's (`randn(fp16).to(int8)`: almost all bytes are 0, +-1, +-2, so the chip holds a much
    higher clock than on uniform int8), per-launch event timing, quantiles 0.5 / 0.2 / 0.8 as its
    `do_bench(quantiles=...)` call.  Its "triton-i8-fp16" / "-bf16" legs (bias and output in that dtype,
    :1015-1050) are timed beside the fp32 one, and one extra leg repeats the fp32 case on uniform int8
    operands (the distribution every other figure of this benchmark uses)."""
    from triton_int_amd.kernels import linear

    out = {}
    b = torch.randn((N, K), device=dev, dtype=torch.float16).to(torch.int8)
    b_uni = torch.randint(-127, 128, (N, K), dtype=torch.int8, device=dev)
    biases = {"f32": torch.randn(N, device=dev)}
    if full:
        biases["f16"] = biases["f32"].half()
        biases["bf16"] = biases["f32"].bfloat16()
    one = torch.tensor(1.0, device=dev)
    ms_list = (32, 64, 128, 256) + tuple(1024 * i for i in range(1, 17)) if full else (32, 64, 128, 256, 1024, 2048, 4096, 8192, 16384)

    def timed(a, w, bias):
        # warm-up by time, 25 ms, as the reference's do_bench does (its default), then 20 timed launches
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < SETTLE_MS:
            for _ in range(3):
                linear.linear_a8_w8_bfp32_ofp32(a, w, bias, one, one)
            torch.cuda.synchronize()
        reps = 20
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
        for s_, e_ in ev:
            s_.record()
            linear.linear_a8_w8_bfp32_ofp32(a, w, bias, one, one)
            e_.record()
        torch.cuda.synchronize()
        ts = sorted(s_.elapsed_time(e_) for s_, e_ in ev)
        return ts[len(ts) // 2], ts[len(ts) // 5], ts[4 * len(ts) // 5]

    for M in ms_list:
        a = torch.randn((M, K), device=dev, dtype=torch.float16).to(torch.int8)
        p50, p20, p80 = timed(a, b, biases["f32"])
        rec = {"ms_p50_p20_p80": [p50, p20, p80], "TOPS": 2.0 * M * N * K / p50 / 1e9,
               "kernel": lib.ti_gemm_config_name(lib.ti_gemm_last_config()).decode(), "k_splits": lib.ti_gemm_last_splits()}
        for name in ("f16", "bf16"):
            if name in biases:
                q50, _, _ = timed(a, b, biases[name])
                rec[f"ms_p50_{name}"] = q50
                rec[f"TOPS_{name}"] = 2.0 * M * N * K / q50 / 1e9
        if full:
            au = torch.randint(-127, 128, (M, K), dtype=torch.int8, device=dev)
            u50, _, _ = timed(au, b_uni, biases["f32"])
            rec["ms_p50_uniform_int8"] = u50
            rec["TOPS_uniform_int8"] = 2.0 * M * N * K / u50 / 1e9
        out[f"M{M}"] = rec
    return out


def cpu_baseline_rows(torch, budget_s=4.0):
    """CPU emulation (torch on the host cores) of the HBM-bound kernels on bounded samples of their
    benchmark shapes: dq + add + LayerNormQ (functional/fused.py:6-15), GELU-quant, one head of Q.K^T,
    and of the single 512 x 768 x 768 int8 linear."""
    import torch.nn.functional as F

    from oracle import cpu_emulation as E

    torch.set_num_threads(min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16"))))
    g = torch.Generator().manual_seed(7)
    out = {"cores": torch.get_num_threads()}

    def timed(fn, unit_bytes, what):
        fn()
        n, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < budget_s / 3 or n == 0:
            fn()
            n += 1
        el = (time.perf_counter() - t0) / n
        return {"GBps": unit_bytes / el / 1e9, "ms": el * 1e3, "sample": what}

    rows, cols = 1024, 5120
    acc = torch.randint(-2**20, 2**20 + 1, (rows, cols), dtype=torch.int32, generator=g)
    res, gam, bet = torch.randn((rows, cols), generator=g), torch.randn(cols, generator=g) * 2 + 20, torch.randn(cols, generator=g) * 2
    out["dq_add_layernorm_q"] = timed(lambda: E.dq_add_layernorm_q(acc, 1e-5, res, gam, bet, 1e-5), rows * cols * 13,
                                      f"{rows} of 8192 rows x {cols}")
    xg = torch.randn((512, 20480), generator=g)
    out["gelu_q"] = timed(lambda: torch.clamp(torch.round(F.gelu(xg, approximate="tanh") * 20.0), -128, 127).to(torch.int8),
                          xg.numel() * 5, "512 of 8192 rows x 20480")
    q = torch.randint(-127, 128, (1, 512, 128), dtype=torch.int8, generator=g)
    k = torch.randint(-127, 128, (1, 2048, 128), dtype=torch.int8, generator=g)
    r = timed(lambda: E.bmm_o8(q, k, 1e-3), 512 * 128 + 2048 * 128 + 512 * 2048, "512 query rows of one of 160 heads, 2048 keys")
    r["TOPS"] = 2.0 * 512 * 2048 * 128 / (r["ms"] * 1e-3) / 1e12
    out["bmm_qk_s8"] = r
    x1 = torch.randint(-127, 128, (512, 768), dtype=torch.int8, generator=g)
    w1 = torch.randint(-127, 128, (768, 768), dtype=torch.int8, generator=g)
    b1 = torch.randint(-127, 128, (768,), dtype=torch.int8, generator=g)
    r = timed(lambda: E.linear_o8(x1, w1, b1, 0.0021, 0.013), 512 * 768 * 2 + 768 * 768 + 768, "the whole 512 x 768 x 768 linear")
    r["TOPS"] = 2.0 * 512 * 768 * 768 / (r["ms"] * 1e-3) / 1e12
    out["single_linear_512x768x768"] = r
    return out


def attention_mismatch(torch, dev):
    """The one-kernel attention against the BMM -> softmax -> BMM chain on the layer's shape (40 heads,
    2048 x 2048, causal): rows of the context that differ and the largest difference."""
    from triton_int_amd.kernels import bmm, fused

    q, k = (torch.randint(-127, 128, (40, 2048, 128), dtype=torch.int8, device=dev) for _ in range(2))
    vt = torch.randint(-127, 128, (40, 128, 2048), dtype=torch.int8, device=dev)
    one = fused.attention_i8(q, k, vt, 1e-3, 0.05, 1.0 / 127.0, causal_q_len=2048)
    chain = bmm.bmm_s8t_s8n_s8t(fused.softmax_q(bmm.bmm_s8t_s8n_s8t(q, k, 1e-3), 0.05, causal_q_len=2048), vt, 1.0 / 127.0)
    d = (one.int() - chain.int()).abs()
    return {"rows": 40 * 2048, "rows_differing": int((d.amax(dim=-1) > 0).sum()), "max_step": int(d.max())}


def decoder_layer_ms(torch, dev):
    """W8A8 OPT-13B-shaped decoder layer (hidden 5120, 40 heads, FFN 20480), random int8 weights:
    prefill (batch 1, seq 2048) and decode (16 tokens against a 2048-long int8 KV).  Two layers with
    different weights alternate so that no weight is cache-resident."""
    from triton_int_amd.nn.opt import W8A8OPTDecoderLayer

    layers = [W8A8OPTDecoderLayer().randomize(seed=i).to(dev) for i in range(2)]
    x = torch.randn((1, 2048, 5120), device=dev)
    state = {"i": 0}

    def prefill():
        state["i"] ^= 1
        layers[state["i"]](x)

    out = {"prefill_1x2048_ms": time_region(torch, prefill, 10, 2)}
    # the same two layers replayed from a HIP graph: the nine launches of a layer back to back, without the
    # bubbles the Python launch path leaves behind the short kernels
    pgraph, pside = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    with torch.cuda.stream(pside):
        prefill(); prefill()
        torch.cuda.synchronize()
        with torch.cuda.graph(pgraph, stream=pside):
            prefill(); prefill()
    torch.cuda.synchronize()
    out["prefill_1x2048_graph_ms"] = time_region(torch, pgraph.replay, 10, 2) / 2
    del pgraph
    # per-stage breakdown of the prefill, in sequence: stream events between the stages of the same
    # alternating forward passes (weights cold, clocks as the whole layer holds them)
    reps, marks = 8, []

    def mark(name):
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        marks.append((name, ev))

    for _ in range(reps):
        state["i"] ^= 1
        mark("start")
        layers[state["i"]](x, _mark=mark)
    torch.cuda.synchronize()
    br = {}
    for (n0, e0), (n1, e1) in zip(marks, marks[1:]):
        if n1 != "start":
            br[n1] = br.get(n1, 0.0) + e0.elapsed_time(e1) / reps
    out["prefill_breakdown_ms"] = br
    out["prefill_breakdown_sum_ms"] = sum(br.values())
    # ideal: GEMM/BMM ops at the 5.0 POP/s peak, row kernels at 8 TB/s on their algorithmic bytes
    S_, H_, F_ = 2048, 5120, 20480
    ideal = 1374.4e9 / 5.0e15 + (S_ * H_ * 5 + S_ * H_ * 13 + 40 * S_ * S_ * 2) / 8.0e12
    out["prefill_ideal_ms"] = ideal * 1e3
    out["prefill_ideal_over_measured"] = ideal * 1e3 / out["prefill_1x2048_ms"]
    kc = torch.randint(-127, 128, (40, 2048, 128), dtype=torch.int8, device=dev)
    vc = torch.randint(-127, 128, (40, 128, 2048), dtype=torch.int8, device=dev)
    xd = torch.randn((1, 16, 5120), device=dev)

    def decode():
        state["i"] ^= 1
        layers[state["i"]](xd, kv_cache=(kc, vc))

    out["decode_16tok_kv2048_eager_ms"] = time_region(torch, decode, 20, 3)
    # the same two layers replayed from a HIP graph: launch overhead removed
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    with torch.cuda.stream(side):
        decode(); decode()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            decode(); decode()
    torch.cuda.synchronize()
    out["decode_16tok_kv2048_graph_ms"] = time_region(torch, graph.replay, 10, 2) / 2
    out["gemm_bmm_ops_prefill"] = 1374.4e9
    out["prefill_tops"] = 1374.4e9 / (out["prefill_1x2048_ms"] * 1e-3) / 1e12
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU emulation baseline")
    ap.add_argument("--no-extra", action="store_true", help="skip the row-kernel / BMM extras")
    ap.add_argument("--qkv-only", type=int, default=0, metavar="N",
                    help="run the q/k/v projections of the linear set N times as three launches and N times as one "
                         "grouped launch, print times and held clocks, and exit: the program profiled for the "
                         "grouped-launch counter summary")
    ap.add_argument("--decode-gemm-only", action="store_true",
                    help="run 24 launches of the M=16 decode GEMM 20480 x 5120 (int8 out, weights rotated through "
                         "6 matrices) and exit: the program profiled for the decode GEMM counter summary")
    ap.add_argument("--attention-only", action="store_true",
                    help="run 3 full and 3 causal launches of the fused attention kernel (40 heads x 2048 x 2048 "
                         "x 128) and exit: the program profiled for the attention counter summary")
    ap.add_argument("--bmm-qk-only", action="store_true",
                    help="run 4 launches of the Q.K^T BMM to int8 (160 x 2048 x 2048 x 128) and exit: the program "
                         "profiled for the Q.K^T counter summary")
    ap.add_argument("--rownorm-only", action="store_true",
                    help="run 6 launches of LayerNormQ and 3 of dq + add + LayerNormQ on 8192 x 5120 and exit: the "
                         "program profiled for the row-norm counter summary")
    ap.add_argument("--settle-ms", type=float, default=40.0,
                    help="during set-up, before the warm-up steps, run untimed steps for this long (each one timed "
                         "on its own and reported under \"cold_start\"): the first ~15 ms of heavy work after a "
                         "process starts are a transient of the chip's power management (three steps at the boost "
                         "clock, then ~25 steps 10-25 %% slower than the level it settles on); 0 turns it off")
    ap.add_argument("--calib-copy-mb", type=int, default=0,
                    help="before the timed region, run 4 device-to-device copies of this many MiB: a kernel of "
                         "known traffic to scale rocprofv3's FETCH_SIZE / WRITE_SIZE readings with")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (every op shards over "
                 "token rows / heads with no exchange step); run with --gpus 1")

    import torch

    from triton_int_amd import _lib

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    lib = _lib.lib()  # raises if the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.qkv_only:
        # q/k/v of the linear set (3 x 2048 x 4096 x 4096, int8 out) as three launches and as one grouped launch,
        # each looped `--qkv-only` times with the shader clock sampled meanwhile; prints one JSON line
        import glob
        import threading

        from triton_int_amd.kernels import linear

        xq = torch.randint(-127, 128, (2048, 4096), dtype=torch.int8, device=dev)
        w3 = torch.randint(-127, 128, (3 * 4096, 4096), dtype=torch.int8, device=dev)
        b3 = torch.randint(-127, 128, (3 * 4096,), dtype=torch.int8, device=dev)
        al3, be3 = torch.rand(3, device=dev) * 9e-3 + 1e-3, torch.rand(3, device=dev) * 9e-3 + 1e-3
        o3 = torch.empty((2048, 3 * 4096), dtype=torch.int8, device=dev)
        outs = [torch.empty((2048, 4096), dtype=torch.int8, device=dev) for _ in range(3)]
        ws = [w3[i * 4096:(i + 1) * 4096] for i in range(3)]
        bs = [b3[i * 4096:(i + 1) * 4096] for i in range(3)]

        def three():
            for i in range(3):
                linear.linear_a8_w8_b8_o8(xq, ws[i], bs[i], al3[i], be3[i], out=outs[i])

        def grouped():
            linear.linear_group_a8_w8_b8_o8(xq, w3, b3, al3, be3, 3, out=o3)

        sclk_file = _find_sclk_file(torch, glob)
        res = {"three_launches": {"ms": [], "sclk_mhz": []}, "grouped_launch": {"ms": [], "sclk_mhz": []}}
        # the two variants alternate, six rounds of N iterations each: the order within a round and the state
        # the previous round left the chip in (clock, caches) weigh on a single reading
        for rnd in range(6):
            for name, fn in ((("three_launches", three), ("grouped_launch", grouped)) if rnd % 2 == 0 else
                             (("grouped_launch", grouped), ("three_launches", three))):
                clocks, on = [], {"v": True}

                def sample():
                    while on["v"]:
                        mhz = _read_sclk_mhz(sclk_file)
                        if mhz:
                            clocks.append(mhz)
                        time.sleep(0.002)

                th = threading.Thread(target=sample)
                th.start()
                ms = time_region(torch, fn, args.qkv_only, 5)
                on["v"] = False
                th.join()
                res[name]["ms"].append(round(ms, 5))
                res[name]["sclk_mhz"].append(sorted(clocks)[len(clocks) // 2] if clocks else None)
        for v in res.values():
            med = sorted(v["ms"])[len(v["ms"]) // 2]
            v["ms_median"] = med
            v["TOPS_median"] = 3 * 2.0 * 2048 * 4096 * 4096 / med / 1e9
        print(json.dumps({"qkv_2048x3x4096x4096": res}))
        return
    if args.decode_gemm_only:
        from triton_int_amd.kernels import linear

        ws = [torch.randint(-127, 128, (20480, 5120), dtype=torch.int8, device=dev) for _ in range(6)]
        x = torch.randint(-127, 128, (16, 5120), dtype=torch.int8, device=dev)
        b8 = torch.randint(-127, 128, (20480,), dtype=torch.int8, device=dev)
        al, be = torch.tensor(0.002, device=dev), torch.tensor(0.01, device=dev)
        for i in range(24):
            linear.linear_a8_w8_b8_o8(x, ws[i % 6], b8, al, be)
        torch.cuda.synchronize()
        return
    if args.rownorm_only:
        from triton_int_amd.kernels import fused

        rows, cols = 8192, 5120
        xs = [torch.randn(rows, cols, device=dev) for _ in range(2)]
        gam, bet = torch.randn(cols, device=dev) * 2 + 20, torch.randn(cols, device=dev) * 2
        acc = torch.randint(-2**20, 2**20 + 1, (rows, cols), dtype=torch.int32, device=dev)
        for i in range(6):
            fused.layer_norm_fwd_fused_single_pass_q(xs[i & 1], gam, bet, 1e-5)
        for i in range(3):
            fused.dq_add_layernorm_q(acc, 1e-5, xs[i & 1], gam, bet, 1e-5)
        torch.cuda.synchronize()
        return
    if args.bmm_qk_only:
        from triton_int_amd.kernels import bmm

        q, k = (torch.randint(-127, 128, (160, 2048, 128), dtype=torch.int8, device=dev) for _ in range(2))
        sc = torch.empty((160, 2048, 2048), dtype=torch.int8, device=dev)
        for _ in range(4):
            bmm.bmm_s8t_s8n_s8t(q, k, 1e-3, out=sc)
        torch.cuda.synchronize()
        return
    if args.attention_only:
        from triton_int_amd.kernels import fused

        q, k = (torch.randint(-127, 128, (40, 2048, 128), dtype=torch.int8, device=dev) for _ in range(2))
        vt = torch.randint(-127, 128, (40, 128, 2048), dtype=torch.int8, device=dev)
        ctx = torch.empty_like(q)
        for q_len in (0, 2048):
            for _ in range(3):
                fused.attention_i8(q, k, vt, 1e-3, 0.05, 1.0 / 127.0, causal_q_len=q_len, out=ctx)
        torch.cuda.synchronize()
        return
    layers = build_linear_set(torch, dev)
    # a second set of weights and activations (other seed): the timed steps alternate between the two,
    # 2 x 264 MB of operands, so that no step finds its operands in the 256 MB Infinity Cache
    layers_b = build_linear_set(torch, dev, seed=4321)
    # which kernel does each GEMM run on?  (one untimed pass)
    keyed = []
    for name, m, x in layers:
        y = m(x)
        cfg = lib.ti_gemm_last_config()
        kernel = f"{lib.ti_gemm_config_name(cfg).decode()}/{str(y.dtype).replace('torch.', '')}"
        ops = 2.0 * x.shape[0] * m.weight.shape[0] * m.weight.shape[1]
        keyed.append((kernel, name, m, x, ops))
    groups = {}
    for kernel, name, m, x, ops in keyed:
        groups.setdefault(kernel, []).append((name, m, x, ops))
    dominant = max(groups, key=lambda k: sum(o for *_, o in groups[k]))
    order = groups[dominant] + [e for k, v in groups.items() if k != dominant for e in v]
    n_dom = len(groups[dominant])
    total_ops = sum(o for *_, o in order)

    by_name_b = {name: (m, x) for name, m, x in layers_b}
    order_b = [(name, *by_name_b[name], ops) for name, _, _, ops in order]
    flip = {"i": 0}

    def step(ev=None):
        flip["i"] ^= 1
        if ev is not None:
            ev[0].record()
        for i, (_, m, x, _) in enumerate(order if flip["i"] else order_b):
            m(x)
            if ev is not None and i == n_dom - 1:
                ev[1].record()

    if args.calib_copy_mb > 0:
        src = torch.randint(-127, 128, (args.calib_copy_mb << 20,), dtype=torch.int8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # Settling (set-up, untimed): what a step costs in the first milliseconds of heavy work of a process is a
    # property of the chip's power management, not of the kernels, and is reported separately.
    cold = None
    sclk_samples = []
    if args.settle_ms > 0:
        # the shader clock the chip holds under the steps: the driver's sysfs file read from a thread, here and
        # not in the timed region (2 000 reads a second cost the timed steps 4-5 %)
        import glob
        import threading

        sclk_file, sampling = _find_sclk_file(torch, glob), {"on": True}

        def sample_sclk():
            time.sleep(0.02)  # past the transient
            while sampling["on"] and len(sclk_samples) < 400:
                mhz = _read_sclk_mhz(sclk_file)
                if mhz:
                    sclk_samples.append(mhz)
                time.sleep(0.001)

        th = threading.Thread(target=sample_sclk)
        if sclk_file:
            th.start()
        marks = [torch.cuda.Event(enable_timing=True) for _ in range(401)]
        n_settle, t_s = 0, time.perf_counter()
        marks[0].record()
        while n_settle < 400 and (time.perf_counter() - t_s) * 1e3 < args.settle_ms:
            for _ in range(10):  # launches are asynchronous: wait per block so that the limit is device time
                step()
                n_settle += 1
                marks[n_settle].record()
            torch.cuda.synchronize()
        sampling["on"] = False
        if sclk_file:
            th.join()
        ts = [marks[i].elapsed_time(marks[i + 1]) for i in range(n_settle)]
        blocks = [ts[i:i + 5] for i in range(0, len(ts), 5)]
        cold = {"steps": n_settle,
                "tops_per_block_of_5_steps": [round(total_ops / (sum(b) / len(b) * 1e-3) / 1e12) for b in blocks],
                "note": "untimed set-up steps before the warm-up, from the first heavy launches of the process on "
                        "(device time per block of 5 steps): boost clock, then the power management's "
                        "over-correction, then the level the timed steps run at"}
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(events[i])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    dom_ms = sum(a.elapsed_time(b) for a, b in events) / args.steps  # per step, all launches of the dominant kernel
    # device time of whole steps: start event of step i to start event of step i+1
    step_ms = sorted(events[i][0].elapsed_time(events[i + 1][0]) for i in range(args.steps - 1))
    dom_ops = sum(o for *_, o in groups[dominant])
    achieved = dom_ops / (dom_ms * 1e-3) / 1e12

    result = {
        "metric": METRIC,
        "value": total_ops / (ms_per_step * 1e-3) / 1e12,
        "unit": "TOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "ms_per_step_device_p20_p50_p80": ([step_ms[int(q * (len(step_ms) - 1))] for q in (0.2, 0.5, 0.8)]
                                           if step_ms else None),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {
            "workload": "OPT-6.7B W8A8 linear set, M=2048 tokens (4x512), hidden 4096: q/k/v/out W8A8B8O8 "
                        "4096x4096, fc1 4096->16384 GELU-quant int8, fc2 16384->4096 fp32 out",
            "gemms_per_step": len(order),
            "operand_sets": "2 sets of weights and activations (2 x 264 MB) alternate between steps: operands come from HBM, "
                            "not from the 256 MB Infinity Cache",
            "int8_ops_per_step": total_ops,
            "kernels": {k: [n for n, *_ in v] for k, v in groups.items()},
        },
        "roofline": {
            "bound": "mfma",
            "kernel": dominant,
            "achieved": achieved,
            "peak": INT8_PEAK_TOPS,
            "unit": "TFLOP/s",
            "frac": achieved / INT8_PEAK_TOPS,
            "traffic": traffic_from_profile(dominant)[0],
            "traffic_source": traffic_from_profile(dominant)[1],
            "algorithmic_bytes": sum(x.numel() + m.weight.numel() + x.shape[0] * m.weight.shape[0]
                                     for _, m, x, _ in groups[dominant]) / n_dom,
            "launches_per_step": n_dom,
            "avg_launch_us": dom_ms * 1e3 / n_dom,
            "sclk_mhz_during_settling_steps": (sorted(sclk_samples)[len(sclk_samples) // 2] if sclk_samples else None),
            "ops_per_launch": dom_ops / n_dom,
        },
    }
    peak_rand = mfma_issue_peak(torch, lib, 1)
    peak_const = mfma_issue_peak(torch, lib, 0)
    result["roofline"]["measured_mfma_issue_peak_random_operands"] = peak_rand
    result["roofline"]["measured_mfma_issue_peak_constant_operands"] = peak_const
    result["roofline"]["frac_of_measured_issue_peak"] = achieved / peak_rand
    if cold is not None:
        result["cold_start"] = cold
    if not args.no_extra:
        result["extra"] = extras(torch, dev)
        result["extra"]["attention_i8_fused_vs_chain_40x2048x2048"] = attention_mismatch(torch, dev)
        result["extra"]["m_sweep_K10240_N6848"] = m_sweep(torch, dev, 6848, 10240, lib)
        result["extra"]["m_sweep_K5120_N5120"] = m_sweep(torch, dev, 5120, 5120, lib, full=False)
        result["extra"]["opt13b_decoder_layer"] = decoder_layer_ms(torch, dev)
        result["extra"]["sustained_fc2_2048x4096x16384"] = sustained_clock(torch, dev)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(torch, layers)
        result["cpu_baseline"]["row_kernels"] = cpu_baseline_rows(torch)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
