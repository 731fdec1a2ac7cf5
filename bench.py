#!/usr/bin/env python3
"""Benchmark of the diagonal-tiled MXFP attention path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c4|c1|c5] [--no-cpu-baseline]

One "step" is one full pass of the hot path over one synthetic batch already resident in HBM:
MX-quantize Q and K (E2M1 + E4M3 in one pass each), repack V, fused attention (diagonal tiles MXFP8,
off-diagonal MXFP4, causal, GQA).  Prints ONE JSON line: whole-step attention TFLOP/s
(FlashAttention convention 2*B*Hq*N^2*D for causal), the roofline of the dominant kernel (the fused
attention kernel, timed alone with HIP events on its launch stream), secondary figures for the
quantizer and the standalone block-scaled GEMM and for the long-context configuration (N = 131072), and the CPU
oracle timed on the host cores on a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "mp-sparse-attn_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

import torch  # noqa: E402

# published MI355X dense peaks
PEAK_FP4_TFLOPS = 10100.0
PEAK_FP8_TFLOPS = 5000.0
PEAK_BF16_TFLOPS = 2500.0
PEAK_HBM_GBS = 8000.0

# HBM-side bytes per launch of the fused attention kernel (L2 <-> fabric) come from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE runs of `bench.py --only attn`, each scaled by the same counter's reading for a 1 GiB copy
# (`bench.py --only copy`).  The summary file carries them in lines of the form
#   #@ traffic workload=c3 mode=diag read_bytes=... write_bytes=... commit=...
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "attn_c3_hbm_traffic.txt")


def measured_traffic(workload, mode):
    """(bytes per launch, commit it was measured at) from the profile summary, or (None, None)."""
    try:
        with open(TRAFFIC_FILE) as f:
            for line in f:
                if not line.startswith("#@ traffic"):
                    continue
                kv = dict(item.split("=", 1) for item in line.split()[2:])
                if kv.get("workload") == workload and kv.get("mode") == mode:
                    return float(kv["read_bytes"]) + float(kv["write_bytes"]), kv.get("commit")
    except (OSError, ValueError, KeyError):
        pass
    return None, None


WORKLOADS = {
    # name: (B, Hq, Hkv, N, D, tile, seed, description)
    "c1": (1, 8, 8, 1024, 64, 64, 0, "C1 B1 H8 N1024 D64 causal tile64 diag"),
    "c3": (1, 32, 8, 8192, 128, 128, 2, "C3 llama3-8b prefill B1 Hq32 Hkv8 N8192 D128 causal tile128 diag(MXFP8)/offdiag(MXFP4), outlier channels"),
    "c4": (1, 32, 8, 131072, 128, 128, 3, "C4 long-context prefill B1 Hq32 Hkv8 N131072 D128 causal tile128 diag, outlier channels"),
    "c5": (1, 40, 40, 32760, 128, 128, 4, "C5 video-DiT B1 H40 N32760 (21 frames x 1560) D128 non-causal tile128 diag, sigma 0.5 + per-frame offsets"),
}
NON_CAUSAL = {"c5"}
PLAIN_DRAWS = {"c1"}          # N(0,1) without outlier channels
ROUTE_THRESH_DEFAULT = 0.97        # on the C5 inputs: about 8 % of the tiles in MXFP8 (see profiles/attn_c5_router_study.txt)


def make_inputs(B, Hq, Hkv, N, D, seed, device, dit_frames=0, outliers=True):
    """The workload's q, k, v: drawn on the CPU from one seeded generator in float32, cast to bf16, copied to the device
    -- bit for bit the tensors the parity tests hand to the CPU oracle and to the kernels (tests/conftest.py::make_qkv;
    the video-DiT offsets as in tests/test_gpu_route.py).  Causal workloads: N(0,1) draws, and (``outliers``: C3, C4) per
    head one channel (1 % of 128, rounded) of q and of k multiplied by 20.  ``dit_frames``: sigma 0.5 draws plus one sigma-0.5 offset per
    frame and channel on q and on k (generator seed + 1)."""
    g = torch.Generator().manual_seed(seed)
    sigma = 0.5 if dit_frames else 1.0
    q = torch.randn(B, Hq, N, D, generator=g) * sigma
    k = torch.randn(B, Hkv, N, D, generator=g) * sigma
    v = torch.randn(B, Hkv, N, D, generator=g) * sigma
    if outliers and not dit_frames:
        n_out = max(1, round(0.01 * D))
        for t, H in ((q, Hq), (k, Hkv)):
            for h in range(H):
                idx = torch.randint(0, D, (n_out,), generator=g)
                t[:, h, :, idx] *= 20.0
    q, k, v = q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16)
    if dit_frames:
        g2 = torch.Generator().manual_seed(seed + 1)
        per = -(-N // dit_frames)
        frame = torch.arange(N) // per
        for t in (q, k):
            off = 0.5 * torch.randn(dit_frames, 1, D, generator=g2)
            t += off[frame].reshape(1, 1, N, D).to(t.dtype)
    return q.to(device), k.to(device), v.to(device)


def composite_peak_tflops(nt, causal=True):
    """Bound when Q.K^T runs at the MXFP4 / MXFP8 peak (diagonal share 2/(nt+1) of the visited tiles, 1/nt
    without the causal mask) and P.V at the bf16 peak: half of the FLOPs each."""
    diag = 2.0 / (nt + 1) if causal else 1.0 / nt
    t = 0.5 * ((1 - diag) / PEAK_FP4_TFLOPS + diag / PEAK_FP8_TFLOPS) + 0.5 / PEAK_BF16_TFLOPS
    return 1.0 / t


def time_events(fn, iters):
    """Average duration (ms) of fn() over iters launches, HIP events on torch's current stream -- the stream
    libmpsa launches on."""
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def wait_for_device():
    """Spin on an event until the stream has drained, then synchronize: the host does not sleep, so its wake-up
    latency (about a tenth of a millisecond) stays out of short timed regions."""
    ev = torch.cuda.Event()
    ev.record()
    while not ev.query():
        pass
    torch.cuda.synchronize()


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(q, k, v, tile, D, causal=True):
    """The CPU oracle (a port of the reference's fake-quant path) on the first 8192 positions of the workload
    (all of it for C1/C3), every head, on the host threads this process may use."""
    import oracle as O
    threads = max(1, min(int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)), os.cpu_count() or 1))
    torch.set_num_threads(threads)
    Hq, Hkv = q.shape[1], k.shape[1]
    group = Hq
    n = min(q.shape[2], 8192)
    qs = q[:, :, :n].cpu()
    ks = k[:, :, :n].cpu()
    vs = v[:, :, :n].cpu()
    t0 = time.perf_counter()
    O.attn_mx(qs, ks, vs, tile=tile, causal=causal, mode="diag")
    dt = time.perf_counter() - t0
    flops = (2.0 if causal else 4.0) * qs.shape[0] * group * n * n * D
    return {
        "value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
        "cpu_model": cpu_model(),
        "sample": f"oracle.attn_mx (quantize+dequantize+tiled attention, torch CPU) on {group} query heads / {Hkv} KV heads, "
                  f"N={n}, D={D}, {'causal' if causal else 'non-causal'}, diag mode: {dt:.2f} s",
        "seconds": dt,
    }


def secondary_c4(device):
    """The long-context configuration (N = 131072) next to the headline line: fused attention kernel (Q quantized in
    the kernel), whole step, and the full operand preparation (Q, K, V) on 2.9 GB of traffic -- far beyond the 256 MB
    last-level cache, i.e. the quantizer's out-of-cache bandwidth."""
    from ours.mxfp_attn_kernel import prepare_operands, attention_from_operands
    B, Hq, Hkv, N, D, tile, seed, desc = WORKLOADS["c4"]
    q, k, v = make_inputs(B, Hq, Hkv, N, D, seed, device)
    out = torch.empty((B, Hq, N, D), dtype=torch.bfloat16, device=device)
    ops = prepare_operands(q, k, v, tile, "diag", fuse_q=True)
    attention_from_operands(ops, out, True)
    torch.cuda.synchronize()
    iters = 10
    attn_ms = time_events(lambda: attention_from_operands(ops, out, True), iters)
    # the operand preparation with Q included: 2.9 GB of traffic, the quantizer's out-of-cache figure
    full = prepare_operands(q, k, v, tile, "diag")
    prep_ms = time_events(lambda: prepare_operands(q, k, v, tile, "diag", reuse=full), iters)
    del full

    def step():
        attention_from_operands(prepare_operands(q, k, v, tile, "diag", reuse=ops, fuse_q=True), out, True)

    step()
    wait_for_device()
    t0 = time.perf_counter()
    for _ in range(iters):
        step()
    wait_for_device()
    step_ms = (time.perf_counter() - t0) * 1e3 / iters
    flops = 2.0 * B * Hq * N * N * D
    comp = composite_peak_tflops(N // tile, True)
    # the preparation reads q, k, v (2 B/elem) and writes both code sets + scales of q and k and the V tiles
    prep_bytes = (q.numel() + k.numel()) * (2 + 0.5 + 1 + 2 / 32) + v.numel() * 4
    ktf, stf = flops / attn_ms / 1e9, flops / step_ms / 1e9
    return {
        "workload": desc, "steps": iters,
        "kernel_ms": round(attn_ms, 3), "kernel_TFLOP/s": round(ktf, 1), "kernel_frac_mxfp4_peak": round(ktf / PEAK_FP4_TFLOPS, 5),
        "kernel_frac_composite": round(ktf / comp, 5),
        "ms_per_step": round(step_ms, 3), "TFLOP/s": round(stf, 1), "frac_mxfp4_peak": round(stf / PEAK_FP4_TFLOPS, 5),
        "frac_composite": round(stf / comp, 5),
        "prepare_ms": round(prep_ms, 4), "prepare_GB/s": round(prep_bytes / prep_ms / 1e6, 1),
        "prepare_frac_hbm": round(prep_bytes / prep_ms / 1e6 / PEAK_HBM_GBS, 4), "prepare_bytes": prep_bytes,
    }


def secondary_c5(device):
    """The video-DiT configuration (non-causal, N = 32760, 40 heads) next to the headline line: the diag mode's kernel and
    whole step, and the routed mode (tile router on the scale bytes + routed attention) at the default thresholds with
    the shares of tiles it sends to each precision."""
    from ours.mxfp_attn_kernel import prepare_operands, attention_from_operands, route_tiles, q_fusable
    B, Hq, Hkv, N, D, tile, seed, desc = WORKLOADS["c5"]
    q, k, v = make_inputs(B, Hq, Hkv, N, D, seed, device, 21)
    out = torch.empty((B, Hq, N, D), dtype=torch.bfloat16, device=device)
    flops = 4.0 * B * Hq * N * N * D
    comp = composite_peak_tflops((N + tile - 1) // tile, False)
    iters = 10
    res = {"workload": desc, "steps": iters}
    for mode in ("diag", "routed"):
        routed = mode == "routed"
        # as the public entry point does: Q stays unquantized where the attention kernel quantizes it itself (the router
        # reads Q's scale bytes, so a routed step quantizes Q beforehand)
        fuse = not routed and q_fusable(q, k, tile, mode, False)
        ops = prepare_operands(q, k, v, tile, mode, fuse_q=fuse)
        route = route_tiles(ops, False, ROUTE_THRESH_DEFAULT, None) if routed else None
        attention_from_operands(ops, out, False, route=route)
        torch.cuda.synchronize()
        attn_ms = time_events(lambda: attention_from_operands(ops, out, False, route=route), iters)

        def step():
            o = prepare_operands(q, k, v, tile, mode, reuse=ops, fuse_q=fuse)
            r = route_tiles(o, False, ROUTE_THRESH_DEFAULT, None) if routed else None
            attention_from_operands(o, out, False, route=r)

        step()
        wait_for_device()
        t0 = time.perf_counter()
        for _ in range(iters):
            step()
        wait_for_device()
        step_ms = (time.perf_counter() - t0) * 1e3 / iters
        ktf, stf = flops / attn_ms / 1e9, flops / step_ms / 1e9
        r = {"kernel_ms": round(attn_ms, 3), "kernel_TFLOP/s": round(ktf, 1), "kernel_frac_mxfp4_peak": round(ktf / PEAK_FP4_TFLOPS, 5),
             "ms_per_step": round(step_ms, 3), "TFLOP/s": round(stf, 1), "frac_mxfp4_peak": round(stf / PEAK_FP4_TFLOPS, 5)}
        if routed:
            cls = route[0]
            visited = float((cls != 255).sum())
            r["route_thresh"] = ROUTE_THRESH_DEFAULT
            r["tile_shares"] = {"mxfp8": round(float((cls == 2).sum()) / visited, 4), "mxfp4": round(float((cls == 1).sum()) / visited, 4),
                                "skipped": round(float((cls == 0).sum()) / visited, 4)}
        else:
            r["kernel_frac_composite"] = round(ktf / comp, 5)
        res[mode] = r
        del ops, route
    return res


def secondary(device, quick):
    """Quantizer GB/s on the 8192x8192 GEMM operand and block-scaled GEMM TFLOP/s at 8192^3."""
    from ours import _lib
    from ours.quant_mxint8 import quantize_mx, quantize_mx_dual
    from ours.block_scaled_matmul import block_scaled_matmul, make_configs, pack_scale_5d
    out = {}
    M = N = K = 8192
    g = torch.Generator(device=device).manual_seed(1)
    a = torch.randn(M, K, generator=g, device=device).to(torch.bfloat16)[None, None]
    b = torch.randn(N, K, generator=g, device=device).to(torch.bfloat16)[None, None]
    it = 5 if quick else 100         # long enough for the clocks to settle (a short burst of GEMMs runs ~8 % faster)
    for name, fmt, bpe in (("quant_e2m1", _lib.FMT_E2M1, 2 + 0.5 + 1 / 32), ("quant_e4m3", _lib.FMT_E4M3, 2 + 1 + 1 / 32)):
        quantize_mx(a, 1.0, fmt)
        ms = time_events(lambda: quantize_mx(a, 1.0, fmt), it)
        gbs = M * K * bpe / ms / 1e6
        out[name] = {"GB/s": round(gbs, 1), "frac_hbm": round(gbs / PEAK_HBM_GBS, 4), "ms": round(ms, 4)}
    quantize_mx_dual(a, 1.0)
    ms = time_events(lambda: quantize_mx_dual(a, 1.0), it)
    gbs = M * K * (2 + 0.5 + 1 + 2 / 32) / ms / 1e6
    out["quant_dual"] = {"GB/s": round(gbs, 1), "frac_hbm": round(gbs / PEAK_HBM_GBS, 4), "ms": round(ms, 4)}
    # "mixed" = the reference's 8-bit A against 4-bit B (ours/block_scaled_matmul.py:318-324); the matrix instruction runs
    # it at the 8-bit rate
    for bst, fmt, fmt_b, peak in (("mxfp4", _lib.FMT_E2M1, _lib.FMT_E2M1, PEAK_FP4_TFLOPS), ("mxfp8", _lib.FMT_E4M3, _lib.FMT_E4M3, PEAK_FP8_TFLOPS),
                                  ("mixed", _lib.FMT_E4M3, _lib.FMT_E2M1, PEAK_FP8_TFLOPS)):
        ac, asc = quantize_mx(a, 1.0, fmt)
        bc, bsc = quantize_mx(b, 1.0, fmt_b)
        cfg = make_configs(bst)
        # scales in the reference's packed form, packed outside the timed region as in the reference's own benchmark
        # (ours/block_scaled_matmul.py:299-406 packs, :409-441 times the matmul alone)
        args = (ac[0, 0], pack_scale_5d(asc[0, 0]), bc[0, 0], pack_scale_5d(bsc[0, 0]), torch.bfloat16, M, N, K, cfg)
        block_scaled_matmul(*args)
        ms = time_events(lambda: block_scaled_matmul(*args), it)
        tf = 2.0 * M * N * K / ms / 1e9
        out["gemm_" + bst] = {"TFLOP/s": round(tf, 1), "frac_peak": round(tf / peak, 4), "ms": round(ms, 4)}
    return out


def mfma_stream_rates(device, seconds=0.05):
    """Sustained rate of a register-resident matrix-instruction stream (two waves per SIMD, every CU): constant
    operands and operands with random bits, for the bf16, MXFP4 and MXFP8 instructions the path uses."""
    import ctypes
    from ours import _lib
    # the measurement kernel lives in a shared object of its own, next to the library (built by build.py)
    path = os.path.join(os.path.dirname(_lib.LIB_PATH), "libmpsa_bench.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build it with `python mp-sparse-attn_amd/build.py`")
    L = ctypes.CDLL(path)
    L.bench_mfma_stream.restype = ctypes.c_int
    L.bench_mfma_stream.argtypes = [ctypes.c_int] * 4 + [ctypes.c_void_p, ctypes.POINTER(ctypes.c_double), ctypes.c_void_p]
    sink = torch.zeros(4, dtype=torch.float32, device=device)
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    out = {}
    for name, kind, peak in (("bf16", 0, PEAK_BF16_TFLOPS), ("mxfp4", 1, PEAK_FP4_TFLOPS), ("mxfp8", 2, PEAK_FP8_TFLOPS)):
        for label, rnd in (("constant", 0), ("random", 1)):
            flop = ctypes.c_double(0.0)
            def run(n):
                rc = L.bench_mfma_stream(kind, rnd, n, cus, _lib.ptr(sink), ctypes.byref(flop), _lib.stream_ptr(device))
                if rc != 0:
                    raise RuntimeError(f"bench_mfma_stream failed with {rc}")
            ms = time_events(lambda: run(2000), 2)
            iters = max(2000, int(2000 * seconds * 1e3 / max(ms, 1e-3)))
            ms = time_events(lambda: run(iters), 3)
            tf = flop.value / ms / 1e9
            out[f"{name}_{label}"] = {"TFLOP/s": round(tf, 1), "frac_peak": round(tf / peak, 4)}
    return out


def router_study(args, device):
    """What per-tile precision routing buys on a workload: for the fixed-precision modes and for the routed mode at a few
    thresholds, the attention kernel's time on the first ``--heads`` heads and the error of its float32 output against
    exact attention (float64 softmax(q k^T) v of the unquantized 16-bit inputs, computed with torch on the device) on
    sampled query tiles."""
    from ours.mxfp_attn_kernel import prepare_operands, attention_from_operands, route_tiles
    from ours.quant_mxint8 import pre_scale_q
    B, Hq, Hkv, N, D, tile, seed, desc = WORKLOADS[args.workload]
    causal = args.workload not in NON_CAUSAL
    q, k, v = make_inputs(B, Hq, Hkv, N, D, seed, device, 0 if causal else 21, args.workload not in PLAIN_DRAWS)
    group = Hq // Hkv
    hq = min(args.heads, Hq)
    hq -= hq % group if hq >= group else 0
    hq = max(hq, group)
    q, k, v = q[:, :hq].contiguous(), k[:, :hq // group].contiguous(), v[:, :hq // group].contiguous()
    nt = (N + tile - 1) // tile
    tiles = sorted({0, nt // 5, nt // 2, (4 * nt) // 5, nt - 1})
    rows = torch.cat([torch.arange(t * tile, min((t + 1) * tile, N)) for t in tiles]).to(device)
    pre = pre_scale_q(D)                                   # sm_scale * log2(e): scores in log2 units
    exact = torch.empty((B, hq, rows.numel(), D), dtype=torch.float64, device=device)
    for h in range(hq):
        sc = (q[0, h, rows].double() @ k[0, h // group].double().T) * pre
        if causal:
            sc = sc.masked_fill(torch.arange(N, device=device)[None, :] > rows[:, None], float("-inf"))
        pr = torch.exp2(sc - sc.amax(dim=1, keepdim=True))
        exact[0, h] = (pr / pr.sum(dim=1, keepdim=True)) @ v[0, h // group].double()
    out = torch.empty((B, hq, N, D), dtype=torch.float32, device=device)
    cases = [("mxfp4", None, None), ("diag", None, None), ("mxfp8", None, None)]
    cases += [("routed", t, None) for t in (0.99, 0.97, 0.95, 0.9, 0.8, 0.5)]
    cases += [("routed", 0.95, 0.5), ("routed", None, 0.5), ("routed", None, 0.8)]
    table = []
    for mode, hi, lo in cases:
        ops = prepare_operands(q, k, v, tile, mode)
        route = route_tiles(ops, causal, hi, lo) if mode == "routed" else None
        attention_from_operands(ops, out, causal, route=route)
        torch.cuda.synchronize()
        t_spin = time.perf_counter()                       # clocks up before the timed launches, the same for every case
        while (time.perf_counter() - t_spin) * 1e3 < args.spinup_ms:
            attention_from_operands(ops, out, causal, route=route)
            wait_for_device()
        ms = time_events(lambda: attention_from_operands(ops, out, causal, route=route), args.steps)
        got = out[:, :, rows].double()
        err = (got - exact).abs()
        row = {"mode": mode, "route_thresh": hi, "skip_thresh": lo, "kernel_ms": round(ms, 4),
               "cos": round(torch.nn.functional.cosine_similarity(got.flatten(), exact.flatten(), dim=0).item(), 7),
               "max_abs": float("%.4g" % err.max().item()), "rmse": float("%.4g" % err.pow(2).mean().sqrt().item()),
               "rel_l1": float("%.4g" % (err.sum() / exact.abs().sum()).item())}
        if route is not None:
            cls = route[0]
            visited = float((cls != 255).sum())
            row["tile_shares"] = {"mxfp8": round(float((cls == 2).sum()) / visited, 4), "mxfp4": round(float((cls == 1).sum()) / visited, 4),
                                  "skipped": round(float((cls == 0).sum()) / visited, 4)}
        table.append(row)
        del ops, route
    print(json.dumps({"kernel": "router study", "workload": desc, "heads": hq, "sampled_query_tiles": tiles,
                      "reference": "float64 softmax(q k^T * scale) v of the unquantized inputs (torch, on the device)", "cases": table}))


def skip_study(args, device):
    """What the reference's tile skipping costs and buys on a workload (first ``--heads`` heads): the attention time with
    the rule applied ahead of the attention kernel (mpsa_skip_route + mpsa_attn_fwd_routed) and inside it
    (mpsa_attn_fwd_skip), next to the kernel without skipping, over thresholds that skip from nothing to nearly everything."""
    from ours.mxfp_attn_kernel import prepare_operands, attention_from_operands, skip_route
    B, Hq, Hkv, N, D, tile, seed, desc = WORKLOADS[args.workload]
    causal = args.workload not in NON_CAUSAL
    q, k, v = make_inputs(B, Hq, Hkv, N, D, seed, device, 0 if causal else 21, args.workload not in PLAIN_DRAWS)
    if args.operands != "random":     # every element the same: what the statistics pass takes without the operands' bit toggling
        q, k, v = (torch.full_like(t, 1.0 if args.operands == "ones" else 0.0) for t in (q, k, v))
    group = Hq // Hkv
    hq = max(min(args.heads, Hq) // group * group, group)
    q, k, v = q[:, :hq].contiguous(), k[:, :hq // group].contiguous(), v[:, :hq // group].contiguous()
    nt = (N + tile - 1) // tile
    visited = (nt * (nt + 1) // 2 if causal else nt * nt) * B * hq
    out = torch.empty((B, hq, N, D), dtype=torch.bfloat16, device=device)
    table = []
    for mode in ("mxfp4", "diag", "mxfp8"):
        ops = prepare_operands(q, k, v, tile, mode)
        attention_from_operands(ops, out, causal)
        dense = time_events(lambda: attention_from_operands(ops, out, causal), args.steps)
        route_ms = time_events(lambda: skip_route(ops, causal, 1.0), args.steps)
        rows = []
        for th in (0.0, 0.5, 0.9, 1.0, 1.1, 2.0):
            skipped = torch.zeros((B, hq, nt), dtype=torch.int32, device=device)
            attention_from_operands(ops, out, causal, skip_thresh=th, skipped=skipped)
            share = float(skipped.sum()) / visited
            ahead = time_events(lambda: attention_from_operands(ops, out, causal, skip_thresh=th, skipped=skipped), args.steps)
            inside = time_events(lambda: attention_from_operands(ops, out, causal, skip_thresh=th, skipped=skipped, skip_in_kernel=True), args.steps)
            rows.append({"skip_thresh": th, "skipped_share": round(share, 4), "ahead_ms": round(ahead, 4), "inside_ms": round(inside, 4)})
        table.append({"mode": mode, "no_skipping_ms": round(dense, 4), "statistics_and_lists_ms": round(route_ms, 4), "thresholds": rows})
        del ops
    print(json.dumps({"kernel": "tile-skipping study", "workload": desc, "heads": hq, "cases": table}))


def run_only(args, device):
    """Launch one kernel repeatedly (for rocprofv3 --pmc / --kernel-trace runs)."""
    from ours import _lib
    from ours.mxfp_attn_kernel import prepare_operands, attention_from_operands, route_tiles
    from ours.quant_mxint8 import quantize_mx, quantize_mx_dual
    from ours.block_scaled_matmul import block_scaled_matmul, make_configs, pack_scale_5d
    if args.only == "router":
        router_study(args, device)
        return
    if args.only == "skip":
        skip_study(args, device)
        return
    if args.only == "mfma":
        print(json.dumps({"kernel": "matrix-instruction stream", "rates": mfma_stream_rates(device, 0.2)}))
        return
    if args.only == "copy":
        src = torch.ones(1 << 29, dtype=torch.bfloat16, device=device)          # 1 GiB
        dst = torch.empty_like(src)
        fn = lambda: dst.copy_(src)
        info = {"kernel": "torch copy", "bytes_read": src.numel() * 2, "bytes_written": src.numel() * 2}
    elif args.only == "attn":
        B, Hq, Hkv, N, D, tile, seed, desc = WORKLOADS[args.workload]
        causal = args.workload not in NON_CAUSAL
        q, k, v = make_inputs(B, Hq, Hkv, N, D, seed, device, 0 if causal else 21, args.workload not in PLAIN_DRAWS)
        if args.operands != "random":     # every element the same: the clock the kernel gets without the operands' bit toggling
            q, k, v = (torch.full_like(t, 1.0 if args.operands == "ones" else 0.0) for t in (q, k, v))
        out = torch.empty((B, Hq, N, D), dtype=torch.bfloat16, device=device)
        from ours.mxfp_attn_kernel import q_fusable
        fuse = args.mode != "routed" and not args.no_fuse_q and q_fusable(q, k, tile, args.mode, causal)
        ops = prepare_operands(q, k, v, tile, args.mode, fuse_q=fuse)
        route = route_tiles(ops, causal, args.route_thresh, args.skip_thresh) if args.mode == "routed" else None
        fn = lambda: attention_from_operands(ops, out, causal, route=route)
        info = {"kernel": "attention", "workload": desc, "mode": args.mode}
    elif args.only == "quant":
        B, Hq, Hkv, N, D, tile, seed, desc = WORKLOADS[args.workload]
        q, k, v = make_inputs(B, Hq, Hkv, N, D, seed, device)
        fn = lambda: quantize_mx_dual(q, 0.1275)
        info = {"kernel": "quantize dual (Q of the workload)", "elements": q.numel(), "algorithmic_bytes": q.numel() * 3.5625}
    else:
        M = N = K = 8192
        g = torch.Generator(device=device).manual_seed(1)
        if args.operands == "random":
            a = torch.randn(M, K, generator=g, device=device).to(torch.bfloat16)[None, None]
            b = torch.randn(N, K, generator=g, device=device).to(torch.bfloat16)[None, None]
        else:          # every code and scale byte the same: what the kernel does when power management leaves the clock alone
            a = torch.full((1, 1, M, K), 1.0 if args.operands == "ones" else 0.0, dtype=torch.bfloat16, device=device)
            b = a.clone()
        bst, fmt, fmt_b = {"gemm4": ("mxfp4", _lib.FMT_E2M1, _lib.FMT_E2M1), "gemm8": ("mxfp8", _lib.FMT_E4M3, _lib.FMT_E4M3),
                           "gemm48": ("mixed", _lib.FMT_E4M3, _lib.FMT_E2M1)}[args.only]
        ac, asc = quantize_mx(a, 1.0, fmt)
        bc, bsc = quantize_mx(b, 1.0, fmt_b)
        cfg = make_configs(bst)
        sa2, sb2 = (asc[0, 0], bsc[0, 0]) if args.linear_scales else (pack_scale_5d(asc[0, 0]), pack_scale_5d(bsc[0, 0]))
        fn = lambda: block_scaled_matmul(ac[0, 0], sa2, bc[0, 0], sb2, torch.bfloat16, M, N, K, cfg)
        info = {"kernel": "gemm " + bst, "flops": 2.0 * M * N * K, "scales": "row-major" if args.linear_scales else "packed",
                "operands": args.operands}
    fn()
    torch.cuda.synchronize()
    ms = time_events(fn, args.steps)
    info["ms"] = round(ms, 4)
    if "flops" in info:
        info["TFLOP/s"] = round(info["flops"] / ms / 1e9, 1)
    print(json.dumps(info))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default: 500; 100 for c5, 30 for c4)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps before them (default: a tenth of --steps)")
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS))
    ap.add_argument("--mode", default="diag", choices=["diag", "mxfp4", "mxfp8", "mixed", "routed"],
                    help="per-tile precision: diag (the headline configuration), one precision everywhere, or routed "
                         "(tile router on the scale bytes, thresholds below)")
    ap.add_argument("--route-thresh", type=float, default=ROUTE_THRESH_DEFAULT, help="routed: 8-bit at or above this share of the row's largest tile statistic")
    ap.add_argument("--skip-thresh", type=float, default=None, help="routed: skipped below this share")
    ap.add_argument("--spinup-ms", type=float, default=80.0, help="untimed device spin-up (steps run for this long) before the warm-up steps")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true")
    ap.add_argument("--no-fuse-q", action="store_true", help="with --only attn: hand the kernel quantized Q operands")
    ap.add_argument("--no-c4", action="store_true", help="leave the long-context figures out of `secondary`")
    ap.add_argument("--heads", type=int, default=4, help="--only router: query heads of the workload to run")
    ap.add_argument("--no-c5", action="store_true", help="leave the video-DiT figures out of `secondary`")
    ap.add_argument("--eager", action="store_true", help="time plain launches instead of replaying the step as a HIP graph")
    ap.add_argument("--operands", default="random", choices=["random", "ones", "zeros"],
                    help="--only gemm4|gemm8|attn|skip: the workload's random operands (default) or constant ones (the clock then stays up)")
    ap.add_argument("--linear-scales", action="store_true",
                    help="with --only gemm4/gemm8: row-major [rows, K/32] scales instead of the reference's packed form")
    ap.add_argument("--only", default=None, choices=["attn", "copy", "quant", "gemm4", "gemm8", "gemm48", "mfma", "router", "skip"],
                    help="profiling aid: launch just this kernel --steps times and exit (copy = 1 GiB torch copy, "
                         "the calibration kernel for HBM counters)")
    args = ap.parse_args()
    # A step is a fraction of a millisecond, while the host's wake-up at the closing synchronize and the GPU's clock
    # ramp after an idle moment cost about a millisecond once: few timed steps (or few warm-up steps) would measure
    # mostly that.  Measured on C3: 20 steps after 5 warm-up steps 0.453 ms/step, 500 after 50 0.376, 2000 0.373.
    if args.steps is None:
        args.steps = {"c4": 30, "c5": 100}.get(args.workload, 500)
    if args.warmup is None:
        args.warmup = max(3, args.steps // 10)
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the kernel is measured on one GPU's "
              "share at its real shape); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a HIP device", file=sys.stderr)
        sys.exit(1)

    from ours.mxfp_attn_kernel import prepare_operands, attention_from_operands, route_tiles, q_fusable

    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.only:
        run_only(args, device)
        return
    B, Hq, Hkv, N, D, tile, seed, desc = WORKLOADS[args.workload]
    causal = args.workload not in NON_CAUSAL
    q, k, v = make_inputs(B, Hq, Hkv, N, D, seed, device, 0 if causal else 21, args.workload not in PLAIN_DRAWS)
    out = torch.empty((B, Hq, N, D), dtype=torch.bfloat16, device=device)

    routed = args.mode == "routed"

    # The secondary figures run first: they are not part of the timed region, and a few hundred milliseconds of
    # matrix work before it bring the GPU's clocks up, which `--warmup` steps of a fraction of a millisecond do not.
    second = None
    if not args.no_secondary:
        second = secondary(device, quick=args.steps < 10)

    # shapes of the paired-tile kernel: Q stays unquantized and the attention kernel quantizes it in registers
    fuse_q = not routed and q_fusable(q, k, tile, args.mode, causal)
    state = {"ops": prepare_operands(q, k, v, tile, args.mode, fuse_q=fuse_q)}

    def step():
        ops = prepare_operands(q, k, v, tile, args.mode, reuse=state["ops"], fuse_q=fuse_q)
        route = route_tiles(ops, causal, args.route_thresh, args.skip_thresh) if routed else None
        attention_from_operands(ops, out, causal, route=route)

    # One step = two kernel launches on a stream.  A serving loop replays them as a HIP graph (the library neither
    # allocates nor synchronises, so the whole step captures); --eager times plain launches instead.
    launch = "eager"
    run_step = step
    if not args.eager and not routed:
        try:
            step()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                step()
            run_step, launch = graph.replay, "hip graph replay"
        except Exception as e:                                    # capture is an optimisation, not a requirement
            print(f"bench: graph capture failed ({e}); timing eager launches", file=sys.stderr)
            run_step, launch = step, "eager"

    # Device spin-up, untimed and before the warm-up steps: a GPU that has idled runs its first milliseconds at a low
    # clock, and `--warmup 5` steps of 0.4 ms do not bring it up (measured: 20 timed steps read 0.42 ms/step without
    # this and 0.37 with it, the same as 500 timed steps).
    t_spin = time.perf_counter()
    spin_steps = 0
    while (time.perf_counter() - t_spin) * 1e3 < args.spinup_ms:
        for _ in range(10):
            run_step()
        spin_steps += 10
        wait_for_device()
    for _ in range(args.warmup):
        run_step()
    wait_for_device()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run_step()
    wait_for_device()
    dt = time.perf_counter() - t0
    ms_per_step = dt * 1e3 / args.steps
    # the same steps as plain launches (no graph), for comparison with figures taken that way
    eager_ms = None
    if run_step is not step:
        for _ in range(args.warmup):
            step()
        wait_for_device()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        wait_for_device()
        eager_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    flops = (2.0 if causal else 4.0) * B * Hq * N * N * D
    tflops = flops / (ms_per_step * 1e-3) / 1e12

    # dominant kernel alone: the fused attention kernel on prepared operands
    ops = prepare_operands(q, k, v, tile, args.mode, fuse_q=fuse_q)
    route = route_tiles(ops, causal, args.route_thresh, args.skip_thresh) if routed else None
    attention_from_operands(ops, out, causal, route=route)
    torch.cuda.synchronize()
    k_iters = max(5, args.steps)
    attn_ms = time_events(lambda: attention_from_operands(ops, out, causal, route=route), k_iters)
    prep_ms = time_events(lambda: prepare_operands(q, k, v, tile, args.mode, reuse=ops, fuse_q=fuse_q), k_iters)
    achieved = flops / (attn_ms * 1e-3) / 1e12
    nt = (N + tile - 1) // tile
    comp = composite_peak_tflops(nt, causal)
    traffic, traffic_commit = measured_traffic(args.workload, args.mode)
    paired = D == 128 and tile == 128 and nt >= (2 if causal else 6) and args.mode in ("diag", "mxfp4", "mxfp8", "mixed")
    roofline = {
        "bound": "mfma", "kernel": ("attn_pp_kernel" if paired else "attn_fwd_kernel") + " (fused attention)", "achieved": round(achieved, 2), "peak": PEAK_FP4_TFLOPS,
        "unit": "TFLOP/s", "frac": round(achieved / PEAK_FP4_TFLOPS, 5),
        "traffic": traffic, "traffic_measured_at": traffic_commit,
        "kernel_ms": round(attn_ms, 4), "prepare_ms": round(prep_ms, 4),
        "composite_peak": round(comp, 1), "frac_composite": round(achieved / comp, 5),
        "flops_per_launch": flops,
    }
    if routed:
        cls = route[0]
        visited = float((cls != 255).sum())
        roofline["route_ms"] = round(time_events(lambda: route_tiles(ops, causal, args.route_thresh, args.skip_thresh), k_iters), 4)
        roofline["tile_shares"] = {"mxfp8": round(float((cls == 2).sum()) / visited, 4),
                                   "mxfp4": round(float((cls == 1).sum()) / visited, 4),
                                   "skipped": round(float((cls == 0).sum()) / visited, 4)}

    result = {
        "metric": "MXFP attn TFLOPS + % of scaled-MFMA peak, causal N=8K/128K D=128, 1 GPU",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "warmup_effective_steps": args.warmup + spin_steps,
        "ms_per_step": round(ms_per_step, 4), "ms_per_step_eager": None if eager_ms is None else round(eager_ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "mxfp4/mxfp8 scores (E2M1/E4M3 + E8M0), bf16 P.V, f32 accumulate", "data": "synthetic",
        "config": {"workload": desc, "B": B, "Hq": Hq, "Hkv": Hkv, "N": N, "D": D, "tile": tile, "mode": args.mode,
                   "step": ("quantize K (dual) + V repack + fused attention with Q quantized in the kernel" if fuse_q else
                            "quantize Q,K (dual) + V repack + " + ("tile router + " if routed else "") + "fused attention"),
                   "launch": launch, "spinup_ms": args.spinup_ms, "spinup_steps": spin_steps,
                   "inputs": "CPU draw (torch.Generator seed %d), bit-identical to the parity tests' tensors" % seed},
        "frac_mxfp4_peak": round(tflops / PEAK_FP4_TFLOPS, 5),
        "roofline": roofline,
    }
    if second is not None:
        result["secondary"] = second
        # what the matrix cores sustain on this chip (its clock is managed by power: operands with random bits run the
        # same instruction stream several hundred MHz lower than constants do), and the composite bound at those rates
        rates = mfma_stream_rates(device)
        second["mfma_stream"] = rates
        diag = 2.0 / (nt + 1) if causal else 1.0 / nt
        sustained = 1.0 / (0.5 * ((1 - diag) / rates["mxfp4_random"]["TFLOP/s"] + diag / rates["mxfp8_random"]["TFLOP/s"]) +
                           0.5 / rates["bf16_random"]["TFLOP/s"])
        roofline["sustained_composite"] = round(sustained, 1)
        roofline["frac_sustained_composite"] = round(achieved / sustained, 5)
        if args.workload == "c3" and args.mode == "diag" and not args.no_c4:
            del ops, route
            state.clear()
            result["secondary"]["c4"] = secondary_c4(device)
        if args.workload == "c3" and args.mode == "diag" and not args.no_c5:
            result["secondary"]["c5"] = secondary_c5(device)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(q, k, v, tile, D, causal)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
