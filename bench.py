"""Benchmark of the quantized-MoE hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-configs]

Default workload: MoE up-projection + fused SwiGLU at the prefill shape (T=4096 tokens, hidden 2880,
128 experts, top-4, MXFP4 weights [128, 2880, 5760], bf16 activations).  A step is one pass of the path over
one batch: routing(logits) then matmul_ogs(gather -> grouped GEMM -> bias + SwiGLU).  Inputs (logits,
activations, quantised weights) are resident in HBM before the timed region.  Prints ONE JSON line; with the
default workload the line also carries short runs of every other configuration of the path ("configs": dense
product, routing, decode, fp8 down projection + combine, quantise, dequantise), each with its kernel time,
achieved rate, roofline fraction and parity flags.
"""
import argparse
import gc
import hashlib
import json
import os
import re
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0
PEAK_BF16_TFLOPS = 2500.0
PEAK_FP8_TFLOPS = 5000.0
PEAK_MXFP4_TFLOPS = 10100.0

WORKLOADS = {
    # name: (T, E, k, K, N, swiglu)
    "fc1_prefill": dict(T=4096, E=128, k=4, K=2880, N=5760, act=True),
    "fc1_decode": dict(T=64, E=128, k=4, K=2880, N=5760, act=True),
    # same rows and FLOPs as fc1_prefill with few experts: weights (66 MB) stay cache resident
    "fc1_prefill_e8": dict(T=4096, E=8, k=4, K=2880, N=5760, act=True),
    # down projection + combine: fp8 (per-tensor scaled) expert-sorted rows x MXFP4 W2, gate weights, scatter, k-way sum
    "fc2_combine": dict(T=16384, E=32, k=4, K=2880, N=2880, act=False, fc2=True),
    # fc1_prefill with the activations quantised to MXFP8 inside the step (downcast_to_mxfp + scaled-MFMA matmul):
    # the block-scaled fp8 x fp4 path of the hardware; NOT interchangeable with the bf16 workload (x loses precision)
    "fc1_prefill_mx8": dict(T=4096, E=128, k=4, K=2880, N=5760, act=True, mx8=True),
    "fc1_prefill_mx4": dict(T=4096, E=128, k=4, K=2880, N=5760, act=True, mx4=True),
    # the down projection at decode size (fp8 rows of 64 tokens): weight streaming through the tiled fp8 kernel
    "fc2_decode": dict(T=64, E=128, k=4, K=2880, N=2880, act=False, fc2=True),
    # BASELINE config 1: one dense bf16 x MXFP4 product with bias (launch / latency bound: 7.6 MB, 4.3 GFLOP)
    "c1_dense": dict(M=256, K=2048, N=4096, dense=True),
    # BASELINE config 2: routing only (top-4 of 128 logits, softmax, histogram, gather / scatter indices, tables)
    "c2_routing": dict(T=4096, E=128, k=4, routing=True),
    # quantise / dequantise of weights in the matmul's layout: [8, 2880, 5760] float32 -> MXFP4 along K -> bfloat16
    "quant": dict(E=8, K=2880, N=5760, quant=True),
    "dequant": dict(E=8, K=2880, N=5760, dequant=True),
    # the whole MoE layer as the reference's bench/bench_mlp.py:60-96 runs it on one GPU, at the largest point of its
    # sweep (:256-279: d_model 5760, 128 experts, top-4, 64 rows per expert -> 2048 tokens, fp8 activations, MXFP4
    # weights): gate matmul -> top-k + softmax -> metadata -> FC1 + SwiGLU (gathered rows) -> FC2 (rows scattered back
    # to token order) -> sum over the k slots
    "mlp": dict(bpe=64, dim1=5760, dim2=5760, E=128, k=4, mlp=True),
    # every point of that sweep (bench_mlp.py:256: 1, 2, 4, ... 64 rows per expert), weights made once
    "mlp_sweep": dict(bpe=[1, 2, 4, 8, 16, 32, 64], dim1=5760, dim2=5760, E=128, k=4, mlp=True),
    # not a path workload: a plain elementwise copy of known size, the yardstick the HBM counters
    # (FETCH_SIZE / WRITE_SIZE) and the achievable copy bandwidth are calibrated with
    "hbm_copy": dict(bytes=1 << 30),
}
# the configurations BASELINE.json lists beside the headline one, and the pair that prepares / checks its weights
CONFIG_RUNS = (("c1_dense", "c1_dense"), ("c2_routing", "c2_routing"), ("c4_decode", "fc1_decode"),
               ("c5_fc2_combine", "fc2_combine"), ("quant", "quant"), ("dequant", "dequant"))


# ---------------------------------------------------------------------------------------------------------------------
# HBM traffic of the dominant kernels: measured with rocprofv3 counters outside this process and kept, with the digest
# of the kernel sources it was measured on, in profiles/hbm_traffic.txt
# ---------------------------------------------------------------------------------------------------------------------
def kernel_sources_digest():
    """sha256 over the kernel sources (csrc/*.h, *.hip, *.cpp and the C header), in name order."""
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "triton_amd", "csrc")
    files = sorted(os.path.join(csrc, f) for f in os.listdir(csrc) if f.endswith((".h", ".hip", ".cpp")))
    for path in files + [os.path.join(ROOT, "include", "triton_amd.h")]:
        h.update(os.path.basename(path).encode())
        h.update(open(path, "rb").read())
    return h.hexdigest()[:16]


def measured_traffic(workload):
    """(bytes per launch or None, where the number comes from).  None when the committed profile holds no line for
    the workload or was taken on other kernel sources than the ones in the tree."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic.txt")
    if not os.path.exists(path):
        return None, "profiles/hbm_traffic.txt is missing"
    text = open(path).read()
    m = re.search(r"kernel sources digest:\s*([0-9a-f]+)", text)
    digest = kernel_sources_digest()
    if not m or m.group(1) != digest:
        return None, (f"profiles/hbm_traffic.txt was measured on kernel sources {m.group(1) if m else '?'}, the tree "
                      f"holds {digest}: stale, not reported")
    for line in text.splitlines():
        lm = re.match(r"\S.*\((\w+)\)\s+([\d,]+)\s+([\d,]+)\s+([\d,]+)\s+([\d,]+)\s+([\d,]+)\s+([\d,]+)\s+[\d.]+\s*$", line)
        if lm and lm.group(1) == workload and "mm_" in line:
            return int(lm.group(6).replace(",", "")), ("profiles/hbm_traffic.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE "
                                                       f"scaled by a copy kernel, kernel sources {digest})")
    return None, "profiles/hbm_traffic.txt has no line for this workload"


SPIN_UP_MS = 0.0  # set for the short runs of the other configurations (see main)


def spin_up(fn):
    """Keeps the GPU busy with `fn` for SPIN_UP_MS before a short timed run: after a pause on the host (an oracle
    check of the previous configuration) the first milliseconds of GPU work run at idle clocks, which a run of a few
    milliseconds would otherwise be measured in."""
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < SPIN_UP_MS:
        for _ in range(4):
            fn()
        torch.cuda.synchronize()


def median(xs):
    xs = sorted(xs)
    n = len(xs)
    return xs[n // 2] if n % 2 else 0.5 * (xs[n // 2 - 1] + xs[n // 2])


class quiet_host:
    """Around a timed region: the collector runs once before it and not inside it.  A collection that frees large
    temporaries (the weights' float32 originals, layout conversions) inside the region returns their memory to the
    driver, which waits for the GPU -- tens of milliseconds charged to a few dozen steps."""

    def __enter__(self):
        gc.collect()
        gc.disable()
        torch.cuda.synchronize()

    def __exit__(self, *exc):
        gc.enable()


def timed(fn, steps, warmup):
    """Runs fn warmup + steps times for the wall time per call, then steps times again with a pair of HIP events around
    every call for the kernel time: for calls of a few tens of microseconds the event records themselves (host time and
    marker packets between the kernels) would otherwise be a third of the step they are meant to measure.  Returns
    (results of the last call, median HIP-event ms around a call, wall ms per call of the uninstrumented pass)."""
    out = None
    spin_up(fn)
    for _ in range(warmup):
        out = fn()
    with quiet_host():
        t0 = time.perf_counter()
        for _ in range(steps):
            out = fn()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e3 / steps
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for a, b in ev:
        a.record()
        out = fn()
        b.record()
    torch.cuda.synchronize()
    # back to back, the wall time per call bounds the time of the call's kernels from above: where the events (which add
    # a marker packet on either side) read more than that, the bound is the better figure
    return out, min(median([a.elapsed_time(b) for a, b in ev]), wall), wall


def graph_ms_per_call(fn, calls=16, replays=20):
    """Device time per call of a latency-bound `fn` (tens of microseconds: less than the host needs to launch it):
    `calls` consecutive calls are recorded into one HIP graph, the graph is replayed with a pair of HIP events around
    every replay, and the median is divided by `calls`.  The kernels then follow one another on the device without
    waiting for the host, so the figure is kernel time plus the device's own launch gaps."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    keep = []
    with torch.cuda.graph(graph):
        for _ in range(calls):
            keep.append(fn())
    for _ in range(3):
        graph.replay()
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(replays)]
    with quiet_host():
        for a, b in ev:
            a.record()
            graph.replay()
            b.record()
        torch.cuda.synchronize()
    return median([a.elapsed_time(b) for a, b in ev]) / calls


def base_line(args, metric, value, unit, ms_per_step, dtype, workload_text, **config):
    return {"metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": dtype, "data": "synthetic", "config": {"workload": workload_text, **config}}


def hbm_copy(args):
    """dst = src * 1 over `bytes` of float32: reads and writes that many bytes once each."""
    n = WORKLOADS["hbm_copy"]["bytes"] // 4
    src = torch.ones(n, dtype=torch.float32, device="cuda:0")
    dst = torch.empty_like(src)
    _, ms, wall = timed(lambda: torch.mul(src, 1.0, out=dst), args.steps, args.warmup)
    gbs = 2 * n * 4 / (ms * 1e-3) / 1e9
    out = base_line(args, "hbm_copy_gbs", round(gbs, 1), "GB/s", wall, "f32",
                    f"hbm_copy: torch.mul(src, 1.0, out=dst), {n * 4} bytes read + written")
    out["roofline"] = {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                       "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None, "kernel_ms": round(ms, 4)}
    out["cpu_baseline"] = None
    return out


def make_weights(E, K, N, device, seed=0):
    """W ~ N(0, 0.02) fp32 generated and quantised to MXFP4 along K one expert at a time."""
    from triton_amd.numerics_details.mxfp import downcast_to_mxfp
    from triton_amd.tensor import FP4, empty
    from triton_amd.tensor_details.dtype import UINT8
    from triton_amd.tensor_details.layout import StridedLayout
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    vals = empty((E, K, N), FP4, device, StridedLayout(-2)).storage.data
    scales = empty((E, K // 32, N), UINT8, device, StridedLayout(-2)).storage.data
    for e in range(E):
        w = torch.randn((1, K, N), generator=g, device=device, dtype=torch.float32) * 0.02
        v, s = downcast_to_mxfp(w, torch.uint8, axis=1)
        vals[e].copy_(v[0])
        scales[e].copy_(s[0])
    return vals, scales


def scales_for_matmul(scales, layout):
    """The weight scales in the encoding asked for on the command line."""
    if layout == "strided":
        return scales
    from triton_amd.tensor import convert_layout, wrap_torch_tensor
    from triton_amd.tensor_details.layout import CDNA4MXScaleLayout
    return convert_layout(wrap_torch_tensor(scales), CDNA4MXScaleLayout())


def weights_for_matmul(vals, layout):
    """The weight codes in the encoding asked for on the command line: as downcast_to_mxfp leaves them (K contiguous per
    column), or in the block layout of the gfx950 kernels (convert_layout(..., CDNA4MXValueLayout()))."""
    if layout == "strided":
        return vals
    from triton_amd.tensor import FP4, convert_layout, wrap_torch_tensor
    from triton_amd.tensor_details.layout import CDNA4MXValueLayout
    return convert_layout(wrap_torch_tensor(vals, dtype=FP4), CDNA4MXValueLayout())


def run_dense(args, cfg, name):
    """BASELINE config 1: y = x . deq(W) + bias, x bf16 [M, K], W fp32 [K, N] quantised to MXFP4 along K; the codes and
    scales of that quantisation are checked against the oracle bit for bit on the way."""
    from oracle import matmul_ref as MR
    from oracle.mxfp_ref import downcast_to_mxfp_ref
    from triton_amd.matmul import PrecisionConfig, matmul
    from triton_amd.numerics_details.mxfp import downcast_to_mxfp
    M, K, N = cfg["M"], cfg["K"], cfg["N"]
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    x_cpu = torch.randn(M, K).to(torch.bfloat16)
    bias_cpu = (torch.randn(N) * 0.01).to(torch.bfloat16)
    w_cpu = torch.randn(K, N) * 0.02
    vals, scales = downcast_to_mxfp(w_cpu.to(dev), torch.uint8, axis=0)
    rv, rs = downcast_to_mxfp_ref(w_cpu, torch.uint8, 0)
    codes_ok = bool(torch.equal(vals.cpu(), rv) and torch.equal(scales.cpu(), rs))
    x, bias = x_cpu.to(dev), bias_cpu.to(dev)
    pc = PrecisionConfig(b_mx_scale=scales_for_matmul(scales, args.scale_layout), b_microblock_size=32)
    wq = weights_for_matmul(vals, args.value_layout)
    from triton_amd.matmul_details.opt_flags import scoped_opt_flags_constraints
    with scoped_opt_flags_constraints({"block_m": args.block_m} if args.block_m else {}):
        y, kernel_ms, wall = timed(lambda: matmul(x, wq, bias, precision_config=pc), args.steps, args.warmup)
        event_ms = kernel_ms
        kernel_ms = min(kernel_ms, graph_ms_per_call(lambda: matmul(x, wq, bias, precision_config=pc)))
    flops = 2.0 * M * K * N
    alg_bytes = M * K * 2 + K // 2 * N + K // 32 * N + N * 2 + M * N * 2
    torch.set_num_threads(os.cpu_count())
    t0 = time.perf_counter()
    ref = MR.matmul_ref(x_cpu, vals.cpu(), bias_cpu, b_mx_scale=scales.cpu())
    cpu_s = time.perf_counter() - t0
    ok = bool(torch.allclose(y.cpu().float(), ref.float(), rtol=1e-2, atol=1e-2))
    gbs = alg_bytes / (kernel_ms * 1e-3) / 1e9
    out = base_line(args, "moe_matmul_ogs_tflops", round(flops / (wall * 1e-3) / 1e12, 2), "TFLOP/s", wall,
                    "bf16 x mxfp4 (fp32 accumulate)",
                    f"{name}: dense matmul + bias, M={M}, K={K}, N={N}, W mxfp4 [{K},{N}]", scale_layout=args.scale_layout,
                    value_layout=args.value_layout)
    out["matmul_kernel_tflops"] = round(flops / (kernel_ms * 1e-3) / 1e12, 2)
    out["roofline"] = {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                       "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None,
                       # 161-256 rows: 32-row tiles shared by four K groups; fewer rows or a forced block of 16: streaming kernel
                       "kernel": "mm_x16_mxfp4_kgroups_kernel" if 160 < M <= 256 and args.block_m in (0, None, 32)
                       else ("mm_stream16_kernel" if args.block_m in (0, None, 16) else "mm_x16_mxfp4_kernel"),
                       "kernel_ms": round(kernel_ms, 4), "algorithmic_bytes": alg_bytes, "algorithmic_flops": flops,
                       "event_pair_ms": round(event_ms, 4),
                       "note": "kernel_ms: 16 calls replayed as one HIP graph, per call (event pairs around single calls "
                               "include the host's launch time: event_pair_ms); the problem is latency bound "
                               "(4.3 GFLOP, 7.6 MB)"}
    out["cpu_baseline"] = {"value": round(flops / cpu_s / 1e12, 4), "unit": "TFLOP/s", "cores": os.cpu_count(),
                           "kind": "port", "sample": f"oracle matmul_ref on the whole problem, {cpu_s:.2f} s"}
    out["parity"] = {"gemm_within_1e-2": ok, "mxfp4_codes_and_scales_bit_exact": codes_ok}
    return out


def run_routing(args, cfg, name):
    """BASELINE config 2: routing(logits) alone.  Bit-exact integers against the oracle; launch-latency bound."""
    from oracle import routing_ref as RR
    from triton_amd.routing import routing
    T, E, k = cfg["T"], cfg["E"], cfg["k"]
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    logits_cpu = torch.randn(T, E)
    logits = logits_cpu.to(dev)
    r, kernel_ms, wall = timed(lambda: routing(logits, k), args.steps, args.warmup)
    event_ms = kernel_ms
    kernel_ms = min(kernel_ms, graph_ms_per_call(lambda: routing(logits, k)))
    t0 = time.perf_counter()
    ref = RR.routing_ref(logits_cpu, k)
    cpu_s = time.perf_counter() - t0
    rm, rr = r.ragged_metadata, ref["ragged"]
    ok = bool(torch.equal(r.indx.cpu().int(), ref["indx"]) and torch.equal(r.col_sum.cpu(), ref["col_sum"])
              and torch.equal(r.gather_indx.cpu(), ref["gather_indx"]) and torch.equal(r.scatter_indx.cpu(), ref["scatter_indx"])
              and torch.equal(r.row_sorted_indx.cpu(), ref["row_sorted_indx"]) and torch.equal(rm.slice_offs.cpu(), rr.slice_offs)
              and torch.equal(rm.block_offs_data.cpu(), rr.block_offs_data)
              and torch.equal(rm.block_schedule_data.cpu(), rr.block_schedule_data))
    vals_ok = bool(torch.allclose(r.vals.cpu(), ref["vals"], rtol=1e-5, atol=1e-7))
    # logits in; indices, values, bit matrix, histogram, three index arrays and the tables out
    alg_bytes = T * E * 4 + T * k * (2 + 4) + T * ((E + 31) // 32) * 4 + E * 4 + 3 * T * k * 4 + 6 * (E + 1) * 4
    gbs = alg_bytes / (kernel_ms * 1e-3) / 1e9
    out = base_line(args, "moe_routing_tokens_per_s", round(T / (wall * 1e-3), 1), "tokens/s", wall, "f32 logits -> int32",
                    f"{name}: routing (top-{k} of {E} + softmax, histogram, gather / scatter indices, ragged tables), T={T}")
    out["roofline"] = {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                       "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None, "kernel": "topk_hist_kernel + order_scan_kernel",
                       "kernel_ms": round(kernel_ms, 4), "algorithmic_bytes": alg_bytes,
                       "event_pair_ms": round(event_ms, 4),
                       "note": "2.4 MB in two launches: bound by launch latency, not by HBM; kernel_ms: 16 calls replayed as "
                               "one HIP graph, per call"}
    out["cpu_baseline"] = {"value": round(T / cpu_s, 1), "unit": "tokens/s", "cores": 1, "kind": "port",
                           "sample": f"oracle routing_ref (numpy) on the whole batch, {cpu_s:.3f} s"}
    out["parity"] = {"routing_bit_exact": ok, "softmax_values_within_1e-5": vals_ok}
    return out


def run_quant(args, cfg, name):
    """Weights [E, K, N] float32 -> MXFP4 along K (the layout the matmul consumes), and back to bfloat16.  HBM bound:
    achieved = (source bytes + codes + scales) / kernel time."""
    from oracle.mxfp_ref import downcast_to_mxfp_ref, upcast_from_mxfp_ref
    from triton_amd.numerics_details.mxfp import downcast_to_mxfp, upcast_from_mxfp
    E, K, N = cfg["E"], cfg["K"], cfg["N"]
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev)
    g.manual_seed(0)
    w = torch.randn((E, K, N), generator=g, device=dev, dtype=torch.float32) * 0.02
    n = E * K * N
    sample = w[:1, :, :256].cpu()  # the oracle checks one expert's first 256 columns (bit-exact)
    if cfg.get("quant"):
        (v, s), kernel_ms, wall = timed(lambda: downcast_to_mxfp(w, torch.uint8, axis=1), args.steps, args.warmup)
        alg_bytes = n * 4 + n // 2 + n // 32
        t0 = time.perf_counter()
        rv, rs = downcast_to_mxfp_ref(sample, torch.uint8, 1)
        cpu_s = time.perf_counter() - t0
        ok = bool(torch.equal(v[:1, :, :256].cpu(), rv) and torch.equal(s[:1, :, :256].cpu(), rs))
        what, kern, dtype = "downcast_to_mxfp: float32 -> e2m1 codes + e8m0 scales", "downcast_cols_tile_kernel", "f32 -> mxfp4"
        parity = {"codes_and_scales_bit_exact": ok}
    else:
        v, s = downcast_to_mxfp(w, torch.uint8, axis=1)
        y, kernel_ms, wall = timed(lambda: upcast_from_mxfp(v, s, torch.bfloat16, axis=1), args.steps, args.warmup)
        alg_bytes = n // 2 + n // 32 + n * 2
        vs, ss = v[:1, :, :256].cpu(), s[:1, :, :256].cpu()
        t0 = time.perf_counter()
        ref = upcast_from_mxfp_ref(vs, ss, torch.bfloat16, 1)
        cpu_s = time.perf_counter() - t0
        ok = bool(torch.equal(y[:1, :, :256].cpu().view(torch.int16), ref.view(torch.int16)))
        what, kern, dtype = "upcast_from_mxfp: e2m1 codes + e8m0 scales -> bfloat16", "upcast_cols_tile_kernel", "mxfp4 -> bf16"
        parity = {"values_bit_exact": ok}
    gbs = alg_bytes / (kernel_ms * 1e-3) / 1e9
    out = base_line(args, "mxfp_gbs", round(alg_bytes / (wall * 1e-3) / 1e9, 1), "GB/s", wall, dtype,
                    f"{name}: {what}, weights [{E},{K},{N}] quantised along K")
    out["roofline"] = {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                       "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None, "kernel": kern,
                       "kernel_ms": round(kernel_ms, 4), "algorithmic_bytes": alg_bytes}
    out["cpu_baseline"] = {"value": round(sample.numel() * (alg_bytes / n) / cpu_s / 1e9, 3), "unit": "GB/s", "cores": 1,
                           "kind": "port", "sample": f"oracle (numpy) on one expert's first 256 columns, {cpu_s:.2f} s"}
    out["parity"] = parity
    return out


def algorithmic_bytes(col_sum, T, k, K, N, act, x_row_bytes=None):
    """x rows read + y rows written + (codes + scales + bias) of the experts that have rows.  `x_row_bytes`: one
    activation row as stored (bf16 unless given: MXFP8 K + K/32, MXFP4 K/2 + K/32)."""
    rows = T * k
    n_active = int((col_sum > 0).sum())
    n_out = N // 2 if act else N
    per_expert = K // 2 * N + K // 32 * N + N * 2
    return rows * (x_row_bytes or K * 2) + rows * n_out * 2 + n_active * per_expert, n_active


def cpu_baseline(x_cpu, vals, scales, bias_cpu, ref, experts, K, N, act, fc2=None):
    """Oracle (CPU restatement of the reference's torch path) timed on a bounded sample: the first
    `experts` experts of the same workload, all host cores.  For the down projection `fc2` holds
    (x_scale, gammas) and the rows are already expert-sorted."""
    from oracle import matmul_ref as MR
    torch.set_num_threads(os.cpu_count())
    sizes = ref["col_sum"][:experts]
    n_rows = int(sizes.sum())
    v = vals[:experts].cpu()
    s = scales[:experts].cpu()
    t0 = time.perf_counter()
    if fc2 is None:
        gather = ref["gather_indx"][:n_rows]
        y = MR.matmul_ref(x_cpu, v, bias_cpu[:experts], slice_sizes=sizes, gather_indx=gather, b_mx_scale=s,
                          fused_swiglu=(1.702, 7.0) if act else None)
    else:
        x_scale, gammas = fc2
        y = MR.matmul_ref(x_cpu[:n_rows], v, bias_cpu[:experts], slice_sizes=sizes, b_mx_scale=s, a_flex_scale=x_scale,
                          gammas=gammas[:n_rows]).to(torch.bfloat16)
    dt = time.perf_counter() - t0
    flops = 2.0 * n_rows * K * N
    return y, n_rows, flops / dt / 1e12, dt


def sample_experts(args, rows, E, K, N):
    """Experts in the CPU sample: as asked, or about 0.6 TFLOP of oracle work (10-15 s on the box's host cores)."""
    if args.cpu_experts > 0:
        return min(args.cpu_experts, E)
    return max(1, min(E, int(6e11 * args.cpu_work / (2.0 * rows / E * K * N))))


def run_fc2(args, cfg, name):
    """BASELINE config 5: y = scatter((x8 . deq(W2[e]) * sx + bias[e]) * gate), z = sum over the k slots."""
    from oracle import matmul_ref as MR
    from oracle import routing_ref as RR
    from triton_amd.matmul import FlexCtx, InFlexData, PrecisionConfig, matmul
    from triton_amd.matmul_details.opt_flags import scoped_opt_flags_constraints
    from triton_amd.reduce import reduce
    from triton_amd.routing import routing
    T, E, k, K, N = cfg["T"], cfg["E"], cfg["k"], cfg["K"], cfg["N"]
    rows = T * k
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    logits_cpu = torch.randn(T, E)
    bias_cpu = (torch.randn(E, N) * 0.01).to(torch.bfloat16)
    g = torch.Generator(device=dev)
    g.manual_seed(1)
    x0 = torch.randn((rows, K), generator=g, device=dev, dtype=torch.float32)
    x_scale = (x0.abs().max() / 448.0).reshape(1)
    x8 = (x0 / x_scale).to(torch.float8_e4m3fn)
    del x0
    logits, bias = logits_cpu.to(dev), bias_cpu.to(dev)
    vals, scales = make_weights(E, K, N, dev)
    pc = PrecisionConfig(b_mx_scale=scales_for_matmul(scales, args.scale_layout), b_microblock_size=32,
                         out_dtype=torch.bfloat16,
                         flex_ctx=FlexCtx(lhs_data=InFlexData(dtype=torch.float8_e4m3fn, scale=x_scale)))
    y_buf = torch.empty((rows, N), dtype=torch.bfloat16, device=dev)
    constraints = {"block_m": args.block_m} if args.block_m else {}
    wq = weights_for_matmul(vals, args.value_layout)

    def step(ev=None):
        r = routing(logits, k)
        gam = r.expert_sorted_gate_weights
        if ev is not None:
            ev[0].record()
        y = matmul(x8, wq, bias, r.ragged_metadata, scatter_indx=r.scatter_indx, precision_config=pc, gammas=gam, c=y_buf)
        if ev is not None:
            ev[1].record()
            ev[2].record()
        z, _ = reduce(y.view(T, k, N), dim=1)
        if ev is not None:
            ev[3].record()
        return r, gam, y, z

    with scoped_opt_flags_constraints(constraints):
        spin_up(step)
        for _ in range(args.warmup):
            r, gam, y, z = step()
        torch.cuda.synchronize()
        events = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(args.steps)]
        with quiet_host():
            t0 = time.perf_counter()
            for i in range(args.steps):
                r, gam, y, z = step(events[i])
            torch.cuda.synchronize()
            wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    kernel_ms = median([e[0].elapsed_time(e[1]) for e in events])
    combine_ms = median([e[2].elapsed_time(e[3]) for e in events])
    flops = 2.0 * rows * K * N
    col_sum = r.col_sum.cpu()
    n_active = int((col_sum > 0).sum())
    mm_bytes = rows * K + n_active * (K // 2 * N + K // 32 * N + N * 2) + rows * 8 + rows * N * 2
    tflops_kernel = flops / (kernel_ms * 1e-3) / 1e12
    gbs_kernel = mm_bytes / (kernel_ms * 1e-3) / 1e9
    traffic, traffic_source = measured_traffic(name)
    if rows <= 16 * E:  # decode size: weight streaming, bound by HBM
        roof = dict(bound="hbm", achieved=round(gbs_kernel, 1), peak=PEAK_HBM_GBS, unit="GB/s",
                    frac=round(gbs_kernel / PEAK_HBM_GBS, 4), traffic=traffic, traffic_source=traffic_source,
                    kernel="mm_stream16_kernel", kernel_ms=round(kernel_ms, 4), algorithmic_bytes=mm_bytes,
                    algorithmic_flops=flops)
    else:
        roof = dict(bound="mfma", achieved=round(tflops_kernel, 1), peak=PEAK_FP8_TFLOPS, unit="TFLOP/s",
                    frac=round(tflops_kernel / PEAK_FP8_TFLOPS, 4), traffic=traffic, traffic_source=traffic_source,
                    kernel="mm_x8_mxfp4_kernel", kernel_ms=round(kernel_ms, 4), algorithmic_bytes=mm_bytes,
                    algorithmic_flops=flops, frac_of_mxfp4_peak=round(tflops_kernel / PEAK_MXFP4_TFLOPS, 4),
                    hbm_gbs=round(gbs_kernel, 1))
    combine_bytes = rows * N * 2 + T * N * 2
    # the least a fused matmul + combine would move (rows, weights, gate weights and scatter indices in, the combined
    # tokens out); what ran is the reference's two-kernel form, whose intermediate rows are written and read once more
    fused_min = rows * K + n_active * (K // 2 * N + K // 32 * N + N * 2) + rows * 8 + T * N * 2
    roof["form"] = "two kernels: matmul_ogs writes bf16 [rows, N] (scattered), reduce sums the k slots"
    roof["algorithmic_bytes_fused_minimum"] = fused_min
    roof["algorithmic_bytes_two_kernel_form"] = mm_bytes + combine_bytes
    if traffic is not None:
        roof["traffic_over_fused_minimum"] = round(traffic / fused_min, 3)
    roof["combine"] = dict(kernel="reduce_kernel", kernel_ms=round(combine_ms, 4), bound="hbm", algorithmic_bytes=combine_bytes,
                           achieved=round(combine_bytes / (combine_ms * 1e-3) / 1e9, 1), unit="GB/s",
                           frac=round(combine_bytes / (combine_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4))
    ref = RR.routing_ref(logits_cpu, k)
    routing_ok = bool(torch.equal(r.scatter_indx.cpu(), ref["scatter_indx"]) and torch.equal(col_sum, ref["col_sum"]))
    gam_ref = ref["vals"].flatten()[ref["col_sorted_indx"].long()]
    routing_ok = routing_ok and bool(torch.allclose(gam.cpu(), gam_ref, rtol=1e-5, atol=1e-7))  # softmax values
    gam_ref = gam.cpu()
    # the combine is a fixed-order fp32 sum: bit-exact given y
    n_chk = min(2048, T)
    combine_ok = bool(torch.equal(z[:n_chk].cpu(), MR.reduce_ref(y.view(T, k, N)[:n_chk].cpu(), 1)))
    cpu, gemm_ok = None, None
    if args.cpu_experts != 0:
        n_e = sample_experts(args, rows, E, K, N)
        y_ref, n_rows, cpu_tflops, cpu_s = cpu_baseline(x8.cpu(), vals, scales, bias_cpu, ref, n_e, K, N, False,
                                                        fc2=(x_scale.cpu(), gam_ref))
        got = y.cpu()[ref["scatter_indx"][:n_rows].long()]
        gemm_ok = bool(torch.allclose(got.float(), y_ref.float(), rtol=1e-2, atol=1e-2))
        cpu = dict(value=round(cpu_tflops, 5), unit="TFLOP/s", cores=os.cpu_count(), kind="port",
                   sample=f"oracle matmul_ref (dequantise + fp32 GEMM, gate weights) on the first {n_e} of {E} experts "
                          f"({n_rows} of {rows} rows), {cpu_s:.1f} s")
    out = base_line(args, "moe_matmul_ogs_tflops", round(flops / (ms_per_step * 1e-3) / 1e12, 2), "TFLOP/s", ms_per_step,
                    "fp8e4m3 x mxfp4 (fp32 accumulate)",
                    f"{name}: routing + matmul_ogs(fp8 rows, grouped GEMM, bias, gate weights, scatter) + "
                    f"top-{k} combine, T={T}, hidden={K}, experts={E}, W2 mxfp4 [{E},{K},{N}]",
                    rows=rows, active_experts=n_active, scale_layout=args.scale_layout, value_layout=args.value_layout)
    out.update({"tokens_per_s": round(T / (ms_per_step * 1e-3), 1), "matmul_kernel_tflops": round(tflops_kernel, 2),
                "roofline": roof, "cpu_baseline": cpu,
                "parity": {"routing_bit_exact": routing_ok, "combine_bit_exact": combine_ok,
                           "gemm_sample_within_1e-2": gemm_ok}})
    return out


def run_fc1(args, cfg, name):
    """BASELINE configs 3 / 4: routing + matmul_ogs(gather, grouped GEMM, bias + SwiGLU)."""
    from oracle import routing_ref as RR
    from triton_amd.matmul import FnSpecs, FusedActivation, PrecisionConfig, matmul
    from triton_amd.matmul_details.opt_flags import scoped_opt_flags_constraints
    from triton_amd.routing import routing
    from triton_amd.swiglu import swiglu_fn

    T, E, k, K, N, act = cfg["T"], cfg["E"], cfg["k"], cfg["K"], cfg["N"], cfg["act"]
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    logits_cpu = torch.randn(T, E)
    x_cpu = torch.randn(T, K).to(torch.bfloat16)
    bias_cpu = (torch.randn(E, N) * 0.01).to(torch.bfloat16)
    logits, x, bias = logits_cpu.to(dev), x_cpu.to(dev), bias_cpu.to(dev)
    vals, scales = make_weights(E, K, N, dev)
    pc = PrecisionConfig(b_mx_scale=scales_for_matmul(scales, args.scale_layout), b_microblock_size=32)
    fa = FusedActivation(FnSpecs("swiglu", swiglu_fn, ("alpha", "limit"), reduction_n=2), (1.702, 7.0)) if act else None
    constraints = {"block_m": args.block_m} if args.block_m else {}
    wq = weights_for_matmul(vals, args.value_layout)

    mx4 = bool(cfg.get("mx4"))   # MXFP4 activations: packed e2m1 codes, widened (exactly) to fp8 inside matmul
    mx8 = bool(cfg.get("mx8")) or mx4
    x_store = torch.uint8 if mx4 else torch.float8_e4m3fn
    if mx8:
        from triton_amd.numerics_details.mxfp import downcast_to_mxfp

    def step(ev=None):
        r = routing(logits, k)
        if mx8:
            xq, xs = downcast_to_mxfp(x, x_store, axis=-1)
            pcs = PrecisionConfig(a_mx_scale=xs, a_microblock_size=32, b_mx_scale=pc.b_mx_scale, b_microblock_size=32)
        if ev is not None:
            ev[0].record()
        if mx8:
            y = matmul(xq, wq, bias, r.ragged_metadata, gather_indx=r.gather_indx, precision_config=pcs, fused_activation=fa)
        else:
            y = matmul(x, wq, bias, r.ragged_metadata, gather_indx=r.gather_indx, precision_config=pc, fused_activation=fa)
        if ev is not None:
            ev[1].record()
        return r, y

    with scoped_opt_flags_constraints(constraints):
        spin_up(step)
        for _ in range(args.warmup):
            r, y = step()
        torch.cuda.synchronize()
        events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
        with quiet_host():
            t0 = time.perf_counter()
            for i in range(args.steps):
                r, y = step(events[i])
            torch.cuda.synchronize()
            wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    kernel_ms = median([a.elapsed_time(b) for a, b in events])

    col_sum = r.col_sum.cpu()
    rows = T * k
    flops = 2.0 * rows * K * N
    x_row_bytes = (K // 2 if mx4 else K) + K // 32 if mx8 else None
    abytes, n_active = algorithmic_bytes(col_sum, T, k, K, N, act, x_row_bytes)
    tflops_step = flops / (ms_per_step * 1e-3) / 1e12
    tflops_kernel = flops / (kernel_ms * 1e-3) / 1e12
    gbs_kernel = abytes / (kernel_ms * 1e-3) / 1e9
    # the operands' own peak decides which roofline binds (MXFP4 x MXFP4: 10.1 PFLOP/s, so the bytes bind); the
    # kernel multiplies widened fp8 values either way
    peak_mfma = PEAK_MXFP4_TFLOPS if mx4 else PEAK_FP8_TFLOPS if mx8 else PEAK_BF16_TFLOPS
    hbm_bound = (abytes / (PEAK_HBM_GBS * 1e9)) > (flops / (peak_mfma * 1e12))
    traffic, traffic_source = measured_traffic(name)
    if hbm_bound:
        roof = dict(bound="hbm", achieved=round(gbs_kernel, 1), peak=PEAK_HBM_GBS, unit="GB/s",
                    frac=round(gbs_kernel / PEAK_HBM_GBS, 4), traffic=traffic, traffic_source=traffic_source)
    else:
        roof = dict(bound="mfma", achieved=round(tflops_kernel, 1), peak=peak_mfma, unit="TFLOP/s",
                    frac=round(tflops_kernel / peak_mfma, 4), traffic=traffic, traffic_source=traffic_source)
    # row blocks of 16 (few rows per expert) run the weight-streaming kernel, everything else the tiled one
    roof["kernel"] = "mm_stream16_kernel" if rows <= 16 * E else ("mm_x8_mxfp4_kernel" if mx8 else "mm_x16_mxfp4_kernel")
    if mx4:
        roof["kernel"] = "widen_e2m1_rows_kernel + " + roof["kernel"]
        roof["frac_of_fp8_mfma_peak"] = round(tflops_kernel / PEAK_FP8_TFLOPS, 4)
    roof["kernel_ms"] = round(kernel_ms, 4)
    roof["algorithmic_bytes"] = abytes
    roof["algorithmic_flops"] = flops
    roof["frac_of_mxfp4_peak"] = round(tflops_kernel / PEAK_MXFP4_TFLOPS, 4)
    roof["hbm_gbs"] = round(gbs_kernel, 1)
    if rows > 16 * E:
        # the tiled kernel computes whole 32-row MFMA fragments: rows of the ragged experts rounded up to 32 are what
        # the matrix cores actually run (the share that is padding is the price of the ragged row counts)
        issued_rows = int(((col_sum + 31) // 32 * 32).sum())
        roof["mfma_rows_issued"] = issued_rows
        roof["mfma_issue_tflops"] = round(2.0 * issued_rows * K * N / (kernel_ms * 1e-3) / 1e12, 1)

    # parity of this very run against the oracle, and the CPU baseline, on a bounded sample
    ref = RR.routing_ref(logits_cpu, k)
    routing_ok = bool(torch.equal(r.scatter_indx.cpu(), ref["scatter_indx"]) and torch.equal(col_sum, ref["col_sum"])
                      and torch.equal(r.gather_indx.cpu(), ref["gather_indx"]))
    cpu = None
    gemm_ok = None
    if args.cpu_experts != 0:
        n_e = sample_experts(args, rows, E, K, N)
        x_ref = x_cpu
        if mx8:  # the oracle sees the same quantised activations, dequantised (exactly) to bf16
            from oracle.mxfp_ref import downcast_to_mxfp_ref, upcast_from_mxfp_ref
            qv, qs = downcast_to_mxfp_ref(x_cpu, x_store, axis=-1)
            x_ref = upcast_from_mxfp_ref(qv, qs, torch.bfloat16, axis=-1)
        y_ref, n_rows, cpu_tflops, cpu_s = cpu_baseline(x_ref, vals, scales, bias_cpu, ref, n_e, K, N, act)
        gemm_ok = bool(torch.allclose(y[:n_rows].cpu().float(), y_ref.float(), rtol=1e-2, atol=1e-2))
        cpu = dict(value=round(cpu_tflops, 5), unit="TFLOP/s", cores=os.cpu_count(), kind="port",
                   sample=f"oracle matmul_ref (dequantise + fp32 GEMM + SwiGLU) on the first {n_e} of {E} experts "
                          f"({n_rows} of {rows} rows), {cpu_s:.1f} s")
    out = base_line(args, "moe_matmul_ogs_tflops", round(tflops_step, 2), "TFLOP/s", ms_per_step,
                    ("mxfp4 x mxfp4 (multiplied as fp8)" if mx4 else "mxfp8 x mxfp4" if mx8 else "bf16 x mxfp4") +
                    " (fp32 accumulate)",
                    f"{name}: routing + " + ("downcast_to_mxfp(x) + " if mx8 else "") +
                    f"matmul_ogs(gather, grouped GEMM, bias+SwiGLU), T={T}, hidden={K}, experts={E}, top-{k}, "
                    f"W1 mxfp4 [{E},{K},{N}]", rows=rows, active_experts=n_active, scale_layout=args.scale_layout,
                    value_layout=args.value_layout)
    out.update({"tokens_per_s": round(T / (ms_per_step * 1e-3), 1), "matmul_kernel_tflops": round(tflops_kernel, 2),
                "roofline": roof, "cpu_baseline": cpu,
                "parity": {"routing_bit_exact": routing_ok, "gemm_sample_within_1e-2": gemm_ok}})
    return out


def run_mlp(args, cfg, name):
    """bench/bench_mlp.py:60-96 of the reference with one rank: every stage is timed with HIP events, and checked
    against the oracle given the GPU's own output of the stage before (logits -> routing, bit-exact; FC1 and FC2 on a
    sample of experts, within the fp8 output step; the combine, bit-exact).  `cfg["bpe"]` may be one number of rows
    per expert or the list of the reference's sweep (bench_mlp.py:256: 1 ... 64); the weights are made once, the
    line describes the last (largest) point and carries every point under "sweep"."""
    from oracle import matmul_ref as MR
    from oracle import routing_ref as RR
    from triton_amd.matmul import FnSpecs, FusedActivation, PrecisionConfig, matmul
    from triton_amd.reduce import reduce
    from triton_amd.routing import routing
    from triton_amd.swiglu import swiglu_fn
    from triton_amd.numerics_details.mxfp import downcast_to_mxfp
    E, k, d1, d2 = cfg["E"], cfg["k"], cfg["dim1"], cfg["dim2"]
    bpes = [args.bpe] if args.bpe else (cfg["bpe"] if isinstance(cfg["bpe"], (list, tuple)) else [cfg["bpe"]])
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev)
    g.manual_seed(0)
    rnd = lambda *shape: torch.randn(shape, generator=g, device=dev, dtype=torch.float32)
    wg = rnd(d1, E).to(torch.bfloat16).t().contiguous().t()  # [d1, E] with unit stride along K, as quantize_weight leaves it
    bg, b1, b2 = rnd(E), rnd(E, d2), rnd(E, d1)

    def quantise(K, N):
        from triton_amd.tensor import FP4, empty
        from triton_amd.tensor_details.dtype import UINT8
        from triton_amd.tensor_details.layout import StridedLayout
        vals = empty((E, K, N), FP4, dev, StridedLayout(-2)).storage.data
        scales = empty((E, K // 32, N), UINT8, dev, StridedLayout(-2)).storage.data
        for e in range(E):
            v, sc = downcast_to_mxfp(rnd(1, K, N).to(torch.bfloat16), torch.uint8, axis=1)
            vals[e].copy_(v[0])
            scales[e].copy_(sc[0])
        return vals, scales
    w1, s1 = quantise(d1, d2)
    w2, s2 = quantise(d2 // 2, d1)
    w1q, w2q = weights_for_matmul(w1, args.value_layout), weights_for_matmul(w2, args.value_layout)
    pc1 = PrecisionConfig(b_mx_scale=scales_for_matmul(s1, args.scale_layout), b_microblock_size=32)
    pc2 = PrecisionConfig(b_mx_scale=scales_for_matmul(s2, args.scale_layout), b_microblock_size=32)
    act1 = FusedActivation(FnSpecs("swiglu", swiglu_fn, ("alpha", "limit"), reduction_n=2), (1.0, 1.0))
    names = ("gate_matmul", "routing", "fc1_swiglu", "fc2_scatter", "combine")
    from triton_amd.matmul_details.opt_flags import scoped_opt_flags_constraints
    constraints = {"block_m": args.block_m} if args.block_m else {}

    def point(bpe):
        T = bpe * E // k
        x8 = rnd(T, d1).to(torch.float8_e4m3fn)
        x16 = x8.to(torch.bfloat16)

        def step(ev=None):
            mark = (lambda i: ev[i].record()) if ev is not None else (lambda i: None)
            mark(0)
            logits = matmul(x16, wg, bg)
            mark(1)
            r = routing(logits, k)
            mark(2)
            with scoped_opt_flags_constraints(constraints):
                y1 = matmul(x8, w1q, b1, r.ragged_metadata, gather_indx=r.gather_indx, precision_config=pc1, fused_activation=act1)
                mark(3)
                y2 = matmul(y1, w2q, b2, r.ragged_metadata, scatter_indx=r.scatter_indx, precision_config=pc2)
            mark(4)
            z, _ = reduce(y2.view(T, k, d1), dim=1)
            mark(5)
            return logits, r, y1, y2, z

        spin_up(step)
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        events = [[torch.cuda.Event(enable_timing=True) for _ in range(6)] for _ in range(args.steps)]
        with quiet_host():
            t0 = time.perf_counter()
            for i in range(args.steps):
                logits, r, y1, y2, z = step(events[i])
            torch.cuda.synchronize()
            ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
        stage_ms = {n: median([e[i].elapsed_time(e[i + 1]) for e in events]) for i, n in enumerate(names)}
        rows = T * k
        flops = {"gate_matmul": 2.0 * T * d1 * E, "fc1_swiglu": 2.0 * rows * d1 * d2, "fc2_scatter": 2.0 * rows * (d2 // 2) * d1}
        n_active = int((r.col_sum > 0).sum())
        w_bytes = lambda K, N: n_active * (K // 2 * N + K // 32 * N + N * 4)
        bytes_ = {"gate_matmul": T * d1 * 2 + d1 * E * 2 + T * E * 2, "fc1_swiglu": rows * d1 + w_bytes(d1, d2) + rows * d2 // 2,
                  "fc2_scatter": rows * d2 // 2 + w_bytes(d2 // 2, d1) + rows * d1, "combine": rows * d1 + T * d1}
        stages = {}
        for n in names:
            st = {"ms": round(stage_ms[n], 4)}
            if n in flops:
                st["tflops"] = round(flops[n] / (stage_ms[n] * 1e-3) / 1e12, 1)
            if n in bytes_:
                st["algorithmic_gbs"] = round(bytes_[n] / (stage_ms[n] * 1e-3) / 1e9, 1)
                st["frac_of_hbm"] = round(bytes_[n] / (stage_ms[n] * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)
            stages[n] = st
        # ---- parity, stage by stage, each against the oracle fed with the GPU's output of the stage before
        logits_ref = MR.matmul_ref(x16.cpu(), wg.cpu(), bg.cpu())
        logits_ok = bool(torch.allclose(logits.cpu().float(), logits_ref.float(), rtol=2e-2, atol=2e-1))
        ref = RR.routing_ref(logits.cpu(), k)
        routing_ok = bool(torch.equal(r.scatter_indx.cpu(), ref["scatter_indx"]) and torch.equal(r.col_sum.cpu(), ref["col_sum"])
                          and torch.equal(r.gather_indx.cpu(), ref["gather_indx"]))
        n_e = 2 if args.cpu_experts <= 0 else min(args.cpu_experts, E)
        busy = torch.nonzero(ref["col_sum"] > 0).flatten()[:n_e].tolist()  # experts with rows (few tokens leave some empty)
        offs = torch.cat([torch.zeros(1, dtype=torch.int64), ref["col_sum"].long().cumsum(0)])
        fc1_ok = fc2_ok = True
        nan_frac, n_rows, cpu_s = 0.0, 0, 0.0
        for e in busy:
            lo, hi = int(offs[e]), int(offs[e + 1])
            sizes = ref["col_sum"][e:e + 1]
            t0 = time.perf_counter()
            y1_ref = MR.matmul_ref(x8.cpu(), w1[e:e + 1].cpu(), b1[e:e + 1].cpu(), slice_sizes=sizes,
                                   gather_indx=ref["gather_indx"][lo:hi], b_mx_scale=s1[e:e + 1].cpu(), fused_swiglu=(1.0, 1.0))
            y2_ref = MR.matmul_ref(y1[lo:hi].cpu(), w2[e:e + 1].cpu(), b2[e:e + 1].cpu(), slice_sizes=sizes,
                                   b_mx_scale=s2[e:e + 1].cpu())
            cpu_s += time.perf_counter() - t0
            n_rows += hi - lo
            # fp8 outputs: one step of the type (2^-3 relative) where an fp32 sum lands on a rounding boundary
            fc1_ok = fc1_ok and bool(torch.allclose(y1[lo:hi].cpu().float(), y1_ref.float(), rtol=0.13, atol=2e-2))
            got2 = y2.cpu()[ref["scatter_indx"][lo:hi].long()].float()
            # NaN marks an overflowed float8_e4m3fn output: the pattern of NaNs must agree, everything else within one step
            ref2 = y2_ref.float()
            nan_frac += float(torch.isnan(ref2).float().sum())
            fc2_ok = fc2_ok and bool(torch.equal(torch.isnan(got2), torch.isnan(ref2)) and
                                     torch.allclose(torch.nan_to_num(got2, nan=0.0), torch.nan_to_num(ref2, nan=0.0), rtol=0.13, atol=2e-2))
        nan_frac /= max(1, n_rows * d1)
        n_chk = min(256, T)
        z_ref, _, _ = MR.reduce_general_ref(y2.view(T, k, d1)[:n_chk].cpu(), 1)
        a, b = z[:n_chk].cpu().float(), z_ref.float()
        combine_ok = bool(torch.equal(torch.isnan(a), torch.isnan(b)) and torch.equal(torch.nan_to_num(a), torch.nan_to_num(b)))
        mm_ms = stage_ms["fc1_swiglu"] + stage_ms["fc2_scatter"]
        mm_flops = flops["fc1_swiglu"] + flops["fc2_scatter"]
        mm_bytes = bytes_["fc1_swiglu"] + bytes_["fc2_scatter"]
        return dict(bpe=bpe, tokens=T, rows=rows, active_experts=n_active, ms_per_step=round(ms_per_step, 4), stages=stages,
                    mm_ms=mm_ms, mm_flops=mm_flops, mm_bytes=mm_bytes,
                    cpu=dict(flops=2.0 * n_rows * d1 * d2 + 2.0 * n_rows * (d2 // 2) * d1, seconds=cpu_s, experts=len(busy), rows=n_rows),
                    parity={"gate_logits_within_2e-2": logits_ok, "routing_bit_exact": routing_ok,
                            "fc1_sample_within_fp8_step": fc1_ok, "fc2_sample_within_fp8_step": fc2_ok,
                            "fc2_sample_overflowed_fraction": round(nan_frac, 5), "combine_bit_exact": combine_ok})

    pts = [point(b) for b in bpes]
    last = pts[-1]
    T = last["tokens"]
    # few rows per expert: both products stream the weights of the active experts once -- bound by HBM; at 64 rows per
    # expert the matrix cores' share is about a third of that time
    gbs = last["mm_bytes"] / (last["mm_ms"] * 1e-3) / 1e9
    tflops = last["mm_flops"] / (last["mm_ms"] * 1e-3) / 1e12
    out = base_line(args, "moe_mlp_tokens_per_s", round(T / (last["ms_per_step"] * 1e-3), 1), "tokens/s", last["ms_per_step"],
                    "fp8e4m3 x mxfp4 (fp32 accumulate), bf16 gate",
                    f"{name}: gate matmul + routing + FC1/SwiGLU + FC2 + combine, tokens={T} ({last['bpe']} rows per expert), "
                    f"d_model={d1}, experts={E}, top-{k}, W1 mxfp4 [{E},{d1},{d2}], W2 mxfp4 [{E},{d2 // 2},{d1}]",
                    scale_layout=args.scale_layout, value_layout=args.value_layout)
    out["stages"] = last["stages"]
    out["roofline"] = {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                       "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None, "kernel": "mm_x8_mxfp4_kernel (FC1 + FC2)",
                       "kernel_ms": round(last["mm_ms"], 4), "algorithmic_flops": last["mm_flops"],
                       "algorithmic_bytes": last["mm_bytes"], "tflops": round(tflops, 1),
                       "frac_of_fp8_mfma_peak": round(tflops / PEAK_FP8_TFLOPS, 4)}
    c = last["cpu"]
    out["cpu_baseline"] = {"value": round(c["flops"] / max(c["seconds"], 1e-9) / 1e12, 5), "unit": "TFLOP/s",
                           "cores": os.cpu_count(), "kind": "port",
                           "sample": f"oracle FC1 + FC2 on {c['experts']} of {E} experts ({c['rows']} of {last['rows']} rows), {c['seconds']:.1f} s"}
    out["parity"] = last["parity"]
    if len(pts) > 1:
        out["sweep"] = [{"bpe": p["bpe"], "tokens": p["tokens"], "active_experts": p["active_experts"], "ms_per_step": p["ms_per_step"],
                         "stages": p["stages"], "parity_all_true": all(v is True for k_, v in p["parity"].items() if isinstance(v, bool))}
                        for p in pts]
    return out


def run_workload(args, name):
    cfg = WORKLOADS[name]
    if name == "hbm_copy":
        return hbm_copy(args)
    if cfg.get("dense"):
        return run_dense(args, cfg, name)
    if cfg.get("routing"):
        return run_routing(args, cfg, name)
    if cfg.get("quant") or cfg.get("dequant"):
        return run_quant(args, cfg, name)
    if cfg.get("fc2"):
        return run_fc2(args, cfg, name)
    if cfg.get("mlp"):
        return run_mlp(args, cfg, name)
    return run_fc1(args, cfg, name)


def config_summary(line):
    """What the headline line carries of another configuration's run."""
    r = line["roofline"]
    s = {"workload": line["config"]["workload"], "ms_per_step": line["ms_per_step"], "kernel": r.get("kernel"),
         "kernel_ms": r["kernel_ms"], "bound": r["bound"], "achieved": r["achieved"], "unit": r["unit"], "peak": r["peak"],
         "frac": r["frac"], "parity": line.get("parity")}
    for key in ("combine", "note", "traffic"):
        if r.get(key) is not None:
            s[key] = r[key]
    if line.get("tokens_per_s") is not None:
        s["tokens_per_s"] = line["tokens_per_s"]
    return s


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="fc1_prefill", choices=sorted(WORKLOADS))
    ap.add_argument("--cpu-experts", type=int, default=-1,
                    help="experts in the CPU baseline sample (0 = skip; default: about 0.6 TFLOP of oracle work, 10-15 s)")
    ap.add_argument("--no-configs", action="store_true",
                    help="default workload only: leave out the short runs of the other configurations")
    ap.add_argument("--block-m", type=int, default=0)
    ap.add_argument("--bpe", type=int, default=0, help="--workload mlp: rows per expert (tokens = bpe * experts / top-k)")
    ap.add_argument("--scale-layout", default=None, choices=["strided", "cdna4"],
                    help="encoding of the weight scales handed to matmul: [E, K/32, N] bytes contiguous along K, or the "
                    "CDNA4 pre-shuffle (convert_layout(..., CDNA4MXScaleLayout())).  Default: cdna4, what the reference "
                    "picks on this target (make_default_matmul_mxfp4_w_scale_layout, tensor_details/layout.py:43-54)")
    ap.add_argument("--value-layout", default="blocks", choices=["strided", "blocks"],
                    help="encoding of the MXFP4 weight codes handed to matmul: K contiguous per column, as "
                    "downcast_to_mxfp leaves them and the reference's AMD path keeps them (tensor_details/layout.py:27-40), or "
                    "the block layout of the gfx950 kernels (convert_layout(..., CDNA4MXValueLayout()); default)")
    args = ap.parse_args()
    if args.scale_layout is None:
        args.scale_layout = "cdna4"
    args.cpu_work = 1.0
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; --gpus > 1 is not supported (with more GPUs the experts "
              "would be sharded across them, one exchange of rows before and after the two matmuls)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the kernels have no CPU path", file=sys.stderr)
        sys.exit(3)

    out = run_workload(args, args.workload)
    if args.workload == "fc1_prefill" and not args.no_configs:
        # the other configurations: fewer steps, and a tenth of the oracle work in their parity samples
        sub = argparse.Namespace(**vars(args))
        sub.steps, sub.warmup, sub.cpu_work = min(args.steps, 10), min(args.warmup, 3), 0.1
        global SPIN_UP_MS
        SPIN_UP_MS = 100.0
        configs = {}
        for key, name in CONFIG_RUNS:
            t0 = time.perf_counter()
            configs[key] = config_summary(run_workload(sub, name))
            configs[key]["bench_seconds"] = round(time.perf_counter() - t0, 1)
            torch.cuda.empty_cache()
        out["configs"] = configs
    print(json.dumps(out))


if __name__ == "__main__":
    main()
