"""Benchmark of the quantized-MoE hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload fc1_prefill|fc1_decode|dense|routing]

Default workload: MoE up-projection + fused SwiGLU at the prefill shape (T=4096 tokens, hidden 2880,
128 experts, top-4, MXFP4 weights [128, 2880, 5760], bf16 activations).  A step is one pass of the path over
one batch: routing(logits) then matmul_ogs(gather -> grouped GEMM -> bias + SwiGLU).  Inputs (logits,
activations, quantised weights) are resident in HBM before the timed region.  Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0
PEAK_BF16_TFLOPS = 2500.0
PEAK_FP8_TFLOPS = 5000.0
PEAK_MXFP4_TFLOPS = 10100.0

# HBM bytes per launch of the dominant kernel (FETCH_SIZE x 2.00 + WRITE_SIZE x 1.00 KiB from rocprofv3 --pmc,
# factors from the hbm_copy workload).  Counters cannot be read from inside this process; re-measure after kernel changes.
MEASURED_TRAFFIC = {"fc1_prefill": 1611457371, "fc1_decode": 976176743, "fc2_combine": 1497319402}

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
    # the down projection at decode size (fp8 rows of 64 tokens): weight streaming through the tiled fp8 kernel
    "fc2_decode": dict(T=64, E=128, k=4, K=2880, N=2880, act=False, fc2=True),
    # BASELINE config 1: one dense bf16 x MXFP4 product with bias (launch / latency bound: 7.6 MB, 4.3 GFLOP)
    "c1_dense": dict(M=256, K=2048, N=4096, dense=True),
    # not a path workload: a plain elementwise copy of known size, the yardstick the HBM counters
    # (FETCH_SIZE / WRITE_SIZE) and the achievable copy bandwidth are calibrated with
    "hbm_copy": dict(bytes=1 << 30),
}


def hbm_copy(args):
    """dst = src * 1 over `bytes` of float32: reads and writes that many bytes once each."""
    n = WORKLOADS["hbm_copy"]["bytes"] // 4
    src = torch.ones(n, dtype=torch.float32, device="cuda:0")
    dst = torch.empty_like(src)
    for _ in range(args.warmup):
        torch.mul(src, 1.0, out=dst)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for a, b in ev:
        a.record()
        torch.mul(src, 1.0, out=dst)
        b.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms = sum(a.elapsed_time(b) for a, b in ev) / args.steps
    gbs = 2 * n * 4 / (ms * 1e-3) / 1e9
    print(json.dumps({"metric": "hbm_copy_gbs", "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
                      "warmup": args.warmup, "ms_per_step": round(wall * 1e3 / args.steps, 4), "higher_is_better": True,
                      "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
                      "config": {"workload": f"hbm_copy: torch.mul(src, 1.0, out=dst), {n * 4} bytes read + written"},
                      "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                   "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None, "kernel_ms": round(ms, 4)},
                      "cpu_baseline": None}))


def run_dense(args, cfg):
    """BASELINE config 1: y = x . deq(W) + bias, x bf16 [M, K], W MXFP4 [K, N] quantised along K."""
    from oracle import matmul_ref as MR
    from triton_amd.matmul import PrecisionConfig, matmul
    M, K, N = cfg["M"], cfg["K"], cfg["N"]
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    x_cpu = torch.randn(M, K).to(torch.bfloat16)
    bias_cpu = (torch.randn(N) * 0.01).to(torch.bfloat16)
    vals, scales = make_weights(1, K, N, dev)
    vals, scales = vals[0], scales[0]
    x, bias = x_cpu.to(dev), bias_cpu.to(dev)
    pc = PrecisionConfig(b_mx_scale=scales_for_matmul(scales, args.scale_layout), b_microblock_size=32)
    for _ in range(args.warmup):
        y = matmul(x, vals, bias, precision_config=pc)
    torch.cuda.synchronize()
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for a, b in events:
        a.record()
        y = matmul(x, vals, bias, precision_config=pc)
        b.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    kernel_ms = sum(a.elapsed_time(b) for a, b in events) / args.steps
    ms_per_step = wall * 1e3 / args.steps
    flops = 2.0 * M * K * N
    alg_bytes = M * K * 2 + K // 2 * N + K // 32 * N + N * 2 + M * N * 2
    torch.set_num_threads(os.cpu_count())
    t0 = time.perf_counter()
    ref = MR.matmul_ref(x_cpu, vals.cpu(), bias_cpu, b_mx_scale=scales.cpu())
    cpu_s = time.perf_counter() - t0
    ok = bool(torch.allclose(y.cpu().float(), ref.float(), rtol=1e-2, atol=1e-2))
    gbs = alg_bytes / (kernel_ms * 1e-3) / 1e9
    print(json.dumps({
        "metric": "moe_matmul_ogs_tflops", "value": round(flops / (ms_per_step * 1e-3) / 1e12, 2), "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16 x mxfp4 (fp32 accumulate)",
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: dense matmul + bias, M={M}, K={K}, N={N}, W mxfp4 [{K},{N}]",
                   "scale_layout": args.scale_layout},
        "matmul_kernel_tflops": round(flops / (kernel_ms * 1e-3) / 1e12, 2),
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None, "kernel": "mm_stream16_kernel",
                     "kernel_ms": round(kernel_ms, 4), "algorithmic_bytes": alg_bytes, "algorithmic_flops": flops,
                     "note": "event pairs around one launch include launch latency; the problem is latency bound"},
        "cpu_baseline": {"value": round(flops / cpu_s / 1e12, 4), "unit": "TFLOP/s", "cores": os.cpu_count(), "kind": "port",
                         "sample": f"oracle matmul_ref on the whole problem, {cpu_s:.2f} s"},
        "parity": {"gemm_within_1e-2": ok}}))


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


def algorithmic_bytes(col_sum, T, k, K, N, act):
    """x rows read + y rows written + (codes + scales + bias) of the experts that have rows."""
    rows = T * k
    n_active = int((col_sum > 0).sum())
    n_out = N // 2 if act else N
    per_expert = K // 2 * N + K // 32 * N + N * 2
    return rows * K * 2 + rows * n_out * 2 + n_active * per_expert, n_active


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


def run_fc2(args, cfg):
    """BASELINE config 5: y = scatter((x8 . deq(W2[e]) * sx + bias[e]) * gate), z = sum over the k slots."""
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

    def step(ev=None):
        r = routing(logits, k)
        gam = r.expert_sorted_gate_weights
        if ev is not None:
            ev[0].record()
        y = matmul(x8, vals, bias, r.ragged_metadata, scatter_indx=r.scatter_indx, precision_config=pc, gammas=gam, c=y_buf)
        if ev is not None:
            ev[1].record()
        z, _ = reduce(y.view(T, k, N), dim=1)
        return r, gam, y, z

    with scoped_opt_flags_constraints(constraints):
        for _ in range(args.warmup):
            r, gam, y, z = step()
        torch.cuda.synchronize()
        events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            r, gam, y, z = step(events[i])
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    kernel_ms = sum(a.elapsed_time(b) for a, b in events) / args.steps
    flops = 2.0 * rows * K * N
    col_sum = r.col_sum.cpu()
    n_active = int((col_sum > 0).sum())
    mm_bytes = rows * K + n_active * (K // 2 * N + K // 32 * N + N * 2) + rows * 8 + rows * N * 2
    tflops_kernel = flops / (kernel_ms * 1e-3) / 1e12
    gbs_kernel = mm_bytes / (kernel_ms * 1e-3) / 1e9
    if rows <= 16 * E:  # decode size: weight streaming, bound by HBM
        roof = dict(bound="hbm", achieved=round(gbs_kernel, 1), peak=PEAK_HBM_GBS, unit="GB/s",
                    frac=round(gbs_kernel / PEAK_HBM_GBS, 4), traffic=MEASURED_TRAFFIC.get(args.workload),
                    kernel="mm_stream16_kernel", kernel_ms=round(kernel_ms, 4), algorithmic_bytes=mm_bytes,
                    algorithmic_flops=flops)
    else:
        roof = dict(bound="mfma", achieved=round(tflops_kernel, 1), peak=PEAK_FP8_TFLOPS, unit="TFLOP/s",
                    frac=round(tflops_kernel / PEAK_FP8_TFLOPS, 4), traffic=MEASURED_TRAFFIC.get(args.workload),
                    kernel="mm_x8_mxfp4_kernel", kernel_ms=round(kernel_ms, 4), algorithmic_bytes=mm_bytes,
                    algorithmic_flops=flops, frac_of_mxfp4_peak=round(tflops_kernel / PEAK_MXFP4_TFLOPS, 4),
                    hbm_gbs=round(gbs_kernel, 1))
    ref = RR.routing_ref(logits_cpu, k)
    routing_ok = bool(torch.equal(r.scatter_indx.cpu(), ref["scatter_indx"]) and torch.equal(col_sum, ref["col_sum"]))
    gam_ref = ref["vals"].flatten()[ref["col_sorted_indx"].long()]
    routing_ok = routing_ok and bool(torch.allclose(gam.cpu(), gam_ref, rtol=1e-5, atol=1e-7))  # softmax values
    gam_ref = gam.cpu()
    # the combine is a fixed-order fp32 sum: bit-exact given y
    from oracle import matmul_ref as MR
    n_chk = 2048
    combine_ok = bool(torch.equal(z[:n_chk].cpu(), MR.reduce_ref(y.view(T, k, N)[:n_chk].cpu(), 1)))
    cpu, gemm_ok = None, None
    if args.cpu_experts != 0:
        n_e = min(args.cpu_experts, E) if args.cpu_experts > 0 else max(1, min(E, int(6e11 / (2.0 * rows / E * K * N))))
        y_ref, n_rows, cpu_tflops, cpu_s = cpu_baseline(x8.cpu(), vals, scales, bias_cpu, ref, n_e, K, N, False,
                                                        fc2=(x_scale.cpu(), gam_ref))
        got = y.cpu()[ref["scatter_indx"][:n_rows].long()]
        gemm_ok = bool(torch.allclose(got.float(), y_ref.float(), rtol=1e-2, atol=1e-2))
        cpu = dict(value=round(cpu_tflops, 5), unit="TFLOP/s", cores=os.cpu_count(), kind="port",
                   sample=f"oracle matmul_ref (dequantise + fp32 GEMM, gate weights) on the first {n_e} of {E} experts "
                          f"({n_rows} of {rows} rows), {cpu_s:.1f} s")
    print(json.dumps({
        "metric": "moe_matmul_ogs_tflops", "value": round(flops / (ms_per_step * 1e-3) / 1e12, 2), "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "fp8e4m3 x mxfp4 (fp32 accumulate)",
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: routing + matmul_ogs(fp8 rows, grouped GEMM, bias, gate weights, scatter) + "
                               f"top-{k} combine, T={T}, hidden={K}, experts={E}, W2 mxfp4 [{E},{K},{N}]",
                   "rows": rows, "active_experts": n_active, "scale_layout": args.scale_layout},
        "tokens_per_s": round(T / (ms_per_step * 1e-3), 1), "matmul_kernel_tflops": round(tflops_kernel, 2),
        "roofline": roof, "cpu_baseline": cpu,
        "parity": {"routing_bit_exact": routing_ok, "combine_bit_exact": combine_ok, "gemm_sample_within_1e-2": gemm_ok},
    }))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="fc1_prefill", choices=sorted(WORKLOADS))
    ap.add_argument("--cpu-experts", type=int, default=-1,
                    help="experts in the CPU baseline sample (0 = skip; default: about 0.6 TFLOP of oracle work, 10-15 s)")
    ap.add_argument("--block-m", type=int, default=0)
    ap.add_argument("--scale-layout", default="strided", choices=["strided", "cdna4"],
                    help="encoding of the weight scales handed to matmul: [E, K/32, N] bytes contiguous along K, or the "
                    "CDNA4 pre-shuffle (convert_layout(..., CDNA4MXScaleLayout()))")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; --gpus > 1 is not supported (with more GPUs the experts "
              "would be sharded across them, one exchange of rows before and after the two matmuls)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the kernels have no CPU path", file=sys.stderr)
        sys.exit(3)

    if args.workload == "hbm_copy":
        hbm_copy(args)
        return

    if WORKLOADS[args.workload].get("dense"):
        run_dense(args, WORKLOADS[args.workload])
        return

    if WORKLOADS[args.workload].get("fc2"):
        run_fc2(args, WORKLOADS[args.workload])
        return

    from oracle import routing_ref as RR
    from triton_amd.matmul import FnSpecs, FusedActivation, PrecisionConfig, matmul
    from triton_amd.matmul_details.opt_flags import scoped_opt_flags_constraints
    from triton_amd.routing import routing
    from triton_amd.swiglu import swiglu_fn

    cfg = WORKLOADS[args.workload]
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

    mx8 = bool(cfg.get("mx8"))
    if mx8:
        from triton_amd.numerics_details.mxfp import downcast_to_mxfp

    def step(ev=None):
        r = routing(logits, k)
        if mx8:
            xq, xs = downcast_to_mxfp(x, torch.float8_e4m3fn, axis=-1)
            pcs = PrecisionConfig(a_mx_scale=xs, a_microblock_size=32, b_mx_scale=pc.b_mx_scale, b_microblock_size=32)
        if ev is not None:
            ev[0].record()
        if mx8:
            y = matmul(xq, vals, bias, r.ragged_metadata, gather_indx=r.gather_indx, precision_config=pcs, fused_activation=fa)
        else:
            y = matmul(x, vals, bias, r.ragged_metadata, gather_indx=r.gather_indx, precision_config=pc, fused_activation=fa)
        if ev is not None:
            ev[1].record()
        return r, y

    with scoped_opt_flags_constraints(constraints):
        for _ in range(args.warmup):
            r, y = step()
        torch.cuda.synchronize()
        events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        start.record()
        for i in range(args.steps):
            r, y = step(events[i])
        stop.record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    kernel_ms = sum(a.elapsed_time(b) for a, b in events) / args.steps

    col_sum = r.col_sum.cpu()
    rows = T * k
    flops = 2.0 * rows * K * N
    abytes, n_active = algorithmic_bytes(col_sum, T, k, K, N, act)
    tflops_step = flops / (ms_per_step * 1e-3) / 1e12
    tflops_kernel = flops / (kernel_ms * 1e-3) / 1e12
    gbs_kernel = abytes / (kernel_ms * 1e-3) / 1e9
    peak_mfma = PEAK_FP8_TFLOPS if mx8 else PEAK_BF16_TFLOPS
    hbm_bound = (abytes / (PEAK_HBM_GBS * 1e9)) > (flops / (peak_mfma * 1e12))
    if hbm_bound:
        roof = dict(bound="hbm", achieved=round(gbs_kernel, 1), peak=PEAK_HBM_GBS, unit="GB/s",
                    frac=round(gbs_kernel / PEAK_HBM_GBS, 4), traffic=MEASURED_TRAFFIC.get(args.workload))
    else:
        roof = dict(bound="mfma", achieved=round(tflops_kernel, 1), peak=peak_mfma, unit="TFLOP/s",
                    frac=round(tflops_kernel / peak_mfma, 4), traffic=MEASURED_TRAFFIC.get(args.workload))
    # row blocks of 16 (few rows per expert) run the weight-streaming kernel, everything else the tiled one
    roof["kernel"] = "mm_stream16_kernel" if rows <= 16 * E else ("mm_x8_mxfp4_kernel" if mx8 else "mm_x16_mxfp4_kernel")
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
        n_e = min(args.cpu_experts, E) if args.cpu_experts > 0 else max(1, min(E, int(6e11 / (2.0 * rows / E * K * N))))
        x_ref = x_cpu
        if mx8:  # the oracle sees the same quantised activations, dequantised (exactly) to bf16
            from oracle.mxfp_ref import downcast_to_mxfp_ref, upcast_from_mxfp_ref
            qv, qs = downcast_to_mxfp_ref(x_cpu, torch.float8_e4m3fn, axis=-1)
            x_ref = upcast_from_mxfp_ref(qv, qs, torch.bfloat16, axis=-1)
        y_ref, n_rows, cpu_tflops, cpu_s = cpu_baseline(x_ref, vals, scales, bias_cpu, ref, n_e, K, N, act)
        gemm_ok = bool(torch.allclose(y[:n_rows].cpu().float(), y_ref.float(), rtol=1e-2, atol=1e-2))
        cpu = dict(value=round(cpu_tflops, 5), unit="TFLOP/s", cores=os.cpu_count(), kind="port",
                   sample=f"oracle matmul_ref (dequantise + fp32 GEMM + SwiGLU) on the first {n_e} of {E} experts "
                          f"({n_rows} of {rows} rows), {cpu_s:.1f} s")
    out = {
        "metric": "moe_matmul_ogs_tflops", "value": round(tflops_step, 2), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": ("mxfp8 x mxfp4" if mx8 else "bf16 x mxfp4") + " (fp32 accumulate)", "data": "synthetic",
        "config": {"workload": f"{args.workload}: routing + " + ("downcast_to_mxfp(x) + " if mx8 else "") +
                               f"matmul_ogs(gather, grouped GEMM, bias+SwiGLU), T={T}, "
                               f"hidden={K}, experts={E}, top-{k}, W1 mxfp4 [{E},{K},{N}]",
                   "rows": rows, "active_experts": n_active, "scale_layout": args.scale_layout},
        "tokens_per_s": round(T / (ms_per_step * 1e-3), 1),
        "matmul_kernel_tflops": round(tflops_kernel, 2),
        "roofline": roof,
        "cpu_baseline": cpu,
        "parity": {"routing_bit_exact": routing_ok, "gemm_sample_within_1e-2": gemm_ok},
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
