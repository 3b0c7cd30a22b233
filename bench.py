"""Headline benchmark: INT4 g128 weight-only-quantized linear on one MI355X.

A step is one woq_linear call (through the C ABI) over one synthetic batch.  The default
workload is the decode shape the metric is quoted on -- activations bf16 [1, 4096], weights
uint4 [14336, 4096], group 128, lowp_mode BF16 -- with the weight rotated over enough distinct
copies (> 512 MB in total) that no launch finds its weights in the 256 MB Infinity Cache.
The same JSON line carries the prefill figure (M = 2048, TFLOP/s), the roofline fraction of
the dominant kernel and a CPU baseline (the oracle's C port on the host cores).

    python bench.py --gpus 1 --steps 2000 --warmup 200
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG_ROOT = os.path.join(ROOT, "intel-extension-for-pytorch_amd")
for _p in (ROOT, PKG_ROOT):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published
MFMA_FP32_PEAK_TFLOPS = 157.3   # MI355X dense fp32 matrix, published
MFMA_I8_PEAK_TOPS = 5000.0      # MI355X dense int8, published


# HBM bytes per launch of the dominant kernel.  Hardware counters cannot be read from inside this process:
# the figure comes from two rocprofv3 --pmc runs of `bench.py --probe decode` (FETCH_SIZE 15291.09 KiB and
# WRITE_SIZE 28.00 KiB per dispatch, scaled by what the same counters read for a 256 MiB copy: x2.000 and
# x1.000), whose summary is the file named beside it; keyed by (M, K, N, group size).  Other shapes: null.
PROFILED_HBM_BYTES_PER_LAUNCH = {(1, 4096, 14336, 128): 31354382}
PROFILED_HBM_BYTES_SOURCE = "profiles/woq_decode_m1_kernel_M1_4096x14336_g128.hbm_traffic_and_counters.txt"
# Launches that precede every timed region whatever --warmup says: the first milliseconds after an idle
# period run 3-10 % slower (clocks, translation caches).
MIN_WARMUP_LAUNCHES = 2000


_SPLIT_K_SCRATCH = {}


def algorithmic_bytes(M, K, N, G):
    """INT4 weights 1/2 B, bf16 scales 2 B and packed uint4 zeros 1/2 B per (n, group),
    bf16 activations and outputs."""
    kg = K // G
    return N * K // 2 + N * kg * 2 + N * kg // 2 + M * K * 2 + M * N * 2


def build_params(lib_mod, x, ctx, out, lowp_mode, act_quant_mode=-1, workspace=None):
    p = lib_mod.LinearParams()
    p.struct_size = ctypes.sizeof(lib_mod.LinearParams)
    p.x = x.data_ptr()
    p.x_dtype = lib_mod.ACT_FP32 if x.element_size() == 4 else lib_mod.ACT_BF16
    p.M, p.K, p.N = x.shape[0], ctx.weight_shape_[1], ctx.weight_shape_[0]
    p.qweight = ctx.at_weight_.data_ptr()
    p.weight_dtype = ctx.weight_dtype_
    p.scales_f32 = ctx.scales_list_[0].data_ptr()
    p.scales_f16 = ctx.scales_list_[1].data_ptr()
    p.scales_bf16 = ctx.scales_list_[2].data_ptr()
    p.zeros_u8 = ctx.zeros_u8_.data_ptr() if ctx.zeros_u8_ is not None else None
    p.scale_zero_f16x2 = ctx.scale_zero_f16x2_.data_ptr() if ctx.scale_zero_f16x2_ is not None else None
    p.scale_zero_bf16 = ctx.scale_zero_bf16_.data_ptr() if ctx.scale_zero_bf16_ is not None else None
    p.group_size = ctx.group_size_
    p.bias = ctx.bias_f32_.data_ptr() if ctx.bias_f32_ is not None else None
    p.lowp_mode = lowp_mode
    p.act_quant_mode = act_quant_mode
    p.fusion = 0
    p.out = out.data_ptr()
    p.out_dtype = lib_mod.ACT_FP32 if out.element_size() == 4 else lib_mod.ACT_BF16
    if workspace is None and lowp_mode != 3:
        # what the op layer passes for small batches: scratch that lets the decode kernel split K
        # across workgroups, and the zeroed counters that go with it.  One block for all launches of
        # this stream, as the op layer gets from torch's caching allocator call after call.
        nbytes = lib_mod.load().woq_hip_linear_split_k_workspace_bytes(p.M, p.N)
        if nbytes:
            import torch

            if "counters" not in _SPLIT_K_SCRATCH:
                _SPLIT_K_SCRATCH["counters"] = torch.zeros(512, dtype=torch.int32, device=x.device)
            if nbytes not in _SPLIT_K_SCRATCH:
                _SPLIT_K_SCRATCH[nbytes] = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
            workspace = _SPLIT_K_SCRATCH[nbytes]
            p.split_k_counters = _SPLIT_K_SCRATCH["counters"].data_ptr()
    if workspace is not None:
        p.workspace = workspace.data_ptr()
        p.workspace_bytes = workspace.numel()
    p.force_kernel = 0
    return p


def time_steps(torch, lib, params, steps, warmup, stream):
    """Launches params round-robin; returns (wall seconds, event milliseconds) for `steps`."""
    n = len(params)
    for i in range(warmup):
        rc = lib.woq_hip_linear(ctypes.byref(params[i % n]))
        assert rc == 0, lib.woq_hip_last_error()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start.record(stream)
    for i in range(steps):
        lib.woq_hip_linear(ctypes.byref(params[i % n]))
    stop.record(stream)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return t1 - t0, start.elapsed_time(stop)


def time_groups(torch, lib, params, steps, stream, groups=9):
    """`groups` timed regions of exactly `steps` launches each (synchronize on both sides, HIP events on
    the launch stream inside); returns the (host wall seconds, event milliseconds) of the median group."""
    runs = sorted((time_steps(torch, lib, params, steps, 0, stream) for _ in range(groups)), key=lambda r: r[1])
    return runs[len(runs) // 2]


def _quantiles(vals):
    v = sorted(vals)
    pick = lambda q: v[min(len(v) - 1, int(q * len(v)))]
    return {"median": round(pick(0.5), 3), "p10": round(pick(0.1), 3), "p90": round(pick(0.9), 3)}


def launch_distribution(torch, lib, params, stream, batches=40, per_batch=100):
    """Spread of the per-launch time: `batches` groups of back-to-back launches, each group between
    its own pair of events (microseconds per launch), and the latency of a single launch on an idle
    device (host clock from the call to the end of a synchronize)."""
    n = len(params)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(batches)]
    torch.cuda.synchronize()
    i = 0
    for e0, e1 in evs:
        e0.record(stream)
        for _ in range(per_batch):
            lib.woq_hip_linear(ctypes.byref(params[i % n]))
            i += 1
        e1.record(stream)
    torch.cuda.synchronize()
    per_launch = [e0.elapsed_time(e1) * 1e3 / per_batch for e0, e1 in evs]
    single = []
    for j in range(200):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        lib.woq_hip_linear(ctypes.byref(params[j % n]))
        torch.cuda.synchronize()
        single.append((time.perf_counter() - t0) * 1e6)
    return ({**_quantiles(per_launch), "batches": batches, "launches_per_batch": per_batch},
            {**_quantiles(single), "launches": len(single), "clock": "host, call to end of synchronize"})


def time_graph(torch, lib, params, steps, warmup):
    """Same launches captured once into a HIP graph (one node per weight copy) and replayed."""
    n = len(params)
    g = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for p in params:
            p.stream = s.cuda_stream
            lib.woq_hip_linear(ctypes.byref(p))
        torch.cuda.synchronize()
        with torch.cuda.graph(g, stream=s):
            for p in params:
                p.stream = torch.cuda.current_stream().cuda_stream
                rc = lib.woq_hip_linear(ctypes.byref(p))
                assert rc == 0, lib.woq_hip_last_error()
    reps = max(1, steps // n)
    for _ in range(max(1, warmup // n)):
        g.replay()
    runs = []
    for _ in range(9):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        start.record()
        for _ in range(reps):
            g.replay()
        stop.record()
        torch.cuda.synchronize()
        runs.append((time.perf_counter() - t0, start.elapsed_time(stop)))
    runs.sort(key=lambda r: r[1])
    return (reps * n,) + runs[len(runs) // 2]


def _rotating_params(torch, lib_mod, ops_mod, case, lowp_mode, dev, stream, min_bytes=640e6, act_quant_mode=-1):
    """One op context per weight copy (enough copies that the working set exceeds the Infinity
    Cache), the launch parameters of each, and the objects that keep the memory alive."""
    M, K, N, G = case["M"], case["K"], case["N"], case["group_size"]
    ctx0 = ops_mod.WoqLinearOpContext(
        case["qweight"].to(dev), case["weight_dtype"], [N, K], case["scales"].to(dev),
        None if case["zeros"] is None else case["zeros"].to(dev),
        None if case["bias"] is None else case["bias"].to(dev), None, None, G, lowp_mode, act_quant_mode,
    )
    ws = None
    if lowp_mode == 3:  # the quantized activations; one block for every launch of this stream
        ws = torch.empty(lib_mod.load().woq_hip_linear_workspace_bytes(M, K, 3, act_quant_mode, G), dtype=torch.uint8,
                         device=dev)
    copies = int(min_bytes // ctx0.at_weight_.numel()) + 1
    x = case["x"].to(dev)
    if case.get("fp32_activations"):  # fp32 compute: lowp_mode NONE on fp32 rows, fp32 output
        x = x.float()
    out = torch.empty(M, N, dtype=x.dtype, device=dev)

    class Copy:
        pass

    params, keep = [], [x, out]
    for i in range(copies):
        c = Copy()
        c.__dict__.update(ctx0.__dict__)
        if i > 0:
            c.at_weight_ = ctx0.at_weight_.clone()
            c.scales_list_ = [t.clone() for t in ctx0.scales_list_]
            c.zeros_u8_ = None if ctx0.zeros_u8_ is None else ctx0.zeros_u8_.clone()
            c.scale_zero_f16x2_ = None if ctx0.scale_zero_f16x2_ is None else ctx0.scale_zero_f16x2_.clone()
            c.scale_zero_bf16_ = None if ctx0.scale_zero_bf16_ is None else ctx0.scale_zero_bf16_.clone()
        keep.append(c)
        p = build_params(lib_mod, x, c, out, lowp_mode, act_quant_mode, ws)
        p.stream = stream.cuda_stream
        params.append(p)
    keep.append(ws)
    return params, keep


def config_sweep(torch, lib, lib_mod, ops_mod, synthetic, dev, stream, steps):
    """The other named configurations, each timed like the headline (rotating weight copies, HIP
    events over back-to-back launches) and reported against its own algorithmic bytes: weights at
    their stored width, bf16 scales (fp32 for the INT8 case), uint4 zeros, bf16 activations, bias
    and outputs."""
    rows = []

    def run(name, case, lowp=2, aq=-1, weight_cache=False):
        M, K, N, G = case["M"], case["K"], case["N"], case["group_size"]
        params, keep = _rotating_params(torch, lib_mod, ops_mod, case, lowp, dev, stream, act_quant_mode=aq)
        if weight_cache:
            # cache_weight_for_large_batch: a dense bf16 copy beside every packed copy (woq_hip_dense_weight)
            from ipex_amd import _kernels as kernels_mod
            for p, c in zip(params, keep[2:]):
                keep.append(kernels_mod.dense_weight(c.at_weight_, c.weight_dtype_, N, K, c.scales_list_[2], c.zeros_u8_, G))
                p.dense_bf16 = keep[-1].data_ptr()
        # Each configuration starts after an idle period (its inputs are generated on the host) and
        # the first few thousand launches after one run up to 10 % slower; single groups of a few
        # hundred launches also scatter by +-5 %.  So: a warm-up as long as one group, then nine
        # groups, and the median group is reported.
        time_steps(torch, lib, params, steps, max(200, steps), stream)
        groups = sorted(time_steps(torch, lib, params, steps, 0, stream)[1] * 1e3 / steps for _ in range(9))
        us = groups[4]
        if case["weight_dtype"] == 2:
            nbytes = algorithmic_bytes(M, K, N, G)
        elif case["weight_dtype"] == 4:  # float8 bytes, bf16 scales per group
            nbytes = N * K + N * ((K + G - 1) // G if G > 0 else 1) * 2 + M * K * 2 + M * N * 2
        else:
            nbytes = N * K + N * 4 + M * K * 2 + M * N * 2 + (N * 2 if case["bias"] is not None else 0)
        row = {"config": name, "M": M, "K": K, "N": N, "group_size": G, "us_per_launch": round(us, 2),
               "us_p10_p90": [round(groups[1], 2), round(groups[7], 2)]}
        if M >= 256:  # MFMA-bound: a rate in flops, not in bytes
            row["tflops"] = round(2.0 * M * K * N / us / 1e6, 1)
            if case.get("fp32_activations"):
                row["frac_of_fp32_mfma_peak"] = round(2.0 * M * K * N / us / 1e6 / MFMA_FP32_PEAK_TFLOPS, 3)
            else:
                row["frac_of_bf16_mfma_peak"] = round(2.0 * M * K * N / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 3)
        else:
            row["GB_per_s"] = round(nbytes / us / 1e3, 1)
            row["frac_of_hbm_peak"] = round(nbytes / us / 1e3 / HBM_PEAK_GBS, 3)
        if weight_cache:
            row["kernel"] = lib_mod.last_kernel()
        rows.append(row)
        del params, keep
        torch.cuda.empty_cache()

    run("C0 int4 g128 M=1 4096->4096", synthetic.make_int4_case(0, 1, 4096, 4096, 128))
    run("C1 int8 per-channel M=32 4096->11008 +bias", synthetic.make_int8_case(1, 32, 4096, 11008))
    for M in (4, 8, 16):
        run(f"C2 int4 g128 M={M} 4096->14336", synthetic.make_int4_case(2, M, 4096, 14336, 128))
    for M in (1, 4, 8, 16):
        run(f"C2 int4 g128 M={M} 14336->4096", synthetic.make_int4_case(2, M, 14336, 4096, 128))
    block = 0.0
    for K, N, what in ((4096, 6144, "qkv"), (4096, 4096, "o"), (4096, 28672, "gate+up"), (14336, 4096, "down")):
        run(f"C4 int4 g32 M=16 {what} {K}->{N}", synthetic.make_int4_case(4, 16, K, N, 32))
        block += rows[-1]["us_per_launch"]
    rows.append({"config": "C4 decoder block, summed WOQ-linear time per token step", "us": round(block, 2)})
    # Beyond the named configurations: what the same layers cost in the neighbouring settings a user of
    # the reference may run (single-stream decode of a group-32 model, lowp_mode INT8 decode with
    # per-row and per-(row, K block) activation scales, INT8 weights at prefill size, asymmetric
    # activations, a group-64 model and INT8 weights at a serving batch under lowp_mode INT8).
    run("extra: int4 g128 M=1 4096->28672 (gate+up in one launch, lowp BF16)", synthetic.make_int4_case(5, 1, 4096, 28672, 128))
    run("extra: int4 g32 M=1 4096->14336 (lowp BF16)", synthetic.make_int4_case(5, 1, 4096, 14336, 32))
    run("extra: int4 g128 M=1 4096->14336 lowp INT8 per-row", synthetic.make_int4_case(5, 1, 4096, 14336, 128), 3, 6)
    run("extra: int4 g128 M=16 4096->14336 lowp INT8 per-row-and-K-block", synthetic.make_int4_case(5, 16, 4096, 14336, 128), 3, 7)
    run("extra: int4 g32 M=1 4096->14336 lowp INT8 per-row-and-K-block", synthetic.make_int4_case(5, 1, 4096, 14336, 32), 3, 7)
    run("extra: int8 per-channel M=2048 4096->11008 +bias (lowp BF16)", synthetic.make_int8_case(5, 2048, 4096, 11008))
    run("extra: int4 g32 M=2048 qkv 4096->6144 (lowp BF16, 256 x 192 tiles)", synthetic.make_int4_case(5, 2048, 4096, 6144, 32))
    run("extra: fp8 e4m3fn g128 M=1 4096->14336 (lowp BF16)", synthetic.make_fp8_case(5, 1, 4096, 14336, bias=False, group_size=128))
    run("extra: fp8 e4m3fn g128 M=2048 4096->14336 (lowp BF16)", synthetic.make_fp8_case(5, 2048, 4096, 14336, bias=False, group_size=128))
    # the same large batches with cache_weight_for_large_batch (dense bf16 copy, rotating like the packed copies)
    run("extra: int8 per-channel M=2048 4096->11008 +bias (lowp BF16, cache_weight_for_large_batch)",
        synthetic.make_int8_case(5, 2048, 4096, 11008), weight_cache=True)
    run("extra: fp8 e4m3fn g128 M=2048 4096->14336 (lowp BF16, cache_weight_for_large_batch)",
        synthetic.make_fp8_case(5, 2048, 4096, 14336, bias=False, group_size=128), weight_cache=True)
    run("extra: int4 g128 M=1024 4096->14336 (lowp BF16)", synthetic.make_int4_case(5, 1024, 4096, 14336, 128))
    run("extra: int4 g128 M=1024 4096->14336 (lowp BF16, cache_weight_for_large_batch)",
        synthetic.make_int4_case(5, 1024, 4096, 14336, 128), weight_cache=True)
    run("extra: int4 g128 M=16 4096->14336 lowp INT8 asymmetric per-row", synthetic.make_int4_case(5, 16, 4096, 14336, 128), 3, 2)
    run("extra: int4 g64 M=128 4096->14336 lowp INT8 per-row", synthetic.make_int4_case(5, 128, 4096, 14336, 64), 3, 6)
    run("extra: int8 per-channel M=128 4096->11008 +bias lowp INT8 per-row", synthetic.make_int8_case(5, 128, 4096, 11008), 3, 6)
    rows.extend(moe_layer_rows(torch, ops_mod, synthetic, dev))
    # fp32 compute: the reference's default qconfig (INT8 weights, lowp_mode NONE) on an fp32 model
    case = synthetic.make_int8_case(5, 2048, 4096, 11008)
    case["fp32_activations"] = True
    run("extra: int8 per-channel M=2048 4096->11008 +bias, fp32 activations, lowp NONE (fp32 MFMA)", case, 0)
    return rows


def moe_layer_rows(torch, ops_mod, synthetic, dev, experts=32, H=7168, I=2048, topk=8):
    """One mixture-of-experts layer over INT4 g128 experts (gate / up 7168 -> 2048, down 2048 -> 7168, top-8 of 32
    experts) through torch.ops.torch_ipex.deepseek_moe_woq: microseconds per layer, wall clock over 20 calls without
    synchronization in between, with the routing sorted on the device and grouped launches (the default up to 64
    tokens) and with the per-expert launches that read the routing on the host."""
    import os
    import time

    def ctx(K, N, seed):
        c = synthetic.make_int4_case(seed, 1, K, N, 128)
        return ops_mod.WoqLinearOpContext(c["qweight"].to(dev), 2, [N, K], c["scales"].to(dev), c["zeros"].to(dev), None, None,
                                          None, 128, 2, -1, False)

    lists = [[ctx(H, I, 600 + e % 4) for e in range(experts)], [ctx(H, I, 610 + e % 4) for e in range(experts)],
             [ctx(I, H, 620 + e % 4) for e in range(experts)]]
    op = torch.ops.torch_ipex.deepseek_moe_woq
    g = torch.Generator().manual_seed(7)
    rows = []
    saved = os.environ.get("IPEX_AMD_MOE_GROUPED")
    try:
        for T in (1, 16):
            x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
            ids = torch.stack([torch.randperm(experts, generator=g)[:topk] for _ in range(T)]).to(dev)
            rw = torch.softmax(torch.randn(T, topk, generator=g), -1).to(torch.bfloat16).to(dev)
            us = {}
            for mode in ("1", "0"):
                os.environ["IPEX_AMD_MOE_GROUPED"] = mode
                for _ in range(3):
                    op(x, ids, lists[0], lists[1], lists[2], rw, False)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(20):
                    op(x, ids, lists[0], lists[1], lists[2], rw, False)
                torch.cuda.synchronize()
                us[mode] = (time.perf_counter() - t0) / 20 * 1e6
            active = len(set(ids.flatten().tolist()))
            wbytes = active * 3 * H * I // 2
            rows.append({"config": f"extra: MoE layer, {experts} INT4 g128 experts 7168->2048->7168, top-{topk}, {T} token(s)",
                         "tokens": T, "active_experts": active, "us_per_layer_grouped": round(us["1"], 1),
                         "us_per_layer_per_expert_launches": round(us["0"], 1),
                         "GB_per_s_of_active_weights": round(wbytes / us["1"] / 1e3, 1),
                         "frac_of_hbm_peak": round(wbytes / us["1"] / 1e3 / HBM_PEAK_GBS, 3)})
    finally:
        if saved is None:
            os.environ.pop("IPEX_AMD_MOE_GROUPED", None)
        else:
            os.environ["IPEX_AMD_MOE_GROUPED"] = saved
    del lists
    torch.cuda.empty_cache()
    return rows


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as fh:
            for line in fh:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _oracle_lib():
    so = os.path.join(ROOT, "oracle", "libwoq_oracle.so")
    if not os.path.exists(so):
        return None
    cores = len(os.sched_getaffinity(0))
    os.environ.setdefault("OMP_NUM_THREADS", str(cores))
    lib = ctypes.CDLL(so)
    vp, i64 = ctypes.c_void_p, ctypes.c_int64
    lib.woq_ref_linear_int4.argtypes = [vp, i64, i64, i64, vp, vp, vp, i64, vp, ctypes.c_int, i64, i64, vp]
    lib.woq_ref_linear_int4_fp16_chain.argtypes = [vp, i64, i64, i64, vp, vp, vp, i64, i64, vp, i64, i64, vp]
    lib.woq_ref_quant_per_row.argtypes = [vp, i64, i64, vp, vp]
    lib.woq_ref_linear_int4_int8.argtypes = [vp, vp, i64, i64, i64, vp, vp, vp, i64, i64, vp, i64, i64, vp]
    return lib, cores


def _case_arrays(case):
    import numpy as np

    torch = __import__("torch")
    x = case["x"].view(torch.int16).numpy().astype(np.uint16)
    qw = np.ascontiguousarray(case["qweight"].numpy())
    sc = np.ascontiguousarray(case["scales"].float().numpy())
    zp = np.ascontiguousarray(case["zeros"].float().numpy())
    return x, qw, sc, zp


def _timed_passes(run, budget_s, at_least=3, at_most=200):
    run()
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < at_least or (time.perf_counter() < t_end and len(times) < at_most):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    return sorted(times)[len(times) // 2], len(times)


CPU_LABEL = "CPU restatement of IPEX woq_linear (IPEX binary unavailable)"


def cpu_baseline_decode(case, K, N, G, budget_s=8.0, gpu_out=None):
    """The oracle's C port (OpenMP over output channels) on the same decode workload, timed on the host cores this
    process may use, in the two numerics the reference has for fewer than five rows: `ref`, its fallback
    (woq_gemm_ref_impl: weights dequantized and rounded to fp16, fp32 accumulation; what it runs on a host without
    AVX512-FP16, and the figure in `value`), and `opt`, its AVX512-FP16 kernel (fp16 fused multiply-adds on integer
    weights per K block of 64, fp16 accumulators).  With `gpu_out` (the GPU's bf16 output for the same inputs, on
    the host) both results check it."""
    import numpy as np

    loaded = _oracle_lib()
    if loaded is None:
        return None
    lib, cores = loaded
    x, qw, sc, zp = _case_arrays(case)
    acc = np.zeros((1, N), dtype=np.float32)
    chain = np.zeros((1, N), dtype=np.float32)
    run_ref = lambda: lib.woq_ref_linear_int4(x.ctypes.data, 1, K, N, qw.ctypes.data, sc.ctypes.data, zp.ctypes.data, G,
                                              None, 0, 0, N, acc.ctypes.data)
    run_opt = lambda: lib.woq_ref_linear_int4_fp16_chain(x.ctypes.data, 1, K, N, qw.ctypes.data, sc.ctypes.data,
                                                         zp.ctypes.data, G, 64, None, 0, N, chain.ctypes.data)
    med, n = _timed_passes(run_ref, budget_s, at_least=10)
    med_o, n_o = _timed_passes(run_opt, budget_s / 2, at_least=5)
    nbytes = algorithmic_bytes(1, K, N, G)
    res = {
        "value": round(nbytes / med / 1e9, 3),
        "unit": "GB/s",
        "cores": cores,
        "kind": "port",
        "numerics": "ref",
        "sample": f"full workload (M=1, K={K}, N={N}), median of {n} passes of oracle/woq_ref.c (woq_ref_linear_int4, fp16-rounded weights)",
        "ms_per_step": round(med * 1e3, 4),
        "cpu_model": _cpu_model(),
        "label": CPU_LABEL,
        "opt": {"value": round(nbytes / med_o / 1e9, 3), "unit": "GB/s", "ms_per_step": round(med_o * 1e3, 4),
                "sample": f"full workload, median of {n_o} passes of woq_ref_linear_int4_fp16_chain (scalar software fp16 "
                          "fused multiply-adds: the arithmetic of the AVX512-FP16 kernel, not its speed)"},
    }
    if gpu_out is not None:
        torch = __import__("torch")
        got = gpu_out.float().numpy().reshape(-1).astype(np.float64)
        # the reference rounds the fp32 sum to fp16 and then to the activation dtype
        want = torch.from_numpy(acc.reshape(-1).copy()).half().bfloat16().double().numpy()
        want_o = torch.from_numpy(chain.reshape(-1).copy()).bfloat16().double().numpy()
        rel = lambda w: float(np.linalg.norm(got - w) / np.linalg.norm(w))
        res["parity_of_gpu_output"] = {
            "max_abs": round(float(np.abs(got - want).max()), 6),
            "rel_l2": round(rel(want), 7),
            "rel_l2_gate": 2e-3,
            "ok": bool(rel(want) <= 2e-3),
            "against": "ref: this port with fp16-rounded weights and fp32 accumulation, sum rounded to fp16 then bf16",
            "rel_l2_vs_opt": round(rel(want_o), 7),
            "vs_opt_note": "opt accumulates in fp16: its own rounding noise at K = 4096 exceeds the gate, so it is reported, not gated",
        }
    return res


def cpu_baseline_prefill(case, M, K, N, G, gpu_out=None, budget_s=8.0):
    """The same port on a bounded sample of the prefill workload: all M rows against the first `cols` output
    channels, sized so that one pass takes about two seconds.  For five rows and more the reference's fallback and
    its optimized bf16 kernel compute the same numbers when there is no bias (weights rounded to bf16, bf16 x bf16
    products, fp32 accumulation), so one timing stands for `ref` and `opt`; lowp_mode INT8 (`opt` only: the fallback
    does not quantize activations) is the per-row quantization plus the int32 block sums with their fp32 epilogue."""
    import numpy as np

    loaded = _oracle_lib()
    if loaded is None:
        return None
    lib, cores = loaded
    x, qw, sc, zp = _case_arrays(case)
    acc = np.zeros((M, N), dtype=np.float32)

    def bf16(cols):
        lib.woq_ref_linear_int4(x.ctypes.data, M, K, N, qw.ctypes.data, sc.ctypes.data, zp.ctypes.data, G, None, 1, 0,
                                cols, acc.ctypes.data)

    t0 = time.perf_counter()
    bf16(4 * cores)
    trial = time.perf_counter() - t0
    cols = int(min(N, max(4 * cores, 4 * cores * 2.0 / max(trial, 1e-4)))) // cores * cores
    med, n = _timed_passes(lambda: bf16(cols), budget_s, at_least=2, at_most=10)
    flops = 2.0 * M * K * cols
    res = {
        "value": round(flops / med / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "numerics": "ref = opt (bf16-rounded weights, fp32 accumulation, no bias)",
        "sample": f"all {M} rows x the first {cols} of {N} output channels, median of {n} passes of oracle/woq_ref.c",
        "seconds_per_full_step_extrapolated": round(med * N / cols, 3),
        "cpu_model": _cpu_model(),
        "label": CPU_LABEL,
    }
    if gpu_out is not None:
        got = gpu_out[:, :cols].float().numpy().astype(np.float64)
        torch = __import__("torch")
        want = torch.from_numpy(acc[:, :cols].copy()).bfloat16().double().numpy()
        rel_l2 = float(np.linalg.norm(got - want) / np.linalg.norm(want))
        res["parity_of_gpu_output"] = {"rel_l2": round(rel_l2, 7), "rel_l2_gate": 2e-3, "ok": bool(rel_l2 <= 2e-3),
                                       "columns": cols}
    # lowp_mode INT8, per-row symmetric activation scales
    xq = np.zeros((M, K), dtype=np.int8)
    sa = np.zeros(M, dtype=np.float32)

    def int8(c):
        lib.woq_ref_quant_per_row(x.ctypes.data, M, K, xq.ctypes.data, sa.ctypes.data)
        lib.woq_ref_linear_int4_int8(xq.ctypes.data, sa.ctypes.data, M, K, N, qw.ctypes.data, sc.ctypes.data,
                                     zp.ctypes.data, G, min(G, 128), None, 0, c, acc.ctypes.data)

    med8, n8 = _timed_passes(lambda: int8(cols), budget_s / 2, at_least=2, at_most=10)
    res["lowp_int8_opt"] = {"value": round(flops / med8 / 1e12, 4), "unit": "TOP/s",
                            "sample": f"the same {cols} channels, activation quantization included, median of {n8} passes"}
    return res


def _calibration_copy(torch, dev):
    """One 256 MiB device-to-device copy: FETCH_SIZE / WRITE_SIZE of this dispatch against its known size
    give the factors that turn the counters of the other dispatches into bytes."""
    src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    dst.copy_(src)
    torch.cuda.synchronize()
    return 256 << 20


def run_probe(name, torch, lib, lib_mod, ops_mod, synthetic, dev, stream):
    """Short fixed workloads for `rocprofv3 --pmc ... -- python3 bench.py --probe NAME` (one counter set per
    run) and for `rocprofv3 --kernel-trace --stats`: a few launches of one kernel family over rotating
    weight copies (every launch reads its weights from HBM), then a device copy of known size that
    calibrates the byte counters.  Prints one JSON line saying what was launched."""
    info = {"probe": name}
    if name == "decode_dq":
        # the bf16-regime decode kernel at the named M = 16 shapes (both layers of a gated MLP)
        info["launches"] = []
        for K, N in ((4096, 14336), (14336, 4096)):
            case = synthetic.make_int4_case(2, 16, K, N, 128)
            params, keep = _rotating_params(torch, lib_mod, ops_mod, case, 2, dev, stream)
            for i in range(66):
                assert lib.woq_hip_linear(ctypes.byref(params[i % len(params)])) == 0, lib.woq_hip_last_error()
            torch.cuda.synchronize()
            info["launches"].append({"M": 16, "K": K, "N": N, "G": 128, "count": 66, "kernel": lib_mod.last_kernel(),
                                     "algorithmic_bytes_per_launch": algorithmic_bytes(16, K, N, 128)})
            del params, keep
    elif name == "prefill":
        # the named prefill configuration under lowp_mode BF16 and INT8 (per-row activation scales)
        K, N, G, Mp = 4096, 14336, 128, 2048
        case = synthetic.make_int4_case(3, Mp, K, N, G, outliers=True)
        info["launches"] = []
        # (third: lowp_mode BF16 on the kernel that dequantizes once per workgroup into LDS)
        # (fourth: lowp_mode BF16 with cache_weight_for_large_batch, the dense kernel on the bf16 copy)
        from ipex_amd import _kernels as kernels_mod
        for lowp, aq, forced in ((2, -1, 0), (3, 6, 0), (2, -1, 21), (2, -1, 23)):
            params, keep = _rotating_params(torch, lib_mod, ops_mod, case, lowp, dev, stream, min_bytes=1, act_quant_mode=aq)
            params[0].force_kernel = forced
            if forced == 23:
                c = keep[2]
                keep.append(kernels_mod.dense_weight(c.at_weight_, c.weight_dtype_, N, K, c.scales_list_[2], c.zeros_u8_, G))
                params[0].dense_bf16 = keep[-1].data_ptr()
            for _ in range(20):
                assert lib.woq_hip_linear(ctypes.byref(params[0])) == 0, lib.woq_hip_last_error()
            torch.cuda.synchronize()
            info["launches"].append({"M": Mp, "K": K, "N": N, "G": G, "lowp_mode": lowp, "count": 20,
                                     "kernel": lib_mod.last_kernel(), "flops_per_launch": 2.0 * Mp * K * N})
            del params, keep
    elif name == "floor":
        # the headline decode workload beside the probes: the kernel and the pure read of its bytes, from HBM and
        # cache-resident
        case = synthetic.make_int4_case(2, 1, 4096, 14336, 128)
        params, keep = _rotating_params(torch, lib_mod, ops_mod, case, 2, dev, stream)
        info.update(floor_probe(torch, lib, dev, stream, decode_params=params))
        info["decode_kernel"] = lib_mod.last_kernel()
        print(json.dumps(info))
        return
    elif name == "mfma":
        info.update(mfma_issue_probe(torch, lib, dev, stream))
        print(json.dumps(info))
        return
    else:
        raise SystemExit(f"unknown probe {name!r}")
    info["calibration_copy_bytes"] = _calibration_copy(torch, dev)
    print(json.dumps(info))


_PROBES = []


def probe_lib():
    """lib/libwoq_bench_probes.so: the streaming-read, empty-kernel and MFMA-issue probes.  A library of the benchmark's
    own, built beside the product libraries; the product library and its C ABI carry no measurement code."""
    if not _PROBES:
        path = os.path.join(PKG_ROOT, "lib", "libwoq_bench_probes.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: run `python __graft_entry__.py` (or csrc/build.py) first")
        lib = ctypes.CDLL(path)
        vp, i32, i64 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64
        lib.woq_bench_probe_stream_read.restype = i32
        lib.woq_bench_probe_stream_read.argtypes = [vp, i64, i32, i32, vp, vp]
        lib.woq_bench_probe_empty.restype = i32
        lib.woq_bench_probe_empty.argtypes = [i64, i32, vp]
        lib.woq_bench_probe_mfma_issue.restype = i32
        lib.woq_bench_probe_mfma_issue.argtypes = [vp, i32, i32, i64, i32, i32, vp, vp]
        _PROBES.append(lib)
    return _PROBES[0]


def floor_probe(torch, lib, dev, stream, groups=9, per_group=200, decode_params=None):
    """What a launch of the headline decode kernel's shape costs without its arithmetic: an empty kernel
    of the same grid (448 workgroups of 16 waves) and pure streaming reads of the same 28 MiB of packed
    weights (rotating over 23 distinct buffers, 675 MB, so that every launch reads HBM) in several
    launch shapes; microseconds per launch, median of `groups` groups of `per_group` back-to-back launches.
    Each read shape is timed a second time on ONE buffer, which the caches then hold (28 MiB in the 256 MiB
    Infinity Cache): what remains of the launch when the bytes do not come from HBM.  With `decode_params` (the launch
    parameters of the decode kernel over rotating weight copies) the kernel itself is timed the same two ways, so that
    its distance to the read of the same bytes is stated for both."""
    probes = probe_lib()
    nbytes = 14336 * 4096 // 2
    bufs = [torch.empty(nbytes, dtype=torch.uint8, device=dev).random_(0, 256) for _ in range(23)]
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    st = ctypes.c_void_p(stream.cuda_stream)

    def timed(launch):
        for i in range(per_group):
            launch(i)
        vals = []
        for _ in range(groups):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record(stream)
            for i in range(per_group):
                launch(i)
            e1.record(stream)
            torch.cuda.synchronize()
            vals.append(e0.elapsed_time(e1) * 1e3 / per_group)
        return round(sorted(vals)[len(vals) // 2], 3)

    out = {"bytes_per_launch": nbytes, "rotating_buffers": len(bufs)}

    def empty(i):
        assert probes.woq_bench_probe_empty(448, 16, st) == 0

    out["empty_kernel_448x16_waves_us"] = timed(empty)
    reads = {}
    for waves, kib in ((16, 4), (16, 2), (8, 4), (8, 8), (4, 8), (16, 1)):
        def read(i, waves=waves, kib=kib, rotate=True):
            buf = bufs[i % len(bufs)] if rotate else bufs[0]
            rc = probes.woq_bench_probe_stream_read(ctypes.c_void_p(buf.data_ptr()), nbytes, waves, kib,
                                                    ctypes.c_void_p(sink.data_ptr()), st)
            assert rc == 0, rc

        us = timed(read)
        hot = timed(lambda i, read=read: read(i, rotate=False))
        reads[f"{waves}_waves_x_{kib}_KiB"] = {"us": us, "GB_per_s": round(nbytes / us / 1e3, 1),
                                               "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 3),
                                               "us_cache_resident": hot}
    out["stream_read_us"] = reads
    best = min(v["us"] for v in reads.values())
    out["best_stream_read_us"] = best
    out["best_stream_read_cache_resident_us"] = min(v["us_cache_resident"] for v in reads.values())
    if decode_params:
        def decode(i, rotate=True):
            rc = lib.woq_hip_linear(ctypes.byref(decode_params[i % len(decode_params) if rotate else 0]))
            assert rc == 0, lib.woq_hip_last_error()

        d_us, d_hot = timed(decode), timed(lambda i: decode(i, rotate=False))
        out["decode_kernel_us"] = {"from_hbm": d_us, "cache_resident": d_hot}
        # the same split for the kernel and for the pure read of its weight bytes
        out["decomposition_us"] = {
            "empty_launch": out["empty_kernel_448x16_waves_us"],
            "read_of_the_weights_cache_resident": out["best_stream_read_cache_resident_us"],
            "read_of_the_weights_from_hbm": best,
            "kernel_cache_resident": d_hot,
            "kernel_from_hbm": d_us,
            "hbm_part_of_the_read": round(best - out["best_stream_read_cache_resident_us"], 3),
            "hbm_part_of_the_kernel": round(d_us - d_hot, 3),
            "kernel_over_read_cache_resident": round(d_hot - out["best_stream_read_cache_resident_us"], 3),
            "kernel_over_read_from_hbm": round(d_us - best, 3),
        }
    return out


def mfma_issue_probe(torch, lib, dev, stream, iters=1500, repeats=5):
    """What bounds the prefill GEMM's K loop, measured without it: 256 workgroups of four waves (one wave per
    SIMD on every CU; some mixes again with eight, two per SIMD), each wave issuing `iters` x 16 independent v_mfma_f32_16x16x32_bf16 on random bf16
    operands with V fp32 FMAs and L ds_read_b128 per 16 MFMAs spread between them.  Per mix: microseconds per
    launch (median of `repeats`), nanoseconds per MFMA and wave, and the TFLOP/s of the whole chip.  The
    prefill kernel's loop issues 40 VALU and 2.8 LDS reads per 16 MFMAs."""
    probes = probe_lib()
    src = torch.randn(3 * 256 * 8, device=dev).to(torch.bfloat16)  # 12 KiB: LDS tile, A and B fragments
    st = ctypes.c_void_p(stream.cuda_stream)
    rows = []
    one = [(0, 0), (16, 0), (32, 0), (40, 0), (48, 0), (64, 0), (0, 3), (0, 8), (0, 16), (32, 3), (40, 3), (48, 3), (20, 6)]
    two = [(0, 0), (40, 0), (40, 3), (48, 3), (20, 6)]
    for waves, valu, lds in [(4, v, l) for v, l in one] + [(8, v, l) for v, l in two]:
        def launch():
            rc = probes.woq_bench_probe_mfma_issue(ctypes.c_void_p(src.data_ptr()), valu, lds, 256, waves, iters, None, st)
            assert rc == 0, rc

        launch()
        vals = []
        for _ in range(repeats):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record(stream)
            launch()
            e1.record(stream)
            torch.cuda.synchronize()
            vals.append(e0.elapsed_time(e1) * 1e3)
        us = sorted(vals)[len(vals) // 2]
        mfmas = iters * 16
        rows.append({"waves_per_workgroup": waves, "valu_per_16_mfma": valu, "lds_reads_per_16_mfma": lds,
                     "us_per_launch": round(us, 1), "ns_per_mfma_and_wave": round(us * 1e3 / mfmas, 2),
                     "tflops": round(256 * waves * mfmas * 16384 / us / 1e6, 1),
                     "frac_of_bf16_mfma_peak": round(256 * waves * mfmas * 16384 / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 3)})
    return {"workgroups": 256, "mfma_per_wave": iters * 16, "mixes": rows}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=4000)
    ap.add_argument("--warmup", type=int, default=2000,
                    help="untimed launches before the timed ones; at least %d are run whatever is asked "
                         "(the first few milliseconds after an idle period run 3-10 %%%% slower: clocks and "
                         "translation caches are still warming up)" % MIN_WARMUP_LAUNCHES)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-prefill", action="store_true", help="skip the M=2048 measurement")
    ap.add_argument("--no-sweep", action="store_true", help="skip the other named configurations")
    ap.add_argument("--no-floor", action="store_true", help="skip the streaming-read / empty-kernel floor")
    ap.add_argument("--M", type=int, default=1, help="decode batch (1..16)")
    ap.add_argument("--probe", choices=["decode", "decode_dq", "prefill", "floor", "mfma"],
                    help="short fixed workload for a rocprofv3 run (counters or kernel trace) instead of the benchmark")
    ap.add_argument("--traffic-probe", action="store_true", help="same as --probe decode")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if args.traffic_probe:
        args.probe = "decode"

    import torch

    import ipex_amd  # noqa: F401
    from ipex_amd import _kernels, _lib, ops
    from ipex_amd.utils import synthetic

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    lib = _lib.load()
    dev = torch.device("cuda", 0)
    stream = torch.cuda.current_stream()
    K, N, G, M = 4096, 14336, 128, args.M

    if args.probe and args.probe != "decode":
        run_probe(args.probe, torch, lib, _lib, ops, synthetic, dev, stream)
        return _finish()

    case = synthetic.make_int4_case(2, M, K, N, G)
    ctx0 = ops.WoqLinearOpContext(
        case["qweight"].to(dev), 2, [N, K], case["scales"].to(dev), case["zeros"].to(dev), None, None, None, G, 2, -1
    )
    per_copy = ctx0.at_weight_.numel() + sum(t.numel() * t.element_size() for t in ctx0.scales_list_) + ctx0.zeros_u8_.numel()
    copies = int(640e6 // per_copy) + 1
    x = case["x"].to(dev)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)

    class Copy:
        pass

    params = []
    keep = []
    for i in range(copies):
        c = Copy()
        c.__dict__.update(ctx0.__dict__)
        if i > 0:
            c.at_weight_ = ctx0.at_weight_.clone()
            c.scales_list_ = [t.clone() for t in ctx0.scales_list_]
            c.zeros_u8_ = ctx0.zeros_u8_.clone()
            c.scale_zero_f16x2_ = ctx0.scale_zero_f16x2_.clone()
            c.scale_zero_bf16_ = None if ctx0.scale_zero_bf16_ is None else ctx0.scale_zero_bf16_.clone()
        keep.append(c)
        p = build_params(_lib, x, c, out, 2)
        p.stream = stream.cuda_stream
        params.append(p)

    nbytes = algorithmic_bytes(M, K, N, G)
    if args.probe == "decode":
        # 64 launches over distinct weight copies, then one 256 MiB device-to-device copy kernel
        for i in range(64):
            lib.woq_hip_linear(ctypes.byref(params[i % len(params)]))
        torch.cuda.synchronize()
        print(json.dumps({"probe": "decode", "decode_launches": 64, "kernel": _lib.last_kernel(),
                          "calibration_copy_bytes": _calibration_copy(torch, dev),
                          "algorithmic_bytes_per_launch": nbytes}))
        return _finish()

    # Whatever --steps / --warmup ask for, the device is warmed up first and the timed region of exactly
    # `steps` launches is repeated nine times, the median region being reported.
    warm = max(args.warmup, MIN_WARMUP_LAUNCHES)
    time_steps(torch, lib, params, 1, warm, stream)
    wall, ev_ms = time_groups(torch, lib, params, args.steps, stream)
    kernel_name = _lib.last_kernel()
    g_steps, g_wall, g_ev_ms = time_graph(torch, lib, params, args.steps, warm)
    for p in params:
        p.stream = stream.cuda_stream
    # cache-resident figure: the same weight every launch
    time_steps(torch, lib, params[:1], 1, 200, stream)
    _, hot_ms = time_groups(torch, lib, params[:1], args.steps, stream)
    spread, single = launch_distribution(torch, lib, params, stream)
    out_host = out.cpu()

    # Host time per call: the C entry point, and the registered operator (the C++ binding: dispatcher,
    # handle lookup, output allocation, launch), over bursts short enough that the launch queue never fills
    def host_us(call, burst=200, reps=7):
        vals = []
        for _ in range(reps):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(burst):
                call()
            vals.append((time.perf_counter() - t0) * 1e6 / burst)
            torch.cuda.synchronize()
        return round(sorted(vals)[len(vals) // 2], 2)

    tctx = torch.ops.ipex_prepack.weight_only_qlinear_prepack(
        case["qweight"].to(dev), 2, [N, K], case["scales"].to(dev), case["zeros"].to(dev), None, None, None, G, 2, -1, False)
    handle = tctx.get_data_handle()
    op = torch.ops.torch_ipex.ipex_woq_linear
    p0 = ctypes.byref(params[0])
    sp = ctypes.c_void_p(stream.cuda_stream)
    pz = _lib.LinearParams.from_buffer_copy(params[0])
    pz.M = 0
    pz_ref = ctypes.byref(pz)
    probe_buf = torch.empty(K * N // 2, dtype=torch.uint8, device=dev)
    probe_sink = torch.zeros(64, dtype=torch.int32, device=dev)
    host = {"c_abi_woq_hip_linear": host_us(lambda: lib.woq_hip_linear(p0)),
            "torch_ops_ipex_woq_linear": host_us(lambda: op(x, handle)),
            # what the library adds to a launch: its argument checks alone (a call with M = 0 returns behind
            # them); and what the runtime's launch path costs for a kernel of this duration and for an empty
            # one, through the same library (with kernels longer than the host's time per call the launch
            # queue grows during a burst, and the runtime's bookkeeping with it)
            "c_abi_checks_only_M0": host_us(lambda: lib.woq_hip_linear(pz_ref)),
            "stream_read_probe_launch": host_us(
                lambda: probe_lib().woq_bench_probe_stream_read(probe_buf.data_ptr(), probe_buf.numel(), 16, 4, probe_sink.data_ptr(), sp)),
            "empty_kernel_launch": host_us(lambda: probe_lib().woq_bench_probe_empty(448, 16, sp)),
            "what": "host microseconds per call, bursts of 200 calls on an idle device, no synchronization inside a burst"}
    del tctx, probe_buf

    us_launch = ev_ms * 1e3 / args.steps
    us_graph = g_ev_ms * 1e3 / g_steps
    best_us = min(us_launch, us_graph)
    # throughput of the timed region on the device clock (HIP events on the launch stream, inputs resident);
    # the host's wall clock around the same region is reported beside it: with few steps it is dominated
    # by the latency of the closing synchronize
    value = nbytes / (best_us * 1e-6) / 1e9

    result = {
        "metric": "INT4 WOQ linear: GB/s (% of HBM peak) at M=1; TFLOPS at M=2048",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(best_us * 1e-3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": ("bf16 activations (as fp16: exact in fp16's normal range) x int4 weights held as exact fp16 integers "
                  "-> fp32 accumulate (v_mfma_f32_16x16x32_f16; the group scale is applied to the group sum in fp32; "
                  "the reference's M < 5 kernel computes the same algebra with fp16 accumulators)") if M == 1
                 else ("bf16 activations x int4 weights held as exact bf16 integers -> fp32 accumulate "
                       "(v_mfma_f32_16x16x32_bf16; group scale applied to the group sum in fp32)") if M < 5
                 else "bf16 x bf16-rounded dequantized int4 -> fp32 accumulate (v_mfma_f32_16x16x32_bf16)",
        "data": "synthetic",
        "config": {
            "workload": f"INT4 g128 woq_linear decode, M={M}, K={K}, N={N}, lowp_mode=BF16, "
                        f"{copies} rotating weight copies ({copies * per_copy / 1e6:.0f} MB)",
            "algorithmic_bytes_per_step": nbytes,
            "timing": f"{warm} warm-up launches, then 9 regions of {args.steps} back-to-back launches each between "
                      "HIP events on the launch stream; median region",
            "ms_per_step_host_wall": round(min(wall / args.steps, g_wall / g_steps) * 1e3, 6),
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(value, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(value / HBM_PEAK_GBS, 4),
            "traffic": PROFILED_HBM_BYTES_PER_LAUNCH.get((M, K, N, G)),
            "traffic_source": PROFILED_HBM_BYTES_SOURCE if (M, K, N, G) in PROFILED_HBM_BYTES_PER_LAUNCH else None,
            "kernel": kernel_name,
            "us_per_launch_stream": round(us_launch, 3),
            "us_per_launch_graph": round(us_graph, 3),
            "us_per_launch_cache_resident": round(hot_ms * 1e3 / args.steps, 3),
            "us_per_launch_spread": spread,
            "single_launch_latency_us": single,
            "host_us_per_call": host,
        },
    }

    if not args.no_prefill:
        Mp = 2048
        casep = synthetic.make_int4_case(3, Mp, K, N, G, outliers=True)
        xp = casep["x"].to(dev)
        outp = torch.empty(Mp, N, dtype=torch.bfloat16, device=dev)
        flops = 2.0 * Mp * K * N
        pre = {}
        # its own fixed counts, whatever --steps says: 200 warm-up launches (the clock needs about 150 launches of this
        # kernel to settle after the decode phase: 245 us per launch at first, 198 us from then on), then five regions of 40
        warm_p, steps_p, groups_p = 200, 40, 5
        # (bf16_lds_tile: the same problem on the kernel that dequantizes once per workgroup into LDS, force_kernel 21)
        for name, lowp, aq, forced in (("bf16", 2, -1, 0), ("int8", 3, 6, 0), ("bf16_lds_tile", 2, -1, 21)):
            ws = None
            wbytes = lib.woq_hip_linear_workspace_bytes(Mp, K, lowp, aq, G)
            if wbytes:
                ws = torch.empty(wbytes, dtype=torch.uint8, device=dev)
            pp = build_params(_lib, xp, keep[0], outp, lowp, aq, ws)
            pp.stream = stream.cuda_stream
            pp.force_kernel = forced
            time_steps(torch, lib, [pp], 1, warm_p, stream)
            _, ms = time_groups(torch, lib, [pp], steps_p, stream, groups=groups_p)
            us = ms * 1e3 / steps_p
            pre[name] = {"us_per_step": round(us, 2), "tflops": round(flops / (us * 1e-6) / 1e12, 1),
                         "kernel": _lib.last_kernel()}
            if name == "bf16":
                outp_host = outp.cpu()
                # the same kernel with every launch reading its weights from HBM (rotating over the decode phase's
                # copies), for the comparison with the dense copy below
                rot = []
                for c in keep[:12]:
                    q = build_params(_lib, xp, c, outp, lowp, aq, ws)
                    q.stream = stream.cuda_stream
                    rot.append(q)
                _, ms_r = time_groups(torch, lib, rot, steps_p, stream, groups=groups_p)
                pre[name]["us_per_step_rotating_%d_copies" % len(rot)] = round(ms_r * 1e3 / steps_p, 2)
                del rot
            if lowp == 3:  # integer products: against the i8 MFMA peak
                pre[name]["frac_of_i8_mfma_peak"] = round(pre[name]["tflops"] / MFMA_I8_PEAK_TOPS, 4)
                pre[name]["peak_tops"] = MFMA_I8_PEAK_TOPS
                pre[name]["includes"] = "the activation quantization kernel"
        # cache_weight_for_large_batch: the same problem on the dense bf16 copy of the weight (four times the packed
        # bytes), first on one copy like the rows above, then rotating over three (351 MB: every launch reads its
        # weights from HBM)
        dense_copies = [_kernels.dense_weight(keep[0].at_weight_, keep[0].weight_dtype_, N, K, keep[0].scales_list_[2],
                                              keep[0].zeros_u8_, G) for _ in range(3)]
        cached = []
        for d in dense_copies:
            pp = build_params(_lib, xp, keep[0], outp, 2, -1, None)
            pp.stream = stream.cuda_stream
            pp.dense_bf16 = d.data_ptr()
            cached.append(pp)
        time_steps(torch, lib, cached[:1], 1, warm_p, stream)
        _, ms = time_groups(torch, lib, cached[:1], steps_p, stream, groups=groups_p)
        us = ms * 1e3 / steps_p
        same_bits = bool(torch.equal(outp.cpu(), outp_host))
        _, ms_r = time_groups(torch, lib, cached, steps_p, stream, groups=groups_p)
        pre["bf16_weight_cache"] = {
            "us_per_step": round(us, 2), "tflops": round(flops / (us * 1e-6) / 1e12, 1), "kernel": _lib.last_kernel(),
            "frac_of_bf16_mfma_peak": round(flops / (us * 1e-6) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
            "us_per_step_rotating_3_copies": round(ms_r * 1e3 / steps_p, 2),
            "dense_copy_bytes": dense_copies[0].numel() * 2,
            "output_equals_lowp_bf16_bit_for_bit": same_bits,
        }
        del dense_copies, cached
        # For scale: the vendor's dense bf16 GEMM (torch.matmul) on the same activations and the
        # already dequantized weight.  It does no dequantization; its rate on random data is what
        # this chip sustains for the shape (the clock drops under MFMA load with non-zero operands).
        wd = _kernels.dequant_weight(keep[0].at_weight_, keep[0].weight_dtype_, N, K, keep[0].scales_list_[0],
                                     keep[0].zeros_u8_, G, torch.bfloat16)
        for _ in range(warm_p):
            torch.matmul(xp, wd.t())
        dense = []
        for _ in range(groups_p):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            for _ in range(steps_p):
                torch.matmul(xp, wd.t())
            e1.record()
            torch.cuda.synchronize()
            dense.append(e0.elapsed_time(e1) * 1e3 / steps_p)
        us_d = sorted(dense)[len(dense) // 2]
        del wd
        result["prefill_m2048"] = {
            "workload": f"INT4 g128 woq_linear prefill, M={Mp}, K={K}, N={N}",
            "timing": f"{warm_p} warm-up launches, then {groups_p} regions of {steps_p} launches; median region",
            "flops_per_step": flops,
            "lowp_bf16": pre["bf16"],
            "lowp_int8_per_row": pre["int8"],
            "lowp_bf16_dequantized_tile_in_lds": pre["bf16_lds_tile"],
            "lowp_bf16_cache_weight_for_large_batch": pre["bf16_weight_cache"],
            "dense_bf16_vendor_gemm_same_shape": {"us_per_step": round(us_d, 2),
                                                  "tflops": round(flops / (us_d * 1e-6) / 1e12, 1)},
            "frac_of_bf16_mfma_peak": round(pre["bf16"]["tflops"] / MFMA_BF16_PEAK_TFLOPS, 4),
            "peak_tflops": MFMA_BF16_PEAK_TFLOPS,
        }
        if not args.no_cpu:
            # (the prefill launches above run the prefill activations against the decode workload's weights)
            cpu_case = dict(case)
            cpu_case["x"] = casep["x"]
            result["prefill_m2048"]["cpu_baseline"] = cpu_baseline_prefill(cpu_case, Mp, K, N, G, gpu_out=outp_host)

    if not args.no_floor and M == 1:
        # the floor of a launch of this size on this GPU, measured in the same process, and the kernel beside it
        result["roofline"]["launch_floor"] = floor_probe(torch, lib, dev, stream, decode_params=params)
    del params, keep
    torch.cuda.empty_cache()

    if not args.no_sweep and M == 1:
        result["other_configs"] = config_sweep(torch, lib, _lib, ops, synthetic, dev, stream,
                                               max(50, min(400, args.steps // 10)))

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline_decode(synthetic.make_int4_case(2, 1, K, N, G), K, N, G,
                                                     gpu_out=out_host if M == 1 else None)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))
    _finish()


def _finish():
    """Leaves at once: everything is printed, and the runtime's teardown (worker threads of the CPU leg,
    the HIP context) has nothing left to do that a result depends on."""
    import torch

    torch.cuda.synchronize()
    sys.stdout.flush()
    sys.stderr.flush()
    # under rocprofv3 the tool writes its files when the process exits the ordinary way
    if "rocprofiler" in os.environ.get("LD_PRELOAD", "") or os.environ.get("ROCPROFILER_LIBRARY_CTOR"):
        return
    os._exit(0)


if __name__ == "__main__":
    main()
