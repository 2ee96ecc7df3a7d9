#!/usr/bin/env python3
"""Benchmark of the INT8 linear layer (forward + backward) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--scheme block_channel] [--config 2]

One step = one pass of the hot path over one batch of synthetic input resident in HBM:
Y = X W^T, dX = dY W, dW = dY^T X, every operand quantised to int8 on the way (all
quantiser launches are inside the timed region).  The workload is BASELINE.json's
config 2: X 8192x4096 bf16 ~N(0,1) with 1% of the input channels x20, W 4096x4096
~N(0,0.02), dY 8192x4096 ~N(0,1e-3), seed 1, block-channel scheme.

``--config 3|4|5`` times the other benchmark configurations (Llama MLP shapes in the double-channel
scheme; the fused Hadamard path at 8192^3; the decoder layer step and the M = 16 / 128 shapes) with the
same protocol and prints a shorter line; the default, config 2, is the headline.

Prints ONE JSON line.  `value` = 6*M*N*K int8 operations (three GEMMs) divided by the
mean wall-clock time of a step, in TOPS.  `roofline` describes the dominant kernel (the
i8 MFMA GEMM): 2*M*N*K operations per launch over its mean launch duration, measured with
HIP events on the launch stream around each of its launches while whole steps run, in a second
pass of K steps (so the events do not sit in the region `value` is timed on).  `cpu_baseline` is the torch-CPU oracle of the same path
timed once on the host cores on a bounded sample; it is a reported baseline, not a target.
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "INT8 linear fwd+bwd TOPS & % INT8 MFMA peak at 8192x4096x4096"
INT8_PEAK_TOPS = 5000.0   # MI355X dense int8 MFMA peak, 5.0 POP/s
HBM_PEAK_GBS = 8000.0     # MI355X HBM3E, 8 TB/s
M, K, N = 8192, 4096, 4096


def make_inputs(m=M, k=K, n=N, seed=1):
    g = torch.Generator().manual_seed(seed)
    X = torch.randn(m, k, generator=g)
    outl = torch.randperm(k, generator=g)[: (k + 99) // 100]
    X[:, outl] *= 20.0
    W = torch.randn(n, k, generator=g) * 0.02
    dY = torch.randn(m, n, generator=g) * 1e-3
    return X.to(torch.bfloat16), W.to(torch.bfloat16), dY.to(torch.bfloat16)


def make_operand(rows, cols, gen, kind, std=1.0, outlier_frac=0.0, outlier_mul=1.0):
    """bf16 operand of a benchmark configuration: N(0, std), optional outlier channels, or Student-t(3)."""
    if kind == "student_t":
        x = torch.randn(rows, cols, generator=gen) / torch.sqrt(torch.randn(3, rows, cols, generator=gen).pow(2).mean(0))
    else:
        x = torch.randn(rows, cols, generator=gen) * std
    if outlier_frac:
        idx = torch.randperm(cols, generator=gen)[: int(-(-cols * outlier_frac // 1))]
        x[:, idx] *= outlier_mul
    return x.to(torch.bfloat16)


def other_config(args, T, dev):
    """Configs 3-5: the same step protocol on their shapes; one short JSON line."""
    from triton_int8_amd import _lib
    cfg = args.config
    g = torch.Generator().manual_seed(cfg - 1)
    layers = []   # (X, W, dY, scheme, hadamard)
    if cfg == 3:
        for (k, n) in ((4096, 14336), (14336, 4096)):
            layers.append((make_operand(16384, k, g, "normal", outlier_frac=0.005, outlier_mul=50.0),
                           make_operand(n, k, g, "normal", std=0.02), make_operand(16384, n, g, "normal", std=1e-3),
                           "double_channel", None))
        name = "config 3: double_channel fwd+bwd, 16384 tokens, 4096->14336 and 14336->4096, 0.5% channels x50"
    elif cfg == 4:
        layers.append((make_operand(8192, 8192, g, "student_t"), make_operand(8192, 8192, g, "normal", std=0.02),
                       make_operand(8192, 8192, g, "normal", std=1e-3), "block_channel", 128))
        name = "config 4: block_channel + fused 128-point Hadamard fwd+bwd, 8192x8192x8192, X Student-t(3)"
    else:
        for m in (16, 128):
            layers.append((make_operand(m, 4096, g, "normal"), make_operand(4096, 4096, g, "normal", std=0.02),
                           make_operand(m, 4096, g, "normal", std=1e-3), "block_channel", None))
        name = "config 5 (skinny part): block_channel fwd+bwd at M=16 and M=128, K=N=4096"
    layers = [tuple(t.to(dev) if isinstance(t, torch.Tensor) else t for t in l) for l in layers]
    T.init()
    settle(dev)
    ops = sum(6.0 * l[0].shape[0] * l[0].shape[1] * l[1].shape[0] for l in layers)

    def step():
        return [T.linear_fwd_bwd(*l) for l in layers]

    def bf16_step():
        return [(X @ W.t(), dY @ W, dY.t() @ X) for X, W, dY, _, _ in layers]

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.steps

    dt = timed(step)
    out = {"metric": METRIC, "value": round(ops / dt / 1e12, 2), "unit": "TOPS", "n_gpus": 1, "steps": args.steps,
           "warmup": args.warmup, "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": "int8", "data": "synthetic", "config": {"workload": name},
           "pct_int8_peak": round(100.0 * ops / dt / 1e12 / INT8_PEAK_TOPS, 2)}
    if cfg == 5:   # launch-bound shapes: the same step replayed from a HIP graph
        graphed = [T.GraphedStep(lambda x, w, dy, l=l: T.linear_fwd_bwd(x, w, dy, l[3], l[4]), *l[:3], copy_inputs=False) for l in layers]
        out["graph_ms_per_step"] = round(timed(lambda: [gs() for gs in graphed]) * 1e3, 4)
    from triton_int8_amd import linear
    linear.ONE_CALL_STEP = False     # entry point by entry point, so that events fit between the launches (same kernels)
    try:
        step()
        with _lib.timed_launches() as rec:
            for _ in range(args.steps):
                step()
        torch.cuda.synchronize()
    finally:
        linear.ONE_CALL_STEP = True
    out["entry_point_ms_per_step"] = {k: round(sum(a.elapsed_time(b) for a, b in ev) / args.steps, 4) for k, ev in sorted(rec.items())}
    gemm_s = sum(out["entry_point_ms_per_step"].get(k, 0.0) for k in ("ti8_gemm_i8_nt", "ti8_gemm_i8_nt_multi")) * 1e-3
    out["roofline"] = {"bound": "mfma", "achieved": round(ops / gemm_s / 1e12, 1), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                       "frac": round(ops / gemm_s / 1e12 / INT8_PEAK_TOPS, 4), "traffic": None,
                       "note": "all GEMM launches of a step together: 6*M*N*K summed over the layers / their summed event time"}
    out["bf16_matmul_ms_per_step"] = round(timed(bf16_step) * 1e3, 4)
    if cfg == 5:   # the decoder layer training step of the same configuration
        torch.manual_seed(4)
        x = torch.randn(4, 4096, 4096, device=dev, dtype=torch.bfloat16)
        for int8 in (True, False):
            lay = T.decoder.DecoderLayer(4096, 32, 14336, int8=int8, device=dev)

            def layer_step():
                xi = x.clone().requires_grad_(True)
                lay(xi).float().pow(2).mean().backward()
            out["decoder_layer_step_ms_" + ("int8" if int8 else "bf16")] = round(timed(layer_step) * 1e3, 3)
            del lay
    print(json.dumps(out), flush=True)


def event_time_ms(fn, reps):
    """Mean duration of fn() over `reps` launches, HIP events on the current stream."""
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return sum(a.elapsed_time(b) for a, b in evs) / reps


SETTLE_MS = 60.0


def settle(dev, ms=SETTLE_MS):
    """Keep the GPU busy for `ms` milliseconds (bf16 GEMMs, results dropped) before anything is measured: a device that
    has idled -- process start, host-side set-up, half a second of sleep -- runs its first ~20 ms of work at a lower
    clock (the first steps of this benchmark take 0.60 instead of 0.47 ms, HBM-bound kernels lose a third), which is a
    property of the device's power management, not of any kernel.  Every figure of the line is taken after it."""
    a = torch.randn(4096, 4096, device=dev, dtype=torch.bfloat16)
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(20):
            a @ a
        torch.cuda.synchronize()


def probe_mfma(dev, iters=4096, reps=5):
    """What the i8 matrix pipe sustains on a loop of nothing but MFMAs (ti8_probe_mfma): all-zero
    operands, pseudo-random operands, and random operands with the block-channel promotion's vector
    work beside them; the shader clock during each.  The random-operand rate is the practical ceiling
    of a GEMM on real data (the clock falls under the power limit when the data toggles)."""
    from triton_int8_amd import _lib
    wgs = torch.cuda.get_device_properties(dev).multi_processor_count
    sink = torch.empty(wgs * 512, dtype=torch.float32, device=dev)
    clocks = torch.zeros(2, dtype=torch.int64, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    out = {}
    for name, rnd, promo in (("zero_operands", 0, 0), ("random_operands", 1, 0), ("random_operands_with_promotion", 1, 1)):
        call = lambda: _lib.call("ti8_probe_mfma", sink.data_ptr(), sink.numel(), clocks.data_ptr(), wgs, iters, rnd, promo, stream)
        call()
        ms = event_time_ms(call, reps)
        ck = clocks.cpu().tolist()
        ops = wgs * 8.0 * iters * 16 * 65536
        out[name] = {"TOPS": round(ops / (ms * 1e-3) / 1e12, 1), "clock_MHz": round(ck[0] / max(ck[1], 1) * 100.0, 0),
                     "frac_of_nominal": round(ops / (ms * 1e-3) / 1e12 / INT8_PEAK_TOPS, 4)}
    return out


def probe_gemm_data_dependence(T, dev, reps=20):
    """The dominant GEMM kernels on random int8 operands and on all-zero operands of the same shape:
    same instructions, same memory traffic, different switching activity."""
    from triton_int8_amd import ops
    from triton_int8_amd._lib import SCALE_BLOCK128, SCALE_ROW
    g = torch.Generator().manual_seed(0)
    A = torch.randint(-127, 128, (1, M, K), generator=g, dtype=torch.int8).to(dev)
    B = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8).to(dev)
    sa_blk = torch.full((1, M // 128, K // 128), 1e-2, device=dev)
    sa_row, sb_row = torch.full((1, M), 1e-2, device=dev), torch.full((N,), 1e-2, device=dev)
    res = {}
    for data, (a, b) in (("random", (A, B)), ("zero", (torch.zeros_like(A), torch.zeros_like(B)))):
        promo = lambda: ops.gemm_i8_nt(a, b, sa_blk, SCALE_BLOCK128, sb_row, SCALE_ROW)
        i32 = lambda: ops.gemm_i8_nt(a, b, sa_row, SCALE_ROW, sb_row, SCALE_ROW, acc_i32_full=True)
        for name, fn in (("promotion_kernel", promo), ("int32_kernel", i32)):
            fn()
            ms = event_time_ms(fn, reps)
            res[f"{name}_{data}_us"] = round(ms * 1e3, 1)
            res[f"{name}_{data}_TOPS"] = round(2.0 * M * N * K / (ms * 1e-3) / 1e12, 1)
    return res


def cpu_baseline(scheme):
    """The torch-CPU oracle of the same path on the host cores, bounded sample."""
    from oracle import linear as olin
    m, reps = M, 3
    X, W, dY = make_inputs(m=m)
    olin.linear_fwd_bwd(X[:512], W, dY[:512], scheme)   # warm the thread pool / sgemm
    t0 = time.time()
    for _ in range(reps):
        olin.linear_fwd_bwd(X, W, dY, scheme)
    dt = (time.time() - t0) / reps
    return {"value": round(6.0 * m * N * K / dt / 1e12, 4), "unit": "TOPS", "cores": torch.get_num_threads(),
            "kind": "port", "host_cpus": os.cpu_count(), "seconds_per_step": round(dt, 2),
            "sample": f"{reps} full steps of config 2 (fwd+bwd: Y, dX, dW incl. quantisation, {m} tokens x K={K} x N={N}, "
                      f"same seed and distributions) through the torch-CPU oracle (fp32 sgemm per 128-deep K block, exact)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200, help="timed steps (200 x 0.5 ms: box-to-box spread, not timer noise, is what is left)")
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--scheme", default="block_channel", choices=["block_channel", "row_block", "double_channel"])
    ap.add_argument("--config", type=int, default=2, choices=[2, 3, 4, 5], help="benchmark configuration (2 = headline)")
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU baseline leg (profiling runs)")
    ap.add_argument("--probe", choices=["mfma"], help="print what the i8 matrix pipe sustains on pure MFMA loops (zero / random operands, "
                    "clock) and the GEMM kernels on zero against random data, then exit")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build runs on ONE GPU only (the path has no collectives yet); use --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback")

    import triton_int8_amd as T
    from triton_int8_amd import ops

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.probe == "mfma":
        print(json.dumps({"probe": "mfma", "nominal_peak_TOPS": INT8_PEAK_TOPS, "pure_mfma_loop": probe_mfma(dev),
                          "gemm_8192x4096x4096": probe_gemm_data_dependence(T, dev)}), flush=True)
        return
    if args.config != 2:
        return other_config(args, T, dev)
    X, W, dY = (t.to(dev) for t in make_inputs())
    # one-time set-up outside the steps: the library's per-device initialisation (kernel attributes; what the
    # reference's first call spends on compiling and autotuning), and the outputs and workspace of the step, which a
    # training loop over one shape allocates once
    init_note = T.init()
    from triton_int8_amd import _lib, linear
    one_call = args.scheme in linear.ONE_CALL_SCHEMES
    if one_call:
        outs = (torch.empty(M, N, dtype=torch.bfloat16, device=dev), torch.empty(M, K, dtype=torch.bfloat16, device=dev),
                torch.empty(N, K, dtype=torch.bfloat16, device=dev))
        ws = torch.empty(ops.linear_step_workspace_bytes(M, K, N, args.scheme), dtype=torch.uint8, device=dev)

        def step():
            return T.linear_fwd_bwd(X, W, dY, args.scheme, out=outs, workspace=ws)
    else:
        def step():
            return T.linear_fwd_bwd(X, W, dY, args.scheme)

    # ---- the device leaves its idle clocks (settle), then secondary figures FIRST: the bf16 GEMMs the reference times
    # beside its int8 path (test.py:34-38) and the pure-MFMA probe.  They run before the steps, not after, so that the
    # device is at its sustained clock when the warm-up starts:
    # a GPU that has idled (process start, host-side set-up) takes some 20 ms of work to get back there -- steps of
    # 0.60 falling to 0.50 ms over the first twenty against 0.47 ms flat -- and a warm-up of a few steps would leave
    # that ramp inside the timed region
    settle(dev)
    side_reps = 30
    bf16_fns = (lambda: X @ W.t(), lambda: dY @ W, lambda: dY.t() @ X)
    for f in bf16_fns:
        f()
        f()
    bf16_ms = sum(event_time_ms(f, side_reps) for f in bf16_fns)
    probe = probe_mfma(dev, iters=2048, reps=5)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    tops = 6.0 * M * N * K / dt / 1e12

    # which GEMM kernel the timed steps ran, read back from the library: `roofline.kernel` is built from it, and for the
    # block-channel scheme anything but the persistent kernel is a fallback that the line must show
    gemm_kernel_id = T.last_gemm_kernel()
    kernel = _lib.describe_gemm_kernel()
    kernel_check = "ok"
    if args.scheme == "block_channel" and gemm_kernel_id != _lib.KERNEL_PERSISTENT_CHAIN:
        kernel_check = f"FALLBACK: the persistent GEMM kernel did not run ({init_note}; last error: {_lib.lib().ti8_last_error().decode()!r})"
        print("bench.py: " + kernel_check, file=sys.stderr, flush=True)

    # ---- dominant kernel: the GEMM launches of a step (Y, dX, dW), bracketed by HIP events on the launch stream while
    # whole steps run, in a second pass of K steps (so the events do not sit in the region `value` is timed on).  The
    # timed steps are ONE library call each; here the same launches are issued entry point by entry point (same kernels,
    # operands and order), so that events fit between them.
    ev_steps = min(args.steps, 50)
    linear.ONE_CALL_STEP = False
    try:
        for _ in range(3):
            T.linear_fwd_bwd(X, W, dY, args.scheme)
        with _lib.timed_launches() as rec:
            for _ in range(ev_steps):
                T.linear_fwd_bwd(X, W, dY, args.scheme)
        torch.cuda.synchronize()
    finally:
        linear.ONE_CALL_STEP = True
    per_entry_ms = {name: sum(a.elapsed_time(b) for a, b in ev) / ev_steps for name, ev in rec.items()}
    if "ti8_gemm_i8_nt_multi" in rec:
        # Y, dX and dW of a step in ONE launch: three GEMMs' worth of operations per launch
        g = [a.elapsed_time(b) for a, b in rec["ti8_gemm_i8_nt_multi"]]
        assert len(g) == ev_steps
        gemm_ms, gemms_per_launch = [sum(g) / ev_steps], 3
    else:
        g = [a.elapsed_time(b) for a, b in rec["ti8_gemm_i8_nt"]]
        assert len(g) == 3 * ev_steps
        gemm_ms, gemms_per_launch = [sum(g[i::3]) / ev_steps for i in range(3)], 1
    avg_ms = sum(gemm_ms) / len(gemm_ms)
    ops_per_launch = gemms_per_launch * 2.0 * M * N * K
    achieved = ops_per_launch / (avg_ms * 1e-3) / 1e12

    # ---- the activation quantiser and a plain device copy against HBM, behind the steps (memory-bound kernels need the
    # memory side of the device awake as well, which the steps' own quantisers have seen to)
    q_bytes = 4.0 * M * K  # 2 B read + 1 B int8 + 1 B transposed int8 per element
    for _ in range(5):
        ops.quant_block(X[None], clamp=True, with_transpose=True)
    q_ms = event_time_ms(lambda: ops.quant_block(X[None], clamp=True, with_transpose=True), side_reps)
    q1_ms = event_time_ms(lambda: ops.quant_block(X[None], clamp=True), side_reps)
    # a plain device copy of X (64 MiB read + 64 MiB write): the reachable HBM rate on this box,
    # and the known-size kernel the rocprofv3 FETCH_SIZE / WRITE_SIZE counters are calibrated on
    X.clone()
    copy_ms = event_time_ms(lambda: X.clone(), side_reps)

    # HBM-side bytes per GEMM launch: NOT measured by this run.  They come from two rocprofv3 --pmc runs of this
    # command (FETCH_SIZE, WRITE_SIZE), scaled on the device copy above, whose summary is the file named in
    # `traffic_source`; measured for these two schemes
    traffic = {"block_channel": 854975877, "double_channel": 848439911}.get(args.scheme)
    traffic_source = {"block_channel": "profiles/bench_config2_block_channel_counters.md (section 3)",
                      "double_channel": "profiles/bench_config2_double_channel_counters.md (section 3)"}.get(args.scheme)

    # the same quantiser where it runs inside a step: X and dY in one launch (block_channel) or one launch each
    in_step = None
    if "ti8_quant_block_multi" in per_entry_ms:
        t = per_entry_ms["ti8_quant_block_multi"]
        in_step = {"launch_ms": round(t, 4), "operands_per_launch": 2, "frac": round(2 * q_bytes / (t * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    elif "ti8_quant_block" in per_entry_ms:
        t = per_entry_ms["ti8_quant_block"] / 2
        in_step = {"launch_ms": round(t, 4), "operands_per_launch": 1, "frac": round(q_bytes / (t * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    out = {
        "metric": METRIC, "value": round(tops, 2), "unit": "TOPS", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": f"config 2: {args.scheme} INT8 linear fwd+bwd (Y, dX, dW + all quantisers), "
                               f"tokens={M} K={K} N={N}, seed 1, X~N(0,1) 1% channels x20, W~N(0,0.02), dY~N(0,1e-3)",
                   "scheme": args.scheme, "M": M, "K": K, "N": N},
        "pct_int8_peak": round(100.0 * tops / INT8_PEAK_TOPS, 2),
        "roofline": {"bound": "mfma", "achieved": round(achieved, 1), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                     "frac": round(achieved / INT8_PEAK_TOPS, 4), "traffic": traffic, "traffic_measured": False, "traffic_source": traffic_source,
                     "practical_peak": probe["random_operands"]["TOPS"],
                     "frac_of_practical_peak": round(achieved / probe["random_operands"]["TOPS"], 4),
                     "practical_peak_note": "pure v_mfma_i32_32x32x32_i8 loop on random operands in this run (bench.py --probe mfma): "
                                            f"{probe['random_operands']['TOPS']} TOPS at {probe['random_operands']['clock_MHz']:.0f} MHz; "
                                            f"on zero operands {probe['zero_operands']['TOPS']} TOPS at {probe['zero_operands']['clock_MHz']:.0f} MHz",
                     "kernel": kernel,
                     "ops_per_launch": int(ops_per_launch), "gemms_per_launch": gemms_per_launch,
                     "launch_ms": [round(t, 4) for t in gemm_ms],
                     "note": "int8 multiply-adds counted as 2*M*N*K operations per GEMM; peak is the dense int8 MFMA rate"},
        "quant_roofline": {"bound": "hbm", "kernel": "quant_block_kernel<1,true,true>",
                           "achieved": round(q_bytes / (q_ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": round(q_bytes / (q_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "launch_ms": round(q_ms, 4),
                           "frac_of_device_copy": round(q_bytes / q_ms / (2.0 * X.numel() * 2 / copy_ms), 4),
                           "bytes_per_launch": int(q_bytes),
                           "note": "launched back to back on X; `in_step` is the same kernel where it runs inside a step (X and dY, behind a GEMM)",
                           "in_step": in_step,
                           "single_output_GBs": round(3.0 * M * K / (q1_ms * 1e-3) / 1e9, 1)},
        "copy_GBs": round(2.0 * X.numel() * 2 / (copy_ms * 1e-3) / 1e9, 1),
        "bf16_matmul_ms_per_step": round(bf16_ms, 4),
        "bf16_matmul_tflops": round(6.0 * M * N * K / (bf16_ms * 1e-3) / 1e12, 1),
        "entry_point_ms_per_step": {k: round(v, 4) for k, v in sorted(per_entry_ms.items())},
        "between_launches_ms_per_step": round(dt * 1e3 - sum(per_entry_ms.values()), 4),
        "order": f"{SETTLE_MS:.0f} ms of untimed bf16 GEMMs take the device out of its idle clocks, then the bf16 GEMMs of the step's shapes and the "
                 "MFMA probe (about 50 ms of GPU work), then the warm-up and the timed steps, then the per-kernel event pass, the quantiser and the copy",
        "step_issue": "one ti8_linear_fwd_bwd call per step on outputs and a workspace allocated once" if one_call else "entry point by entry point",
        "gemm_kernel_id": gemm_kernel_id, "gemm_kernel_check": kernel_check, "init_note": init_note,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args.scheme)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
