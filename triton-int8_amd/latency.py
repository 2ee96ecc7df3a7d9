"""Latency harness with the protocol and output of the reference's test.py: bf16 ``matmul``
against ``fwd_32`` / ``bwd_33``, 80 calls of which the first 20 are discarded, each timed call
bracketed by a device synchronise, mean wall-clock milliseconds (test.py:13-48).

    python -m triton_int8_amd.latency [--scheme double_channel|block_channel|fused|tilelang] [--size 8192] [--batch 4]
"""
import argparse
import importlib
import time

import torch


def bf16_training(a, b):
    """test.py:7-10: the bf16 baseline, a @ b^T."""
    b_T = b.transpose(-2, -1)
    return torch.matmul(a, b_T)


def measure_latency(func, *args, total_repeat=80, warmup=20, device=None):
    """test.py:13-26, unchanged protocol."""
    times = []
    for i in range(total_repeat):
        if i < warmup:
            func(*args)
            continue
        torch.cuda.synchronize(device)
        start = time.time()
        func(*args)
        torch.cuda.synchronize(device)
        end = time.time()
        times.append(end - start)
    return sum(times) / len(times) * 1000


_MODULES = {"double_channel": ("double_channel_triton_fwd", "double_channel_triton_bwd"),
            "block_channel": ("block_channel_fwd32", "block_channel_bwd33"),
            "fused": ("fused_fwd32", "fused_bwd33"),
            "tilelang": ("tilelang_block_channel_fwd", "tilelang_block_channel_bwd")}


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--scheme", default="double_channel", choices=sorted(_MODULES))
    ap.add_argument("--size", type=int, default=8192, help="M = N = K (test.py uses 8192)")
    ap.add_argument("--batch", type=int, default=4)
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)
    pkg = __package__ or __name__.rsplit(".", 1)[0]
    fwd_32 = importlib.import_module(f"{pkg}.{_MODULES[args.scheme][0]}").fwd_32
    bwd_33 = importlib.import_module(f"{pkg}.{_MODULES[args.scheme][1]}").bwd_33
    device = torch.device(args.device)
    S, B = args.size, args.batch

    a = torch.randn(B, S, S, device=device, dtype=torch.bfloat16)
    b = torch.randn(S, S, device=device, dtype=torch.bfloat16)
    bf16_time = measure_latency(bf16_training, a, b, device=device)
    quant_time = measure_latency(fwd_32, a, b, device=device)
    print(f"fwd32_bf16 time: {bf16_time:.2f} ms")
    print(f"fwd32_int8 time: {quant_time:.2f} ms")
    print(f"fwd32_speedup: {100 * abs(bf16_time - quant_time) / bf16_time:.2f}%")   # the reference's (mis)label
    print("--------------------------------------------------")
    a = torch.randn(B, S, S, device=device, dtype=torch.bfloat16)
    b = torch.randn(B, S, S, device=device, dtype=torch.bfloat16)
    bf16_time = measure_latency(bf16_training, a, b, device=device)
    quant_time = measure_latency(bwd_33, a, b, device=device)
    print(f"bwd33_bf16 time: {bf16_time:.2f} ms")
    print(f"bwd33_int8 time: {quant_time:.2f} ms")
    print(f"bwd33_speedup: {100 * abs(bf16_time - quant_time) / bf16_time:.2f}%")


if __name__ == "__main__":
    main()
