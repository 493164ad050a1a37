"""Sequence-length sweep of one attention layer on the MI355X: forward, backward, or both.

Same command line, shapes and output lines as the reference's sweep (benchmark_single_attention.py:14-22,
92-111: batch 1, 24 heads, head dim 64, bf16, seq 2^10 .. 2^17, block 256, sample 256):

    python -m hyperattention_amd.benchmark_single_attention --mode fwd --attn_method hyper [--no_causal] [--smooth_block]
    python -m hyperattention_amd.benchmark_single_attention --mode fwd+bwd --attn_method flash [--no_causal]

`flash` is this library's exact MFMA attention.  `--mode fwd` times the forward without autograd (for
`hyper` that is the one-call forward); `bwd` times `o.backward(do, retain_graph=True)` and `fwd+bwd` adds
to it the forward as autograd runs it (operator by operator), quantile by quantile, as the reference's
script does (benchmark_single_attention.py:42-52, 70-80).  Times are the 20 % / 50 % / 80 % quantiles in
ms over `rep` calls, each bracketed by events on the launch stream.
"""
import argparse
import sys

import torch

from . import HyperAttention, flash_attn_func


def get_arguments(argv=None):
    parser = argparse.ArgumentParser()
    parser.add_argument("--no_causal", action="store_true")
    parser.add_argument("--smooth_block", action="store_true")
    parser.add_argument("--mode", type=str, default="fwd", choices=["fwd", "bwd", "fwd+bwd"])
    parser.add_argument("--attn_method", type=str, default="flash", choices=["flash", "flash-cuda", "hyper"])
    parser.add_argument("--min_log2_seq", type=int, default=10, help="first sequence length of the sweep (2^k)")
    parser.add_argument("--max_log2_seq", type=int, default=17, help="last sequence length of the sweep (2^k)")
    parser.add_argument("--rep", type=int, default=100)
    # beyond the reference's command line (its shapes are the defaults): other workloads of the same sweep
    parser.add_argument("--batch_size", type=int, default=1)
    parser.add_argument("--head_size", type=int, default=24, help="number of heads")
    parser.add_argument("--dim", type=int, default=64, help="head dim")
    parser.add_argument("--block_size", type=int, default=256)
    parser.add_argument("--sample_size", type=int, default=256)
    return parser.parse_args(argv)


def time_quantiles(fn, warmup=20, rep=100, quantiles=(0.2, 0.5, 0.8)):
    """ms per call of fn at the given quantiles; every call has its own pair of events."""
    for _ in range(warmup):
        fn()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(rep)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(rep)]
    for a, b in zip(starts, stops):
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    times = torch.tensor([a.elapsed_time(b) for a, b in zip(starts, stops)], dtype=torch.float64)
    return [float(x) for x in torch.quantile(times, torch.tensor(quantiles, dtype=torch.float64))]


def time_mode(fn, mode, warmup, rep):
    """fn: the forward, returning the attention output.  Quantiles of the forward, the backward, or their sum."""
    if mode == "fwd":
        return time_quantiles(fn, warmup, rep)
    fwd = time_quantiles(fn, warmup, rep) if mode == "fwd+bwd" else [0.0, 0.0, 0.0]
    o = fn()
    do = torch.randn_like(o)
    bwd = time_quantiles(lambda: o.backward(do, retain_graph=True), warmup, rep)
    return [a + b for a, b in zip(fwd, bwd)]


def run_flash_attn(batch_size, head_size, seq_len, dim, causal, mode="fwd", warmup=20, rep=100):
    q, k, v = (torch.randn((batch_size, seq_len, head_size, dim), dtype=torch.bfloat16, device="cuda",
                           requires_grad=mode != "fwd") for _ in range(3))
    return time_mode(lambda: flash_attn_func(q, k, v, None, causal, None)[0], mode, warmup, rep)


def run_hyper_attn(batch_size, head_size, seq_len, dim, causal, smooth_block, mode="fwd", warmup=20, rep=100,
                   block_size=256, sample_size=256):
    q, k, v = (torch.randn((batch_size, head_size, seq_len, dim), dtype=torch.bfloat16, device="cuda",
                           requires_grad=mode != "fwd") for _ in range(3))
    attn = HyperAttention(input_dim=dim, block_size=block_size, sample_size=sample_size, smooth_block=smooth_block).to(
        device="cuda", dtype=q.dtype)
    return time_mode(lambda: attn(q, k, v, causal=causal), mode, warmup, rep)


def main(argv=None):
    args = get_arguments(argv)
    for arg_name, arg_var in args.__dict__.items():
        print(f"{arg_name:<16} : {arg_var}")
    if args.attn_method == "flash-cuda":
        sys.exit("flash-cuda is a CUDA package; use --attn_method flash for this library's exact attention")

    seq_lens = [2 ** i for i in range(args.min_log2_seq, args.max_log2_seq + 1)]
    batch_size, head_size, dim = args.batch_size, args.head_size, args.dim
    print(f"mode: {args.mode}, attn_method: {args.attn_method}, batch_size: {batch_size}, head_size: {head_size}, dim: {dim}")
    causal = not args.no_causal
    for seq_len in seq_lens:
        if args.attn_method == "flash":
            ms = run_flash_attn(batch_size, head_size, seq_len, dim, causal, args.mode, rep=args.rep)
        else:
            ms = run_hyper_attn(batch_size, head_size, seq_len, dim, causal, args.smooth_block, args.mode, rep=args.rep,
                                block_size=args.block_size, sample_size=args.sample_size)
        print(f"[{args.mode:<8}], {args.attn_method}, seq_len: {seq_len:<8}, causal: {causal}, "
              f"ms: {ms[0]:.5f} ({ms[1]:.5f}, {ms[2]:.5f}) | ", flush=True)


if __name__ == "__main__":
    main()
