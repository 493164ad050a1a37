#!/usr/bin/env python3
"""Benchmark of the HyperAttention forward path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c2|c4|c5]

A step is one forward pass over one batch of synthetic input already resident in HBM.  The default
workload is the configuration the headline metric is quoted on (benchmark configuration c3): batch 1,
32 heads, seq 131072, head dim 64, fp16, causal, 8 projections, block 256, sample 256,
min_seq_len 2048.  Prints one JSON line (see the keys below).

Besides the whole-forward time the line carries
  roofline      the dominant kernel (gathered block-diagonal + sampled attention), its algorithmic
                flops per launch over its average launch time measured here with events on the
                launch stream, against the MI355X dense fp16/bf16 MFMA peak;
  kernels       the same figure for the other kernels of the path (hash, sort: HBM; exact leaves: MFMA);
  exact_flash   our exact MFMA flash-attention forward at the same shape (the 20x comparison);
  backward      forward under autograd + backward of the module at the same shape, and of the exact
                attention, as the reference's sweep script times them (not part of `value`);
  cpu_baseline  the CPU oracle (float32, torch) on a bounded sample of the same workload.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "HyperAttention fwd ms + MFMA util at seq 131k, 32 heads, d=64, fp16 causal"
MFMA_PEAK_TFLOPS = 2500.0   # MI355X dense fp16/bf16
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the gathered attention kernel, measured with rocprofv3 --pmc (see the
# summary of that run under profiles/); only the workload that was measured has a figure
MEASURED_TRAFFIC_BYTES = {"c3": 1.3903e9}

WORKLOADS = {
    # name: batch, q heads, kv heads, n, d, dtype, causal, block, sample, min_seq_len, smooth
    "c2": dict(batch=1, heads=32, kv_heads=32, n=32768, d=64, dtype="fp16", causal=False, block=256, sample=256,
               min_seq_len=2048, smooth=False),
    "c3": dict(batch=1, heads=32, kv_heads=32, n=131072, d=64, dtype="fp16", causal=True, block=256, sample=256,
               min_seq_len=2048, smooth=False),
    "c4": dict(batch=2, heads=32, kv_heads=32, n=65536, d=128, dtype="bf16", causal=False, block=512, sample=512,
               min_seq_len=2048, smooth=True),
    "c5": dict(batch=1, heads=32, kv_heads=2, n=32768, d=128, dtype="bf16", causal=True, block=256, sample=256,
               min_seq_len=2048, smooth=False),
}


def levels_of(n, min_seq_len, causal):
    """(hashed off-diagonal half lengths per level, leaf length) of the causal recursion."""
    if not causal:
        return [n], None
    halves = []
    while n > min_seq_len:
        n //= 2
        if not (min_seq_len > n):
            halves.append(n)
    return halves, n


def algorithmic_flops(w):
    """Flops of one forward: 4*d per (query, key) pair actually visited."""
    rows = w["batch"] * w["heads"]
    halves, leaf = levels_of(w["n"], w["min_seq_len"], w["causal"])
    per_level = []
    for i, half in enumerate(halves):
        q_rows = rows * (w["n"] // 2 if w["causal"] else w["n"])
        per_level.append(q_rows * 4 * w["d"] * (w["block"] + w["sample"]))
    leaf_flops = 0
    if leaf is not None:
        leaf_flops = rows * (w["n"] // leaf) * 4 * w["d"] * leaf * (leaf + 1) // 2
    exact = rows * 4 * w["d"] * (w["n"] * (w["n"] + 1) // 2 if w["causal"] else w["n"] * w["n"])
    return per_level, leaf_flops, exact


def time_events(fn, reps, torch):
    """Average ms per call of fn, bracketed by events on the current (launch) stream."""
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    fn()
    torch.cuda.synchronize()
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / reps


def cpu_baseline(w, seed):
    """The CPU oracle in float32 on a bounded sample: one query head (and its kv head) at full length."""
    import torch
    from oracle import hyper_oracle as O
    g = torch.Generator().manual_seed(seed)
    n = w["n"]
    heads_sampled = 1
    n_sample = n
    # keep the sample to roughly 10-30 s of CPU work: shorten the sequence for the wide-head shapes
    if w["d"] * n > 64 * 131072:
        n_sample = n // 2
    tdt = torch.float16 if w["dtype"] == "fp16" else torch.bfloat16
    q, k, v = (torch.randn((1, heads_sampled, n_sample, w["d"]), generator=g).to(tdt).float() for _ in range(3))
    proj = torch.randn((w["d"], 8), generator=g).to(tdt).float()
    threads = torch.get_num_threads()
    t0 = time.perf_counter()
    O.hyper_forward(q, k, v, proj, causal=w["causal"], block_size=w["block"], sample_size=w["sample"],
                    min_seq_len=w["min_seq_len"], smooth_block=w["smooth"], dtype=torch.float32)
    dt = time.perf_counter() - t0
    scale = w["batch"] * w["heads"] / heads_sampled * (n / n_sample)
    return {
        "value": round(dt * 1e3 * scale, 1), "unit": "ms", "cores": threads, "kind": "port",
        "sample": f"CPU oracle (torch float32, {threads} threads) on {heads_sampled} of {w['batch'] * w['heads']} "
                  f"heads at seq {n_sample}: {dt:.2f} s measured, scaled x{scale:g} to the full workload",
        "measured_s": round(dt, 3),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-exact", action="store_true", help="skip timing the exact flash kernel at the same shape")
    ap.add_argument("--no-backward", action="store_true", help="skip timing forward + backward under autograd")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three plain device copies of Q (a kernel of known traffic, to scale HBM byte "
                         "counters collected with rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; the path shards by (batch, head) with no communication, "
              "so multi-GPU figures are not produced here (--gpus must be 1).", file=sys.stderr)
        sys.exit(2)

    import torch
    from hyperattention_amd import HyperAttention, _lib, ops
    L = _lib.lib()
    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    torch.cuda.set_device(0)
    w = WORKLOADS[args.workload]
    tdt = torch.float16 if w["dtype"] == "fp16" else torch.bfloat16
    seed = 1234
    g = torch.Generator(device="cuda").manual_seed(seed)
    b, h, hk, n, d = w["batch"], w["heads"], w["kv_heads"], w["n"], w["d"]
    q = torch.randn((b, h, n, d), generator=g, device="cuda", dtype=tdt)
    if args.workload == "c5":
        # clustered keys/queries: 64 unit-norm centroids x4 plus N(0, 0.5^2) noise
        cent = torch.nn.functional.normalize(torch.randn((64, d), generator=g, device="cuda"), dim=-1)
        kc = torch.randint(0, 64, (b, hk, n), generator=g, device="cuda")
        qc = torch.randint(0, 64, (b, h, n), generator=g, device="cuda")
        k = (4 * cent[kc] + 0.5 * torch.randn((b, hk, n, d), generator=g, device="cuda")).to(tdt)
        q = (4 * cent[qc] + 0.5 * torch.randn((b, h, n, d), generator=g, device="cuda")).to(tdt)
    else:
        k = torch.randn((b, hk, n, d), generator=g, device="cuda", dtype=tdt)
    v = torch.randn((b, hk, n, d), generator=g, device="cuda", dtype=tdt)
    m = HyperAttention(input_dim=d, lsh_num_projs=8, block_size=w["block"], sample_size=w["sample"],
                       min_seq_len=w["min_seq_len"], smooth_block=w["smooth"],
                       rng=torch.Generator().manual_seed(seed)).to(device="cuda", dtype=tdt)
    scale = d ** -0.5

    def step():
        return ops.hyper_forward(q, k, v, m.lsh.proj_dir, scale=scale, causal=w["causal"], lsh_num_projs=8,
                                 block_size=w["block"], sample_size=w["sample"], min_seq_len=w["min_seq_len"],
                                 smooth_block=w["smooth"])

    if args.calibrate_copy:
        dst = torch.empty_like(q)
        for _ in range(3):
            dst.copy_(q)
        torch.cuda.synchronize()
        del dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    per_level, leaf_flops, exact_flops = algorithmic_flops(w)
    algo_flops = sum(per_level) + leaf_flops

    # ---- per-kernel timing, events on the launch stream ------------------------------------------
    reps = max(3, min(args.steps, 20))
    kernels = {}
    rows_q, rows_k = b * h * n, b * hk * n
    proj2 = m.lsh.proj_dir.reshape(1, 1, d, 8)
    ms = time_events(lambda: ops.lsh_hash(q, proj2), reps, torch)
    hash_bytes = rows_q * (d * 2 + 4)
    kernels["lsh_hash(q)"] = {"ms": round(ms, 4), "bound": "hbm", "achieved_GBs": round(hash_bytes / ms / 1e6, 1),
                              "frac": round(hash_bytes / ms / 1e6 / HBM_PEAK_GBS, 4), "bytes": hash_bytes}
    bq = ops.lsh_hash(q, proj2)
    bk = ops.lsh_hash(k, proj2)

    halves, leaf = levels_of(n, w["min_seq_len"], w["causal"])
    blk_ms, sort_ms = [], []
    out = torch.zeros((b, h, n, d), device="cuda", dtype=tdt)
    lse = torch.zeros((b, h, n), device="cuda", dtype=torch.float32)
    for j, half in enumerate(halves):
        segs = (n // (2 * half)) if w["causal"] else 1
        stride = 2 * half if w["causal"] else n

        def sort_side(keys, nheads, offset):
            nseg = b * nheads * segs
            idx = torch.empty((nseg, half), device="cuda", dtype=torch.int32)
            ws_bytes = L.ha_bucket_argsort_workspace_bytes(nseg, half, 256)
            ws = torch.empty(max(int(ws_bytes), 256), device="cuda", dtype=torch.uint8)
            st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            fn = lambda: _lib.check(L.ha_bucket_argsort(keys.data_ptr(), idx.data_ptr(), 0, nseg, half, stride, offset,
                                                        256, ws.data_ptr(), ws.numel(), st))
            return idx, time_events(fn, reps, torch)

        qi, t1 = sort_side(bq, h, half if w["causal"] else 0)
        ki, t2 = sort_side(bk, hk, 0)
        sort_ms.append(t1 + t2)

        a = _lib.BlockAttnArgs()
        t = a.t
        t.q, t.k, t.v, t.out, t.lse = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr()
        t.batch, t.heads, t.n_q, t.n_k, t.d, t.dv = b, h, half, half, d, d
        t.q_stride_b, t.q_stride_h, t.q_stride_n = h * n * d, n * d, d
        t.k_stride_b, t.k_stride_h, t.k_stride_n = hk * n * d, n * d, d
        t.v_stride_b, t.v_stride_h, t.v_stride_n = hk * n * d, n * d, d
        t.o_stride_b, t.o_stride_h, t.o_stride_n = h * n * d, n * d, d
        t.lse_stride_b, t.lse_stride_h = h * n, n
        t.segs, t.seg_stride_rows = segs, stride
        t.q_seg_offset, t.k_seg_offset = (half if w["causal"] else 0), 0
        t.kv_group, t.scale, t.dtype = h // hk, scale, (0 if tdt == torch.float16 else 1)
        a.q_idx, a.k_idx, a.sampled_idx, a.idx_type = qi.data_ptr(), ki.data_ptr(), None, 0
        a.q_idx_stride_b, a.q_idx_stride_h, a.q_idx_stride_n = h * segs * half, segs * half, 1
        a.k_idx_stride_b, a.k_idx_stride_h, a.k_idx_stride_n = hk * segs * half, segs * half, 1
        a.block_size, a.sample_size = w["block"], w["sample"]
        a.smooth_block, a.accumulate = int(w["smooth"]), int(w["causal"])
        st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        blk_ms.append(time_events(lambda: _lib.check(L.ha_block_attn_fwd(ctypes.byref(a), st)), reps, torch))

    blk_avg = sum(blk_ms) / len(blk_ms)
    blk_flops = per_level[0]
    # algorithmic HBM bytes of one launch: Q rows, the gathered K and V rows of the blocks, output rows and
    # lse, the sorted index arrays, and (causal: resumed partial result) the previous rows and lse; the
    # sampled rows are shared by all query blocks of a head
    lvl_q = b * h * (n // 2 if w["causal"] else n)
    lvl_k = lvl_q  # one key block per query block
    row_b = d * 2
    blk_bytes = lvl_q * row_b + 2 * lvl_k * row_b + lvl_q * (row_b + 4) + (lvl_q + lvl_k) * 4
    if w["causal"]:
        blk_bytes += lvl_q * (row_b + 4)
    achieved = blk_flops / blk_avg / 1e9  # TFLOP/s
    roofline = {"kernel": "attn_fwd_kernel<gather> (block-diagonal + sampled attention)", "bound": "mfma",
                "achieved": round(achieved, 1), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / MFMA_PEAK_TFLOPS, 4),
                # HBM bytes per launch from the FETCH_SIZE / WRITE_SIZE counter runs of this workload
                # (fetch counter x 2.000, write counter x 1.000, factors from a plain copy of known size)
                "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload),
                "algorithmic_bytes": blk_bytes,
                "flops_per_launch": blk_flops, "avg_launch_ms": round(blk_avg, 4),
                "launch_ms_by_level": [round(x, 4) for x in blk_ms]}
    sort_elems = sum((rows_q // 2 + rows_k // 2) if w["causal"] else (rows_q + rows_k) for _ in halves)
    sort_total = sum(sort_ms)
    kernels["bucket_argsort(one launch per level and side)"] = {"ms": round(sort_total, 4), "bound": "hbm", "bytes": sort_elems * 8,
                                             "achieved_GBs": round(sort_elems * 8 / sort_total / 1e6, 1),
                                             "frac": round(sort_elems * 8 / sort_total / 1e6 / HBM_PEAK_GBS, 4)}
    if leaf is not None:
        def leaves():
            t = _lib.AttnOperands()
            t.q, t.k, t.v, t.out, t.lse = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr()
            t.batch, t.heads, t.n_q, t.n_k, t.d, t.dv = b, h, leaf, leaf, d, d
            t.q_stride_b, t.q_stride_h, t.q_stride_n = h * n * d, n * d, d
            t.k_stride_b, t.k_stride_h, t.k_stride_n = hk * n * d, n * d, d
            t.v_stride_b, t.v_stride_h, t.v_stride_n = hk * n * d, n * d, d
            t.o_stride_b, t.o_stride_h, t.o_stride_n = h * n * d, n * d, d
            t.lse_stride_b, t.lse_stride_h = h * n, n
            t.segs, t.seg_stride_rows, t.q_seg_offset, t.k_seg_offset = n // leaf, leaf, 0, 0
            t.kv_group, t.scale, t.dtype = h // hk, scale, (0 if tdt == torch.float16 else 1)
            st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            _lib.check(L.ha_flash_attn_fwd(ctypes.byref(t), 1, st))
        ms = time_events(leaves, reps, torch)
        kernels["flash leaves (exact causal)"] = {"ms": round(ms, 4), "bound": "mfma", "flops": leaf_flops,
                                                  "achieved_TFLOPs": round(leaf_flops / ms / 1e9, 1),
                                                  "frac": round(leaf_flops / ms / 1e9 / MFMA_PEAK_TFLOPS, 4)}

    exact = None
    if not args.no_exact and hk == h:
        qt, kt, vt = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
        ms = time_events(lambda: ops.flash_attn_func(qt, kt, vt, None, w["causal"], scale), 2, torch)
        exact = {"ms": round(ms, 3), "flops": exact_flops, "achieved_TFLOPs": round(exact_flops / ms / 1e9, 1),
                 "frac_of_mfma_peak": round(exact_flops / ms / 1e9 / MFMA_PEAK_TFLOPS, 4),
                 "speedup_of_hyper": round(ms / ms_per_step, 2)}

    backward = None
    if not args.no_backward:
        def fwd_bwd_ms(fn, tensors, reps):
            """(ms of the forward under autograd, ms of the backward), each the mean over reps calls"""
            leaves = [x.detach().clone().requires_grad_() for x in tensors]
            o = fn(*leaves)
            do = torch.randn_like(o)
            o.backward(do)
            f = time_events(lambda: fn(*leaves), reps, torch)
            o = fn(*leaves)
            bw = time_events(lambda: o.backward(do, retain_graph=True), reps, torch)
            return f, bw

        f_ms, b_ms = fwd_bwd_ms(lambda a, b_, c: m(a, b_, c, causal=w["causal"]), (q, k, v), 5)
        backward = {"fwd_autograd_ms": round(f_ms, 3), "bwd_ms": round(b_ms, 3), "fwd_bwd_ms": round(f_ms + b_ms, 3)}
        if not args.no_exact and hk == h:
            ef, eb = fwd_bwd_ms(lambda a, b_, c: ops.flash_attn_func(a.transpose(1, 2), b_.transpose(1, 2), c.transpose(1, 2),
                                                                    None, w["causal"], scale)[0], (q, k, v), 2)
            backward["exact_fwd_bwd_ms"] = round(ef + eb, 3)
            backward["speedup_of_hyper"] = round((ef + eb) / (f_ms + b_ms), 2)
        torch.cuda.empty_cache()

    result = {
        "metric": METRIC if args.workload == "c3" else f"HyperAttention fwd ms ({args.workload})",
        "value": round(ms_per_step, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": w["dtype"], "data": "synthetic",
        "config": {"workload": f"{args.workload}: batch {b}, {h} heads ({hk} kv), seq {n}, d {d}, {w['dtype']}, "
                               f"{'causal' if w['causal'] else 'non-causal'}, block {w['block']}, sample {w['sample']}, "
                               f"min_seq_len {w['min_seq_len']}, smooth_block {w['smooth']}, 8 projections",
                   "seed": seed},
        "algorithmic_TFLOPs": round(algo_flops / ms_per_step / 1e9, 1),
        "exact_equivalent_TFLOPs": round(exact_flops / ms_per_step / 1e9, 1),
        "roofline": roofline, "kernels": kernels, "exact_flash": exact, "backward": backward,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(w, seed)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
