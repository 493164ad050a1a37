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
                launch stream, against the MI355X dense fp16/bf16 MFMA peak (`frac` = `frac_mfma`; the
                fraction of the HBM peak by its algorithmic bytes is `frac_hbm`), and against the board's
                power limit priced by the single-purpose loops of `power_roof` (`power_floor_ms`,
                `frac_power`);
  quantiles_ms  20 % / 50 % / 80 % quantiles of the forward over 100 steps, each bracketed by its own events;
  kernels       the same figures for the other kernels of the path (hash, sort: HBM; exact leaves: MFMA);
  exact_flash   our exact MFMA flash-attention forward at the same shape (the 20x comparison);
  workloads     the other single-GPU benchmark configurations (c2, c4, c5; default run only): forward ms, the
                gathered kernel's launch time and fractions, the leaves where causal, the first stage, and
                the exact kernel at the same shape;
  backward      forward under autograd + backward of the module at the same shape, and of the exact
                attention, as the reference's sweep script times them (not part of `value`);
  power_roof    board power and clock, idle and under four single-purpose loops (MFMA on registers, MFMA fed
                from LDS, the soft-max arithmetic, all of it) and a plain copy: the dynamic energy of a matrix
                flop, of a soft-max pair and of an HBM byte, separated from the idle draw;
  cpu_baseline  the CPU oracle (float32, torch) on a bounded sample of the same workload;
  cpu_baseline_c1  the CPU oracle on benchmark configuration c1 exactly (batch 1, 4 heads, seq 4096, d 64, fp32,
                non-causal): all host threads and one thread, 3 warm-ups, 10 repetitions, median; with the
                GPU forward on the same inputs (fp16) beside it;
  sustained     the forward and its kernels repeated for about a second each with board power and shader
                clock sampled from the driver's sysfs files.
"""
import argparse
import ctypes
import glob
import hashlib
import json
import os
import re
import statistics
import sys
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "HyperAttention fwd ms + MFMA util at seq 131k, 32 heads, d=64, fp16 causal"
MFMA_PEAK_TFLOPS = 2500.0   # MI355X dense fp16/bf16
HBM_PEAK_GBS = 8000.0


def kernel_source_digest():
    """sha256 (first 16 hex digits) of the attention kernels' sources: the counter summaries under profiles/
    record the digest of the sources they were measured on."""
    h = hashlib.sha256()
    try:
        for name in ("attn_fwd.hip", "attn_fwd_tile.inc", "attn_fwd_stream.inc", "attn_tiles.h"):
            h.update(open(os.path.join(ROOT, "hyperattention_amd", "csrc", name), "rb").read())
    except OSError:
        return None
    return h.hexdigest()[:16]


def quoted_traffic(workload):
    """HBM bytes per launch of the gathered attention kernel QUOTED from the counter summary committed for
    this workload (profiles/hbm_traffic_<workload>_pmc.md, line "traffic_bytes_per_launch = ..."); not
    measured in this run.  Returns (bytes, file, stale): stale is True when the summary names a kernel source
    digest ("kernel_source_sha256 = ...") other than the current one, None when it names none."""
    path = os.path.join(ROOT, "profiles", f"hbm_traffic_{workload}_pmc.md")
    try:
        text = open(path).read()
    except OSError:
        return None, None, None
    m = re.search(r"traffic_bytes_per_launch\s*=\s*([0-9.eE+]+)", text)
    if not m:
        return None, None, None
    d = re.search(r"kernel_source_sha256\s*=\s*([0-9a-f]+)", text)
    stale = None if not d else d.group(1) != kernel_source_digest()
    if stale:
        print(f"bench.py: {os.path.relpath(path, ROOT)} was measured on another version of attn_fwd.hip; "
              "roofline.traffic is stale", file=sys.stderr)
    return float(m.group(1)), os.path.relpath(path, ROOT), stale


WORKLOADS = {
    # name: batch, q heads, kv heads, n, d, dtype, causal, block, sample, min_seq_len, smooth
    "c1": dict(batch=1, heads=4, kv_heads=4, n=4096, d=64, dtype="fp16", causal=False, block=256, sample=256,
               min_seq_len=2048, smooth=False),
    "c2": dict(batch=1, heads=32, kv_heads=32, n=32768, d=64, dtype="fp16", causal=False, block=256, sample=256,
               min_seq_len=2048, smooth=False),
    "c3": dict(batch=1, heads=32, kv_heads=32, n=131072, d=64, dtype="fp16", causal=True, block=256, sample=256,
               min_seq_len=2048, smooth=False),
    "c4": dict(batch=2, heads=32, kv_heads=32, n=65536, d=128, dtype="bf16", causal=False, block=512, sample=512,
               min_seq_len=2048, smooth=True),
    "c5": dict(batch=1, heads=32, kv_heads=2, n=32768, d=128, dtype="bf16", causal=True, block=256, sample=256,
               min_seq_len=2048, smooth=False),
}


def describe(name):
    w = WORKLOADS[name]
    return (f"{name}: batch {w['batch']}, {w['heads']} heads ({w['kv_heads']} kv), seq {w['n']}, d {w['d']}, "
            f"{w['dtype']}, {'causal' if w['causal'] else 'non-causal'}, block {w['block']}, sample {w['sample']}, "
            f"min_seq_len {w['min_seq_len']}, smooth_block {w['smooth']}, 8 projections")


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
    for half in halves:
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


def time_quantiles(fn, reps, torch, quantiles=(0.2, 0.5, 0.8)):
    """ms per call of fn at the given quantiles, every call bracketed by its own pair of events (the
    protocol of the reference's sweep, benchmark_single_attention.py:31,40)."""
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    for a, b in zip(starts, stops):
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    times = sorted(a.elapsed_time(b) for a, b in zip(starts, stops))
    return [round(times[min(len(times) - 1, int(q * len(times)))], 4) for q in quantiles]


def cpu_baseline(w, seed):
    """The CPU oracle in float32 on a bounded sample: one query head (and its kv head) at full length, one
    warm-up and three timed runs (median)."""
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

    def run():
        t0 = time.perf_counter()
        O.hyper_forward(q, k, v, proj, causal=w["causal"], block_size=w["block"], sample_size=w["sample"],
                        min_seq_len=w["min_seq_len"], smooth_block=w["smooth"], dtype=torch.float32)
        return time.perf_counter() - t0

    run()
    times = sorted(run() for _ in range(3))
    dt = times[1]
    scale = w["batch"] * w["heads"] / heads_sampled * (n / n_sample)
    return {
        "value": round(dt * 1e3 * scale, 1), "unit": "ms", "cores": threads, "kind": "port",
        "sample": f"CPU oracle (torch float32, {threads} threads) on {heads_sampled} of {w['batch'] * w['heads']} "
                  f"heads at seq {n_sample}: median of 3 runs after a warm-up {dt:.2f} s, scaled x{scale:g} to the "
                  f"full workload",
        "measured_s": round(dt, 3), "runs_s": [round(x, 3) for x in times],
    }


def cpu_baseline_c1(seed):
    """Benchmark configuration c1 exactly (batch 1, 4 heads, seq 4096, d 64, fp32, non-causal, 8 projections, block 256,
    sample 256, min_seq_len 2048): the CPU oracle with all host threads and with one, 3 warm-ups, 10
    repetitions each (median, min, max), exact attention on the CPU for context, and the GPU forward on
    the same inputs cast to fp16."""
    import torch
    from oracle import hyper_oracle as O
    from hyperattention_amd import HyperAttention
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn((1, 4, 4096, 64), generator=g) for _ in range(3))
    proj = torch.randn((64, 8), generator=g)
    all_threads = torch.get_num_threads()

    def timed(fn, warm=3, reps=10):
        for _ in range(warm):
            fn()
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            ts.append((time.perf_counter() - t0) * 1e3)
        return {"median_ms": round(statistics.median(ts), 2), "min_ms": round(min(ts), 2), "max_ms": round(max(ts), 2)}

    hyper = lambda: O.hyper_forward(q, k, v, proj, causal=False, block_size=256, sample_size=256, min_seq_len=2048,
                                    dtype=torch.float32)
    exact = lambda: O.exact_attention(q, k, v, dtype=torch.float32)
    res = {"config": "c1: batch 1, 4 heads, seq 4096, d 64, fp32, non-causal, block 256, sample 256, 8 projections",
           "kind": "port", "host_cores": os.cpu_count()}
    res[f"threads_{all_threads}"] = timed(hyper)
    res[f"exact_attention_threads_{all_threads}"] = timed(exact, 1, 3)
    torch.set_num_threads(1)
    try:
        res["threads_1"] = timed(hyper)
    finally:
        torch.set_num_threads(all_threads)
    m = HyperAttention(input_dim=64, proj_dir=proj).to(device="cuda", dtype=torch.float16)
    qg, kg, vg = (x.half().cuda() for x in (q, k, v))
    ms = time_events(lambda: m(qg, kg, vg), 50, torch)
    res["gpu_fp16_ms"] = round(ms, 4)
    return res


class PowerSampler:
    """Board power (W) and shader clock (MHz) read from the amdgpu sysfs files of the first card every 20 ms
    on a background thread; empty when the files are not there or not readable."""

    def __init__(self):
        hw = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*"))
        self.hwmon = hw[0] if hw else None
        self.samples = []
        self._stop = threading.Event()
        self._thread = None

    def _read(self):
        try:
            for name in ("power1_input", "power1_average"):
                path = os.path.join(self.hwmon, name)
                if os.path.exists(path):
                    watts = int(open(path).read()) / 1e6
                    break
            else:
                return None
            sclk = None
            for line in open(os.path.join(os.path.dirname(os.path.dirname(self.hwmon)), "pp_dpm_sclk")):
                if "*" in line:
                    sclk = float(re.search(r"(\d+)\s*[Mm]hz", line).group(1))
            return watts, sclk
        except (OSError, ValueError, AttributeError):
            return None

    def cap_watts(self):
        try:
            return int(open(os.path.join(self.hwmon, "power1_cap")).read()) / 1e6
        except (OSError, ValueError, TypeError):
            return None

    def __enter__(self):
        if self.hwmon:
            def loop():
                while not self._stop.is_set():
                    r = self._read()
                    if r:
                        self.samples.append(r)
                    time.sleep(0.02)
            self._thread = threading.Thread(target=loop, daemon=True)
            self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        if self._thread:
            self._thread.join()

    def summary(self, skip_s=0.3):
        rows = self.samples[int(skip_s / 0.02):]  # the first samples still see the clock ramping
        if not rows:
            return {"power_W": None, "sclk_MHz": None, "samples": 0}
        clocks = [c for _, c in rows if c]
        return {"power_W": round(statistics.mean(p for p, _ in rows), 1),
                "sclk_MHz": round(statistics.mean(clocks), 0) if clocks else None, "samples": len(rows)}


def sustained(fn, seconds, torch, batch=20):
    """fn repeated for about `seconds`: ms per call over the whole loop, average board power and clock"""
    fn()
    torch.cuda.synchronize()
    n = 0
    with PowerSampler() as ps:
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            for _ in range(batch):
                fn()
            torch.cuda.synchronize()
            n += batch
        dt = time.perf_counter() - t0
    out = {"ms": round(dt * 1e3 / n, 4), "calls": n, "seconds": round(dt, 2)}
    out.update(ps.summary())
    out["power_cap_W"] = ps.cap_watts()
    if out["power_W"]:
        out["energy_J_per_call"] = round(out["power_W"] * dt / n, 4)
    return out


def power_roof(torch, _lib, q):
    """Idle draw, then four single-purpose loops (ha_power_probe, two workgroups of four waves per CU) and a
    plain device copy for about 0.8 s each with the board's power and clock sampled: the dynamic energy (above
    idle) of a matrix flop, of the soft-max arithmetic of one (query, key) pair and of an HBM byte."""
    L = _lib.lib()
    torch.cuda.synchronize()
    time.sleep(0.5)
    with PowerSampler() as ps:
        time.sleep(1.0)
    idle = ps.summary(0.2)
    cap = ps.cap_watts()
    if not idle["power_W"]:
        return None
    sink = torch.zeros(256, device="cuda")
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    wgs, trips = 512, 2000
    kinds = {"mfma_registers": 0, "mfma_from_lds": 1, "softmax_arithmetic": 2, "half_step_block": 3,
             "half_step_block_16_mfma": 4}
    out = {"idle": idle, "power_cap_W": cap, "loops": {}}
    for name, kind in kinds.items():
        r = sustained(lambda: _lib.check(L.ha_power_probe(kind, trips, wgs, sink.data_ptr(), st)), 0.8, torch, batch=4)
        blocks = wgs * 4 * trips * 4  # wave-blocks per launch
        r["blocks_per_launch"] = blocks
        if kind != 2:
            flops = blocks * (16 if kind == 4 else 8) * 32768
            r["TFLOPs"] = round(flops / r["ms"] / 1e9, 1)
        out["loops"][name] = r
    dst = torch.empty_like(q)
    r = sustained(lambda: dst.copy_(q), 0.8, torch)
    r["bytes_moved"] = 2 * q.numel() * q.element_size()
    r["GBs"] = round(r["bytes_moved"] / r["ms"] / 1e6, 1)
    out["loops"]["copy"] = r
    del dst
    p_idle = idle["power_W"]
    lm, ls, lc = out["loops"]["mfma_registers"], out["loops"]["softmax_arithmetic"], out["loops"]["copy"]
    out["pJ_per_flop_mfma"] = round((lm["power_W"] - p_idle) * lm["ms"] * 1e-3 / (lm["blocks_per_launch"] * 8 * 32768) * 1e12, 4)
    # a block is 16 keys x 64 queries = 1024 (query, key) pairs
    out["pJ_per_pair_softmax"] = round((ls["power_W"] - p_idle) * ls["ms"] * 1e-3 / (ls["blocks_per_launch"] * 1024) * 1e12, 3)
    out["pJ_per_byte_hbm"] = round((lc["power_W"] - p_idle) * lc["ms"] * 1e-3 / lc["bytes_moved"] * 1e12, 2)
    out["mfma_TFLOPs_under_the_limit"] = lm["TFLOPs"]
    return out


def power_floor(roof, flops, hbm_bytes, d, measured_ms):
    """Time below which the board's power limit does not let a kernel with this work go: the dynamic energy of
    its matrix flops and HBM bytes (and, second figure, of its soft-max pairs too: one per 4*d flops) over the
    power left above idle."""
    if not roof or not roof.get("power_cap_W"):
        return None
    budget = roof["power_cap_W"] - roof["idle"]["power_W"]
    e_mfma = flops * roof["pJ_per_flop_mfma"] * 1e-12
    e_hbm = hbm_bytes * roof["pJ_per_byte_hbm"] * 1e-12
    e_soft = flops / (4 * d) * roof["pJ_per_pair_softmax"] * 1e-12
    floor = (e_mfma + e_hbm) / budget * 1e3
    floor_soft = (e_mfma + e_hbm + e_soft) / budget * 1e3
    return {"power_floor_ms": round(floor, 4), "frac_power": round(floor / measured_ms, 4),
            "power_floor_with_softmax_ms": round(floor_soft, 4),
            "frac_power_with_softmax": round(floor_soft / measured_ms, 4)}


class Workload:
    """Synthetic inputs of one benchmark configuration on the GPU, its forward step and its kernels."""

    def __init__(self, name, torch, seed=1234):
        from hyperattention_amd import HyperAttention
        self.name, self.torch = name, torch
        w = self.w = WORKLOADS[name]
        self.tdt = torch.float16 if w["dtype"] == "fp16" else torch.bfloat16
        g = torch.Generator(device="cuda").manual_seed(seed)
        b, h, hk, n, d = w["batch"], w["heads"], w["kv_heads"], w["n"], w["d"]
        q = torch.randn((b, h, n, d), generator=g, device="cuda", dtype=self.tdt)
        if name == "c5":
            # clustered keys/queries: 64 unit-norm centroids x4 plus N(0, 0.5^2) noise
            cent = torch.nn.functional.normalize(torch.randn((64, d), generator=g, device="cuda"), dim=-1)
            kc = torch.randint(0, 64, (b, hk, n), generator=g, device="cuda")
            qc = torch.randint(0, 64, (b, h, n), generator=g, device="cuda")
            k = (4 * cent[kc] + 0.5 * torch.randn((b, hk, n, d), generator=g, device="cuda")).to(self.tdt)
            q = (4 * cent[qc] + 0.5 * torch.randn((b, h, n, d), generator=g, device="cuda")).to(self.tdt)
        else:
            k = torch.randn((b, hk, n, d), generator=g, device="cuda", dtype=self.tdt)
        v = torch.randn((b, hk, n, d), generator=g, device="cuda", dtype=self.tdt)
        self.q, self.k, self.v = q, k, v
        self.module = HyperAttention(input_dim=d, lsh_num_projs=8, block_size=w["block"], sample_size=w["sample"],
                                     min_seq_len=w["min_seq_len"], smooth_block=w["smooth"],
                                     rng=torch.Generator().manual_seed(seed)).to(device="cuda", dtype=self.tdt)
        self.scale = d ** -0.5
        self.proj2 = self.module.lsh.proj_dir.reshape(1, 1, d, 8)
        from hyperattention_amd import ops
        self.workspace = ops.WorkspaceCache()
        self.out = torch.zeros((b, h, n, d), device="cuda", dtype=self.tdt)
        self.lse = torch.zeros((b, h, n), device="cuda", dtype=torch.float32)

    def step(self):
        from hyperattention_amd import ops
        w = self.w
        return ops.hyper_forward(self.q, self.k, self.v, self.module.lsh.proj_dir, scale=self.scale, causal=w["causal"],
                                 lsh_num_projs=8, block_size=w["block"], sample_size=w["sample"],
                                 min_seq_len=w["min_seq_len"], smooth_block=w["smooth"], workspace=self.workspace)

    def operands(self, n_q, segs, stride, q_off):
        """ha_attn_operands of one launch over segments of the whole tensors"""
        from hyperattention_amd import _lib
        w = self.w
        b, h, hk, n, d = w["batch"], w["heads"], w["kv_heads"], w["n"], w["d"]
        t = _lib.AttnOperands()
        t.q, t.k, t.v, t.out, t.lse = (x.data_ptr() for x in (self.q, self.k, self.v, self.out, self.lse))
        t.batch, t.heads, t.n_q, t.n_k, t.d, t.dv = b, h, n_q, n_q, d, d
        t.q_stride_b, t.q_stride_h, t.q_stride_n = h * n * d, n * d, d
        t.k_stride_b, t.k_stride_h, t.k_stride_n = hk * n * d, n * d, d
        t.v_stride_b, t.v_stride_h, t.v_stride_n = hk * n * d, n * d, d
        t.o_stride_b, t.o_stride_h, t.o_stride_n = h * n * d, n * d, d
        t.lse_stride_b, t.lse_stride_h = h * n, n
        t.segs, t.seg_stride_rows, t.q_seg_offset, t.k_seg_offset = segs, stride, q_off, 0
        t.kv_group, t.scale, t.dtype = h // hk, self.scale, (0 if self.tdt == self.torch.float16 else 1)
        return t

    def level_launches(self):
        """One closure per hashed level that launches the gathered kernel exactly as the forward does (the
        orders come from the forward's own first stage), and the tensors they point to."""
        from hyperattention_amd import _lib, ops
        L = _lib.lib()
        w = self.w
        b, h, hk, n = w["batch"], w["heads"], w["kv_heads"], w["n"]
        halves, _ = levels_of(n, w["min_seq_len"], w["causal"])
        q_idx, k_idx = ops.forward_sort(self.q, self.k, self.proj2, causal=w["causal"], lsh_num_projs=8,
                                        min_seq_len=w["min_seq_len"])
        launches = []
        for j, half in enumerate(halves):
            segs = (n // (2 * half)) if w["causal"] else 1
            a = _lib.BlockAttnArgs()
            a.t = self.operands(half, segs, 2 * half if w["causal"] else n, half if w["causal"] else 0)
            a.q_idx, a.k_idx, a.sampled_idx, a.idx_type = q_idx[j].data_ptr(), k_idx[j].data_ptr(), None, 0
            a.q_idx_stride_b, a.q_idx_stride_h, a.q_idx_stride_n = h * segs * half, segs * half, 1
            a.k_idx_stride_b, a.k_idx_stride_h, a.k_idx_stride_n = hk * segs * half, segs * half, 1
            a.block_size, a.sample_size = w["block"], w["sample"]
            a.smooth_block, a.accumulate = int(w["smooth"]), int(w["causal"])
            st = ctypes.c_void_p(self.torch.cuda.current_stream().cuda_stream)
            launches.append(lambda a=a, st=st: _lib.check(L.ha_block_attn_fwd(ctypes.byref(a), st)))
        return launches, (q_idx, k_idx)

    def leaves_launch(self):
        from hyperattention_amd import _lib
        L = _lib.lib()
        w = self.w
        _, leaf = levels_of(w["n"], w["min_seq_len"], w["causal"])
        if leaf is None:
            return None
        t = self.operands(leaf, w["n"] // leaf, leaf, 0)
        st = ctypes.c_void_p(self.torch.cuda.current_stream().cuda_stream)
        return lambda: _lib.check(L.ha_flash_attn_fwd(ctypes.byref(t), 1, st))

    def gathered_work(self):
        """(flops, algorithmic HBM bytes) of one launch of the gathered kernel: Q rows, the gathered K and V
        rows of the blocks, output rows and lse, the sorted index arrays, and (causal: resumed partial result)
        the previous rows and lse; the sampled rows are shared by all query blocks of a head."""
        w = self.w
        per_level, _, _ = algorithmic_flops(w)
        lvl_q = w["batch"] * w["heads"] * (w["n"] // 2 if w["causal"] else w["n"])
        lvl_k = lvl_q * w["kv_heads"] // w["heads"]  # the query heads of a KV group share its rows
        row_b = w["d"] * 2
        nbytes = lvl_q * row_b + 2 * lvl_k * row_b + lvl_q * (row_b + 4) + (lvl_q + lvl_k) * 4
        if w["causal"]:
            nbytes += lvl_q * (row_b + 4)
        return per_level[0], nbytes


def measure_light(name, torch, steps, warmup, roof, with_exact=True):
    """Forward ms and the launch times of its kernels for one of the other benchmark configurations."""
    from hyperattention_amd import ops
    wl = Workload(name, torch)
    w = wl.w
    for _ in range(warmup):
        wl.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        wl.step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    per_level, leaf_flops, exact_flops = algorithmic_flops(w)
    res = {"config": describe(name), "ms": round(ms, 4), "steps": steps, "warmup": warmup,
           "algorithmic_TFLOPs": round((sum(per_level) + leaf_flops) / ms / 1e9, 1),
           "exact_equivalent_TFLOPs": round(exact_flops / ms / 1e9, 1)}
    reps = max(3, min(steps, 10))
    launches, keep = wl.level_launches()
    blk_ms = [time_events(fn, reps, torch) for fn in launches]
    blk_avg = sum(blk_ms) / len(blk_ms)
    flops, nbytes = wl.gathered_work()
    res["gathered_kernel"] = {"avg_launch_ms": round(blk_avg, 4), "launch_ms_by_level": [round(x, 4) for x in blk_ms],
                              "flops_per_launch": flops, "algorithmic_bytes": nbytes,
                              "achieved_TFLOPs": round(flops / blk_avg / 1e9, 1),
                              "frac_mfma": round(flops / blk_avg / 1e9 / MFMA_PEAK_TFLOPS, 4),
                              "achieved_GBs": round(nbytes / blk_avg / 1e6, 1),
                              "frac_hbm": round(nbytes / blk_avg / 1e6 / HBM_PEAK_GBS, 4)}
    pf = power_floor(roof, flops, nbytes, w["d"], blk_avg)
    if pf:
        res["gathered_kernel"].update(pf)
    leaves = wl.leaves_launch()
    if leaves:
        lms = time_events(leaves, reps, torch)
        res["leaves"] = {"ms": round(lms, 4), "flops": leaf_flops, "achieved_TFLOPs": round(leaf_flops / lms / 1e9, 1),
                         "frac_mfma": round(leaf_flops / lms / 1e9 / MFMA_PEAK_TFLOPS, 4)}
    rows_q, rows_k = w["batch"] * w["heads"] * w["n"], w["batch"] * w["kv_heads"] * w["n"]
    halves, _ = levels_of(w["n"], w["min_seq_len"], w["causal"])
    sort_elems = sum((rows_q // 2 + rows_k // 2) if w["causal"] else (rows_q + rows_k) for _ in halves)
    fs = time_events(lambda: ops.forward_sort(wl.q, wl.k, wl.proj2, causal=w["causal"], lsh_num_projs=8,
                                              min_seq_len=w["min_seq_len"]), reps, torch)
    stage_bytes = (rows_q + rows_k) * w["d"] * 2 + sort_elems * 4
    res["first_stage"] = {"ms": round(fs, 4), "bytes": stage_bytes, "achieved_GBs": round(stage_bytes / fs / 1e6, 1),
                          "frac_hbm": round(stage_bytes / fs / 1e6 / HBM_PEAK_GBS, 4)}
    if with_exact:
        qt, kt, vt = wl.q.transpose(1, 2), wl.k.transpose(1, 2), wl.v.transpose(1, 2)
        launches_exact = 2
        ems = time_events(lambda: ops.flash_attn_func(qt, kt, vt, None, w["causal"], wl.scale), launches_exact, torch)
        res["exact_flash"] = {"ms": round(ems, 3), "launches_timed": launches_exact, "flops": exact_flops,
                              "achieved_TFLOPs": round(exact_flops / ems / 1e9, 1),
                              "frac_of_mfma_peak": round(exact_flops / ems / 1e9 / MFMA_PEAK_TFLOPS, 4),
                              "speedup_of_hyper": round(ems / ms, 2)}
    del wl, launches, keep
    torch.cuda.empty_cache()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-sustained", action="store_true", help="skip the sustained loops with power sampling")
    ap.add_argument("--no-power-roof", action="store_true", help="skip the single-purpose loops that price the power limit")
    ap.add_argument("--no-exact", action="store_true", help="skip timing the exact flash kernel at the same shape")
    ap.add_argument("--no-backward", action="store_true", help="skip timing forward + backward under autograd")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="default workload only: skip the c2, c4 and c5 entries of `workloads`")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three plain device copies of Q (a kernel of known traffic, to scale HBM byte "
                         "counters collected with rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; the path shards by (batch, head) with no communication, "
              "so multi-GPU figures are not produced here (--gpus must be 1).", file=sys.stderr)
        sys.exit(2)

    import torch
    from hyperattention_amd import _lib, ops
    L = _lib.lib()
    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    torch.cuda.set_device(0)
    seed = 1234
    wl = Workload(args.workload, torch, seed)
    w, q, k, v, m = wl.w, wl.q, wl.k, wl.v, wl.module
    tdt, scale, proj2 = wl.tdt, wl.scale, wl.proj2
    b, h, hk, n, d = w["batch"], w["heads"], w["kv_heads"], w["n"], w["d"]
    step = wl.step

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
    quantiles = time_quantiles(step, 100, torch)

    roof = None
    if not args.no_power_roof:
        roof = power_roof(torch, _lib, q)

    per_level, leaf_flops, exact_flops = algorithmic_flops(w)
    algo_flops = sum(per_level) + leaf_flops

    # ---- per-kernel timing, events on the launch stream ------------------------------------------
    reps = max(3, min(args.steps, 20))
    kernels = {}
    rows_q, rows_k = b * h * n, b * hk * n
    ms = time_events(lambda: ops.lsh_hash(q, proj2), reps, torch)
    hash_bytes = rows_q * (d * 2 + 4)
    kernels["lsh_hash operator (q alone, int32 ids)"] = {"ms": round(ms, 4), "bound": "hbm", "achieved_GBs": round(hash_bytes / ms / 1e6, 1),
                              "frac": round(hash_bytes / ms / 1e6 / HBM_PEAK_GBS, 4), "bytes": hash_bytes}
    bq = ops.lsh_hash(q, proj2)
    bk = ops.lsh_hash(k, proj2)

    halves, leaf = levels_of(n, w["min_seq_len"], w["causal"])
    sort_ms = []
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
            return time_events(fn, reps, torch)

        sort_ms.append(sort_side(bq, h, half if w["causal"] else 0) + sort_side(bk, hk, 0))

    launches, keep_idx = wl.level_launches()
    blk_ms = [time_events(fn, reps, torch) for fn in launches]
    blk_launch = launches[0]
    blk_avg = sum(blk_ms) / len(blk_ms)
    blk_flops, blk_bytes = wl.gathered_work()
    achieved = blk_flops / blk_avg / 1e9  # TFLOP/s
    achieved_gbs = blk_bytes / blk_avg / 1e6
    intensity = blk_flops / blk_bytes
    ridge = MFMA_PEAK_TFLOPS * 1e12 / (HBM_PEAK_GBS * 1e9)
    traffic, traffic_source, traffic_stale = quoted_traffic(args.workload)
    roofline = {"kernel": "attn_fwd_kernel<gather> (block-diagonal + sampled attention)",
                # the metric names the MFMA utilisation: `frac` is the fraction of the dense fp16/bf16 MFMA peak
                "bound": "mfma", "achieved": round(achieved, 1), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / MFMA_PEAK_TFLOPS, 4),
                "frac_mfma": round(achieved / MFMA_PEAK_TFLOPS, 4), "achieved_TFLOPs": round(achieved, 1),
                # by its algorithmic bytes; the side the kernel's intensity puts it on is `intensity_side`
                "frac_hbm": round(achieved_gbs / HBM_PEAK_GBS, 4), "achieved_GBs": round(achieved_gbs, 1),
                "intensity_flop_per_byte": round(intensity, 1), "ridge_flop_per_byte": round(ridge, 1),
                "intensity_side": "hbm" if intensity < ridge else "mfma",
                # HBM bytes per launch QUOTED from the committed FETCH_SIZE / WRITE_SIZE counter summary of this
                # workload (fetch counter x 2.000, write counter x 1.000, factors from a plain copy of known
                # size); not measured in this run
                "traffic": traffic, "traffic_source": traffic_source,
                "traffic_kind": "quoted from the committed rocprofv3 --pmc summary, not measured in this run",
                "traffic_stale": traffic_stale,
                "algorithmic_bytes": blk_bytes,
                "flops_per_launch": blk_flops, "avg_launch_ms": round(blk_avg, 4),
                "launch_ms_by_level": [round(x, 4) for x in blk_ms]}
    pf = power_floor(roof, blk_flops, blk_bytes, d, blk_avg)
    if pf:
        roofline.update(pf)
    sort_elems = sum((rows_q // 2 + rows_k // 2) if w["causal"] else (rows_q + rows_k) for _ in halves)
    sort_total = sum(sort_ms)
    kernels["bucket_argsort operator (one call per level and side; the forward ranks once instead)"] = {"ms": round(sort_total, 4), "bound": "hbm", "bytes": sort_elems * 8,
                                             "achieved_GBs": round(sort_elems * 8 / sort_total / 1e6, 1),
                                             "frac": round(sort_elems * 8 / sort_total / 1e6 / HBM_PEAK_GBS, 4)}
    # the first stage of the one-call forward: bucket ids of q and k in one launch, one ranking of the rows,
    # one placement launch for all levels.  Algorithmic bytes: q and k read once, the orders written once.
    ms = time_events(lambda: ops.forward_sort(q, k, proj2, causal=w["causal"], lsh_num_projs=8,
                                              min_seq_len=w["min_seq_len"]), reps, torch)
    stage_bytes = (rows_q + rows_k) * d * 2 + sort_elems * 4
    kernels["first stage of the forward: hash q+k in one launch, rank once, place all levels (ha_forward_sort)"] = {
        "ms": round(ms, 4), "bound": "hbm", "bytes": stage_bytes, "achieved_GBs": round(stage_bytes / ms / 1e6, 1),
        "frac": round(stage_bytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
    leaves = wl.leaves_launch()
    if leaves is not None:
        ms = time_events(leaves, reps, torch)
        leaf_bytes = rows_q * (2 * d * 2 + 4) + 2 * rows_k * d * 2
        kernels["flash leaves (exact causal)"] = {"ms": round(ms, 4), "bound": "mfma", "flops": leaf_flops,
                                                  "achieved_TFLOPs": round(leaf_flops / ms / 1e9, 1),
                                                  "frac": round(leaf_flops / ms / 1e9 / MFMA_PEAK_TFLOPS, 4)}
        pf = power_floor(roof, leaf_flops, leaf_bytes, d, ms)
        if pf:
            kernels["flash leaves (exact causal)"].update(pf)

        if w["causal"] and not args.no_exact:
            # what a workgroup of the exact causal kernel costs beyond its key chunks: the same rows cut into
            # segments of other lengths (a workgroup takes a pair of 256-query tiles (s, T-1-s): 4 (T + 1) chunks
            # of 64 keys), per-workgroup time = launch time / rounds of workgroups per CU slot, fitted as
            # a * chunks + c.  c is the fixed cost of a pair of tiles (query rows, first tiles, two epilogues),
            # which is what separates the leaves from the same kernel on one long sequence
            slots = 256 * (2 if d == 64 else 1)
            pts, by_len = [], {}
            for seg_len in (1024, 2048, 4096, 8192, 16384):
                if seg_len > n or n % seg_len:
                    continue
                t_seg = wl.operands(seg_len, n // seg_len, seg_len, 0)
                st_seg = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
                ms_seg = time_events(lambda: _lib.check(L.ha_flash_attn_fwd(ctypes.byref(t_seg), 1, st_seg)), 3, torch)
                tiles = seg_len // 256
                wgs = b * h * (n // seg_len) * ((tiles + 1) // 2)
                chunks = 4 * (tiles + 1)
                pts.append((chunks, ms_seg * 1e3 / (wgs / slots)))
                seg_flops = b * h * (n // seg_len) * seg_len * seg_len // 2 * 4 * d
                by_len[str(seg_len)] = {"ms": round(ms_seg, 4), "chunks_per_workgroup": chunks,
                                        "frac": round(seg_flops / ms_seg / 1e9 / MFMA_PEAK_TFLOPS, 4)}
            if len(pts) >= 3:
                mx, my = sum(x for x, _ in pts) / len(pts), sum(y for _, y in pts) / len(pts)
                slope = sum((x - mx) * (y - my) for x, y in pts) / sum((x - mx) ** 2 for x, _ in pts)
                kernels["flash leaves (exact causal)"]["by_segment_length"] = {
                    "segments": by_len, "us_per_chunk": round(slope, 3), "us_per_pair_of_tiles": round(my - slope * mx, 2),
                    "note": "least-squares line through (chunks per workgroup, launch time / workgroup rounds per CU slot)"}

    # the operator-level kernels that the one-call forward does not launch (row gather of the reference's
    # `indexing`, merge of two partial attentions), at this workload's tensor size
    perm = torch.argsort(bq.view(b, h, n), dim=2)
    ms = time_events(lambda: ops.indexing(q, perm), reps, torch)
    g_bytes = rows_q * (2 * d * 2 + 8)
    kernels["gather_rows (indexing, bucket-sorted order)"] = {
        "ms": round(ms, 4), "bound": "hbm", "bytes": g_bytes, "achieved_GBs": round(g_bytes / ms / 1e6, 1),
        "frac": round(g_bytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
    lse4 = wl.lse.unsqueeze(-1)
    ms = time_events(lambda: ops.add_self_attentions(q, lse4, wl.out, lse4), reps, torch)
    m_bytes = rows_q * (3 * d * 2 + 12)
    kernels["lse_merge (add_self_attentions)"] = {
        "ms": round(ms, 4), "bound": "hbm", "bytes": m_bytes, "achieved_GBs": round(m_bytes / ms / 1e6, 1),
        "frac": round(m_bytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
    del perm

    exact = None
    qt, kt, vt = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
    if not args.no_exact:
        ms = time_events(lambda: ops.flash_attn_func(qt, kt, vt, None, w["causal"], scale), 2, torch)
        exact = {"ms": round(ms, 3), "flops": exact_flops, "achieved_TFLOPs": round(exact_flops / ms / 1e9, 1),
                 "frac_of_mfma_peak": round(exact_flops / ms / 1e9 / MFMA_PEAK_TFLOPS, 4),
                 "speedup_of_hyper": round(ms / ms_per_step, 2)}
        pf = power_floor(roof, exact_flops, 4 * rows_q * d * 2, d, ms)
        if pf:
            exact.update(pf)

    backward = None
    if not args.no_backward:
        def fwd_bwd_ms(fn, tensors, reps, sustain=False):
            """(ms of the forward under autograd, ms of the backward), each the mean over reps calls"""
            leaves_ = [x.detach().clone().requires_grad_() for x in tensors]
            o = fn(*leaves_)
            do = torch.randn_like(o)
            o.backward(do)
            f = time_events(lambda: fn(*leaves_), reps, torch)
            o = fn(*leaves_)
            bw = time_events(lambda: o.backward(do, retain_graph=True), reps, torch)
            power = None
            if sustain:
                # the backward alone for a second, with board power and shader clock (gradients accumulate into
                # the leaves, as in the timed calls)
                power = sustained(lambda: o.backward(do, retain_graph=True), 1.0, torch)
            return f, bw, power

        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        held = torch.cuda.memory_allocated()
        f_ms, b_ms, b_power = fwd_bwd_ms(lambda a, b_, c: m(a, b_, c, causal=w["causal"]), (q, k, v), 5,
                                         sustain=not args.no_sustained)
        backward = {"fwd_autograd_ms": round(f_ms, 3), "bwd_ms": round(b_ms, 3), "fwd_bwd_ms": round(f_ms + b_ms, 3),
                    # device memory the forward + backward of the module took on top of what was held before
                    # (inputs and the bench's own tensors), and the size of q, k, v together for comparison
                    "peak_extra_memory_GB": round((torch.cuda.max_memory_allocated() - held) / 1e9, 3),
                    "qkv_GB": round(sum(x.numel() * x.element_size() for x in (q, k, v)) / 1e9, 3)}
        if b_power:
            backward["sustained"] = b_power
        if not args.no_exact and hk == h:
            ef, eb, _ = fwd_bwd_ms(lambda a, b_, c: ops.flash_attn_func(a.transpose(1, 2), b_.transpose(1, 2), c.transpose(1, 2),
                                                                    None, w["causal"], scale)[0], (q, k, v), 2)
            backward["exact_fwd_bwd_ms"] = round(ef + eb, 3)
            backward["speedup_of_hyper"] = round((ef + eb) / (f_ms + b_ms), 2)
        torch.cuda.empty_cache()

    result = {
        "metric": METRIC if args.workload == "c3" else f"HyperAttention fwd ms ({args.workload})",
        "value": round(ms_per_step, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": w["dtype"], "data": "synthetic",
        "config": {"workload": describe(args.workload), "seed": seed},
        "quantiles_ms": {"q20": quantiles[0], "q50": quantiles[1], "q80": quantiles[2], "steps": 100,
                         "protocol": "every step bracketed by its own pair of events on the launch stream"},
        "algorithmic_TFLOPs": round(algo_flops / ms_per_step / 1e9, 1),
        "exact_equivalent_TFLOPs": round(exact_flops / ms_per_step / 1e9, 1),
        "roofline": roofline, "kernels": kernels, "exact_flash": exact, "backward": backward,
        "power_roof": roof,
    }
    if not args.no_sustained:
        # every kernel of the path (and a plain copy, and the exact kernel) on its own for about a second: the
        # board's power and the clock it holds under each of them
        sus = {"forward": sustained(step, 1.5, torch), "roofline_kernel": sustained(blk_launch, 1.0, torch)}
        sus["lsh_hash"] = sustained(lambda: ops.lsh_hash(q, proj2), 0.7, torch)
        if leaves is not None:
            sus["leaves"] = sustained(leaves, 0.7, torch)
        dst = torch.empty_like(q)
        sus["copy_of_q"] = sustained(lambda: dst.copy_(q), 0.7, torch)
        sus["copy_of_q"]["bytes_moved"] = 2 * q.numel() * q.element_size()
        del dst
        if not args.no_exact:
            sus["exact_flash"] = sustained(lambda: ops.flash_attn_func(qt, kt, vt, None, w["causal"], scale), 1.0, torch,
                                           batch=2)
        result["sustained"] = sus
    if args.workload == "c3" and not args.no_other_workloads:
        # the other single-GPU benchmark configurations, lighter: the tensors of this one are released first
        del wl, q, k, v, m, qt, kt, vt, launches, keep_idx, blk_launch, leaves, step, bq, bk, lse4
        torch.cuda.empty_cache()
        result["workloads"] = {name: measure_light(name, torch, 10, 3, roof) for name in ("c2", "c4", "c5")}
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(w, seed)
        result["cpu_baseline_c1"] = cpu_baseline_c1(seed)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
