#!/usr/bin/env python3
"""Benchmark of the paged KV-cache attention path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config all|c2|c2_8k|c3a|c3b|c4|c5|mixed] [--no-cpu]

A step is one call of the hot path (append + rotary + attention + split combine for the decode
configs, one varlen forward for c5) on synthetic inputs that are resident in HBM before the
timed region.  Several input sets (distinct physical pools) are rotated so that no step finds its K/V in the
256 MB last-level cache: as many as it takes for one rotation to read 512 MB.  Prints ONE JSON line: whole-call throughput (`value`, K steps between two device
synchronisations after W untimed ones; without --warmup, at least 10 calls and at least 0.1 s of them, which is
what the device's clocks take to settle), the median of the per-call durations taken with HIP events in the same
pass (an event every K/10 calls for the decode configs, where one between every two calls would cost each call
≈ 3 µs), the roofline record of
the dominant kernel (its duration measured with HIP events the library records around it on the
launch stream) and the CPU golden path timed on the host cores of this box.  The default (`all`) is
the headline config c2 plus a `configs` object with the same measurements, on the same K, for
every other configuration of the baseline (c2_8k, c3a, c3b, c4, c5), each with a short CPU sample.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (os.path.join(ROOT, "flash-attention-npu_amd"), os.path.join(ROOT, "oracle"), os.path.join(ROOT, "tests")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
COLD_BYTES = 512 << 20      # bytes the rotated pools of a decode config must add up to: twice the last-level cache

# HBM bytes per launch of the dominant kernel are not something a timing run can see: they come from the
# FETCH_SIZE / WRITE_SIZE counter passes whose summaries are tracked under profiles/ (a line
# "traffic_bytes_per_launch: N" in the summary of that kernel and workload).  The workloads are seeded, so the
# figure belongs to the kernel as it was when the summary was made; the record names the file it was read from.
PROFILE_OF = {"c2": "decode_wave_kernel_c2.txt", "c2_8k": "decode_wave_kernel_c2_8k.txt", "c3a": "decode_wave_kernel_c3a.txt", "c3b": "decode_wave_kernel_c3b.txt",
              "c4": "decode_mla_i8_kernel_c4.txt", "c5": "prefill_kernel_c5.txt",
              "mqa32": "prefill_kernel_mqa32.txt", "mqa32_d256": "prefill_kernel_mqa32_d256.txt",
              "g32k8": "decode_wave_kernel_g32k8.txt"}


def traffic_from_profile(name: str):
    """(bytes, file) of the counter-measured HBM traffic per launch for config `name`, or (None, None)."""
    fn = PROFILE_OF.get(name)
    path = os.path.join(ROOT, "profiles", fn) if fn else None
    if not path or not os.path.exists(path):
        return None, None
    for line in open(path):
        if line.startswith("traffic_bytes_per_launch:"):
            try:
                return float(line.split(":", 1)[1].split()[0]), "profiles/" + fn
            except ValueError:
                return None, None
    return None, None


def median(xs):
    xs = sorted(xs)
    n = len(xs)
    return xs[n // 2] if n % 2 else 0.5 * (xs[n // 2 - 1] + xs[n // 2])


# ----------------------------------------------------------------------------- HIP events
class HipEvents:
    """hipEvent_t handles created through the HIP runtime the process already has loaded."""

    def __init__(self, n: int):
        self.hip = C.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        self.hip.hipEventDestroy.argtypes = [C.c_void_p]
        self.hip.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        self.ev = (C.c_void_p * n)()
        for i in range(n):
            e = C.c_void_p()
            rc = self.hip.hipEventCreate(C.byref(e))
            if rc != 0:
                raise RuntimeError(f"hipEventCreate failed: {rc}")
            self.ev[i] = e

    def group(self, i: int, width: int = 4):
        return C.cast(C.byref(self.ev, i * width * C.sizeof(C.c_void_p)), C.POINTER(C.c_void_p))

    def elapsed_ms(self, a: int, b: int) -> float:
        ms = C.c_float()
        rc = self.hip.hipEventElapsedTime(C.byref(ms), self.ev[a], self.ev[b])
        if rc != 0:
            raise RuntimeError(f"hipEventElapsedTime failed: {rc}")
        return ms.value

    def record(self, i: int, stream) -> None:
        self.hip.hipEventRecord(self.ev[i], stream)

    def close(self):
        for e in self.ev:
            self.hip.hipEventDestroy(e)


# ----------------------------------------------------------------------------- workloads
def decode_workload(name: str, device, seed: int = 0, kv_layout: str = "nhd"):
    """Synthetic inputs of the decode configs (BASELINE.json configs[1..3]); returns a dict."""
    import torch
    g = torch.Generator(device="cpu").manual_seed(seed)
    page = 256
    if name in ("c2", "c2_8k") or name.startswith("c2_u"):
        B, hq, hk, d = 64, 32, 8, 128
        if name.startswith("c2_u"):
            lens = torch.full((B,), int(name[4:]))      # c2_u<len>: every row the same length (scaling probe)
        elif name == "c2":
            # uniform in [1024, 8191]: the appended key sits at position len <= 8191 < seqlen_ro
            lens = torch.randint(1024, 8192, (B,), generator=g)
        else:
            lens = torch.full((B,), 8191)
        snew, rotary, window, spare = 1, True, (-1, -1), 64
        desc = ("Llama-3-8B bf16 paged decode B=64 32q/8kv d=128 page=256 "
                + ("lens U[1024,8191]" if name == "c2" else "all rows 8191 keys") + " append+RoPE causal")
    elif name in ("c3a", "c3b"):
        B, hq, hk, d = 4, 64, 8, 128
        lens = torch.full((B,), 131072)
        snew, rotary, spare = 0, False, 0
        window = (-1, -1) if name == "c3a" else (4095, 0)
        desc = f"long-context split-KV decode bf16 B=4 64q/8kv d=128 Lk=131072 window={window} causal"
    elif name in ("mqa32", "mqa32_d256", "mqa32_d64", "g32k8", "g32k8_d64", "g32k8_d256", "g64k8", "g48k8", "g32k4", "g32k2"):
        # query blocks of 17..32 rows (one token x 32 q heads of one kv head): past the 16 rows of one decode tile;
        # mqa32*: one kv head; g32k8*: eight kv heads of 32 q heads each; the suffix _d<n> sets the head dimension
        B, hq, hk, d = 64, 32, 1, (128 if name in ("mqa32", "g32k8", "g64k8", "g48k8", "g32k4", "g32k2") else int(name[7:]))
        if name in ("g32k4", "g32k2"):
            hk = int(name[4:])
            hq = 32 * hk
        if name.startswith("g32k8"):
            hq, hk = 256, 8
        if name in ("g64k8", "g48k8"):
            hq, hk = 8 * int(name[1:3]), 8
        lens = torch.full((B,), 8192)
        snew, rotary, window, spare = 0, False, (-1, -1), 16
        desc = f"paged decode bf16 B=64 {hq}q/{hk}kv d={d} page=256 all rows 8192 keys causal (32-row query blocks)"
    else:
        raise ValueError(name)
    pages = [math.ceil((int(l) + snew) / page) for l in lens]
    pool = sum(pages) + spare
    perm = torch.randperm(pool, generator=g)
    bt = torch.zeros(B, max(pages), dtype=torch.int32)
    o = 0
    for b in range(B):
        bt[b, :pages[b]] = perm[o:o + pages[b]].to(torch.int32)
        o += pages[b]
    gd = torch.Generator(device=device).manual_seed(seed + 1)
    dt = torch.bfloat16

    def rn(*shape):
        return torch.randn(*shape, generator=gd, device=device, dtype=torch.float32).to(dt)

    def cache(*shape):
        # "nhd": (num_blocks, page, Hk, d) contiguous, the layout the API documents;
        # "hnd": same logical shape, memory laid out (num_blocks, Hk, page, d)
        if kv_layout == "hnd":
            nb, pg, h, dd = shape
            return rn(nb, h, pg, dd).permute(0, 2, 1, 3)
        return rn(*shape)

    w = dict(name=name, desc=desc, B=B, hq=hq, hk=hk, d=d, dv=d, page=page, lens=lens, snew=snew, window=window,
             causal=True, scale=d ** -0.5,
             q=rn(B, 1, hq, d), k_cache=cache(pool, page, hk, d), v_cache=cache(pool, page, hk, d),
             cache_seqlens=lens.to(torch.int32).to(device), block_table=bt.to(device), k=None, v=None,
             rotary_cos=None, rotary_sin=None)
    if snew:
        w["k"], w["v"] = rn(B, snew, hk, d), rn(B, snew, hk, d)
    if rotary:
        inv = 500000.0 ** (-torch.arange(0, d, 2, dtype=torch.float64) / d)
        ang = torch.arange(8192, dtype=torch.float64)[:, None] * inv[None, :]
        w["rotary_cos"], w["rotary_sin"] = torch.cos(ang).to(dt).to(device), torch.sin(ang).to(dt).to(device)
    return w


def mla_workload(device, seed: int = 0):
    """BASELINE.json configs[3]: DeepSeek-V3-shaped latent decode, int8 cache with per-token fp32 scales."""
    import torch
    g = torch.Generator(device="cpu").manual_seed(seed)
    B, hq, page = 32, 128, 256
    lens = torch.randint(2048, 16385, (B,), generator=g)
    pages = [math.ceil(int(l) / page) for l in lens]
    pool = sum(pages) + 8
    perm = torch.randperm(pool, generator=g)
    bt = torch.zeros(B, max(pages), dtype=torch.int32)
    o = 0
    for b in range(B):
        bt[b, :pages[b]] = perm[o:o + pages[b]].to(torch.int32)
        o += pages[b]
    gd = torch.Generator(device=device).manual_seed(seed + 1)
    latent = torch.randn(pool, page, 1, 576, generator=gd, device=device, dtype=torch.float32).to(torch.bfloat16)
    # symmetric per-token quantiser: scale = absmax / 127 (fp32), code = clamp(rne(x / scale), -127, 127)
    xf = latent.float()
    scale = xf.abs().amax(dim=-1, keepdim=True) / 127.0
    safe = torch.where(scale > 0, scale, torch.ones_like(scale))
    code = torch.clamp(torch.round(xf / safe), -127, 127).to(torch.int8)
    q = torch.randn(B, 1, hq, 576, generator=gd, device=device, dtype=torch.float32).to(torch.bfloat16)
    return dict(name="c4", desc="DeepSeek-V3-shaped MLA decode, int8 latent cache (576 B + fp32 scale per token, V aliased "
                                 "to the first 512 dims), B=32, 128 q heads, lens U[2048,16384], causal",
                B=B, hq=hq, hk=1, d=576, dv=512, page=page, lens=lens, snew=0, window=(-1, -1), causal=True,
                scale=192 ** -0.5, q=q, k_cache=code, v_cache=code[..., :512], k_scale=scale.squeeze(-1).contiguous(),
                cache_seqlens=lens.to(torch.int32).to(device), block_table=bt.to(device), k=None, v=None,
                rotary_cos=None, rotary_sin=None)


def decode_algorithmic_bytes(w):
    """Algorithmic HBM bytes of one decode call: every visible K and V element once, q, out, LSE,
    the block-table entries touched, plus (separately) the append's read+write."""
    B, hq, hk, d, dv, page, snew = w["B"], w["hq"], w["hk"], w["d"], w["dv"], w["page"], w["snew"]
    wl = w["window"][0]
    if w["k_cache"].dtype.itemsize == 1:
        # aliased int8 latent: 576 code bytes + one fp32 scale per token, read once
        per_key = d + 4
    else:
        per_key = hk * (d * 2 + dv * 2)
    kv = 0
    tbl = 0
    for l in w["lens"].tolist():
        lk = l + snew
        vis = lk if wl < 0 else min(lk, wl + 1)
        kv += vis * per_key
        tbl += 4 * math.ceil(vis / page)
    attn = kv + tbl + B * hq * (d * 2 + dv * 2) + B * hq * 4
    append = B * snew * hk * (d + dv) * (2 + 2)
    return attn, append


def bind_decode(w, num_splits=0):
    from flash_attn_npu import flash_attn_npu as ops
    return ops.bind_kvcache(w["q"], w["k_cache"], w["v_cache"], w["k"], w["v"], w["cache_seqlens"], w["rotary_cos"],
                            w["rotary_sin"], None, None, w["block_table"], None, None, w["scale"], w["causal"],
                            w["window"][0], w["window"][1], 0.0, False, num_splits, w.get("k_scale"), None)


def cpu_decode_baseline(w, budget_s: float = 20.0, min_s: float = 10.0):
    """The oracle's blocked golden (restated reference test golden) on host cores."""
    import torch
    import fa_oracle as O
    keys = ("q", "k_cache", "v_cache", "k", "v", "cache_seqlens", "block_table", "rotary_cos", "rotary_sin", "k_scale")
    h = {k: (w[k].cpu() if isinstance(w.get(k), torch.Tensor) else w.get(k)) for k in keys}
    if h["k_scale"] is not None:
        h["v_cache"] = h["k_cache"][..., :w["dv"]]
    # bounded sample: whole passes over the batch rows for at least min_s seconds, cut off inside a
    # pass once the budget is used up
    B = w["B"]
    t0 = time.perf_counter()
    secs, bytes_done, rows_done, passes = 0.0, 0.0, 0, 0
    while time.perf_counter() - t0 < min_s:
        times = []
        for start in range(0, B):
            sl = slice(start, start + 1)
            t1 = time.perf_counter()
            O.flash_attn_with_kvcache(h["q"][sl], h["k_cache"], h["v_cache"],
                                      None if h["k"] is None else h["k"][sl], None if h["v"] is None else h["v"][sl],
                                      rotary_cos=h["rotary_cos"], rotary_sin=h["rotary_sin"],
                                      cache_seqlens=h["cache_seqlens"][sl], block_table=h["block_table"][sl],
                                      softmax_scale=w["scale"], causal=w["causal"], window_size=w["window"],
                                      rotary_interleaved=False, k_scale_cache=h["k_scale"], mode="golden")
            times.append(time.perf_counter() - t1)
            if time.perf_counter() - t0 > budget_s:
                break
        done = len(times)
        sub = dict(w)
        sub["lens"] = w["lens"][:done]
        sub["B"] = done
        attn, app = decode_algorithmic_bytes(sub)
        bytes_done += attn + app
        secs += sum(times)
        rows_done += done
        passes += 1
        if done < B:
            break
    return dict(value=bytes_done / secs / 1e9, unit="GB/s", cores=torch.get_num_threads(), kind="port",
                sample=f"oracle blocked golden (fp32 math, 512-key chunks), {rows_done} batch rows of the same workload "
                       f"({passes} passes over its {B} rows), {secs:.2f} s on {os.cpu_count()} host cpus, "
                       f"torch threads {torch.get_num_threads()}",
                ms_per_call_extrapolated=secs / rows_done * B * 1e3)


# ----------------------------------------------------------------------------- warm-up
WARM_SECONDS = 0.1


def warm_up(args, run_one) -> int:
    """The untimed calls in front of a timed pass; returns how many were made.

    --warmup W makes exactly W.  Without it: at least 10 calls and at least WARM_SECONDS of them.  The device needs
    tens of milliseconds of work before its clocks have settled, and a matrix-bound call of 0.1 ms feels that: timed
    after 10 / 100 / 400 untimed calls, the latent decode config takes 130 / 121 / 111 us per call and its kernel
    105 / 104 / 98 us, where the memory-bound configs move by less than 1 %."""
    import torch
    if args.warmup is not None:
        for i in range(args.warmup):
            run_one(i)
        torch.cuda.synchronize()
        return args.warmup
    n, t0 = 0, time.perf_counter()
    while n < 10 or time.perf_counter() - t0 < WARM_SECONDS:
        run_one(n)
        n += 1
        if n % 8 == 0:
            torch.cuda.synchronize()   # the queue stays short, so the wall clock follows the device
    torch.cuda.synchronize()
    return n


# ----------------------------------------------------------------------------- main
def run_decode(args, name, cpu_budget=(20.0, 10.0)):
    import torch
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    # same seed -> same lengths and table, but distinct physical pools, rotated so that no step finds its K/V in the
    # 256 MB last-level cache: as many pools as it takes for the bytes a step reads, times the pools, to reach 512 MB
    first = mla_workload(dev, seed=0) if name == "c4" else decode_workload(name, dev, seed=0, kv_layout=args.kv_layout)
    attn_bytes, append_bytes = decode_algorithmic_bytes(first)
    total_bytes = attn_bytes + append_bytes
    npools = max(2, math.ceil(COLD_BYTES / attn_bytes))
    sets = [first] + [mla_workload(dev, seed=0) if name == "c4" else decode_workload(name, dev, seed=0, kv_layout=args.kv_layout)
                      for _ in range(npools - 1)]
    calls = [bind_decode(w, args.num_splits) for w in sets]
    w = sets[0]

    warmup = warm_up(args, lambda i: calls[i % npools].run())
    # the timed pass: K calls between two device synchronisations, with an event on the launch stream after every
    # `every`-th call, so that the wall mean and the median (of the groups' per-call durations) describe the same
    # launches.  An event between every two calls would cost each call 2.5-3 us (c2 204.7 -> 201.9 us, c3b 29.6 ->
    # 27.0 us, the same box with the marks 1 and 10 calls apart; no marks at all: 201.3 and 26.9 us): the kernel
    # behind a mark starts only when the one in front has drained, which no caller's loop would impose.
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    every = max(1, args.steps // 10)
    groups = args.steps // every
    marks = HipEvents(groups + 1)
    t0 = time.perf_counter()
    marks.record(0, stream)
    for i in range(args.steps):
        calls[i % npools].run()
        if (i + 1) % every == 0:
            marks.record((i + 1) // every, stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3
    call_ms = [marks.elapsed_ms(i, i + 1) / every for i in range(groups)]
    marks.close()

    # a second pass with the library's phase events, for the duration of the attention kernel alone (the events
    # between the kernels of a call would widen the call, so they stay out of the timed pass)
    ev = HipEvents(4 * args.steps)
    for i in range(args.steps):
        calls[i % npools].run(events=ev.group(i))
    torch.cuda.synchronize()
    k_ms = [ev.elapsed_ms(4 * i + 1, 4 * i + 2) for i in range(args.steps)]
    a_ms = [ev.elapsed_ms(4 * i + 0, 4 * i + 1) for i in range(args.steps)]
    c_ms = [ev.elapsed_ms(4 * i + 2, 4 * i + 3) for i in range(args.steps)]
    ev.close()
    kern_ms = median(k_ms)
    achieved = attn_bytes / (kern_ms * 1e-3) / 1e9
    traffic, traffic_file = traffic_from_profile(name) if args.kv_layout == "nhd" and args.num_splits == 0 else (None, None)

    from flash_attn_npu import _lib
    lib = _lib.load()
    plan = _lib.SplitPlan()
    lib.fa_rocm_plan_kvcache(C.byref(calls[0].args), lib.fa_rocm_num_cus(), C.byref(plan))

    if name == "c4":
        kernel_name = "decode_mla_i8_kernel"
    elif plan.mode != 1 and w["hq"] // w["hk"] > 16:
        kernel_name = "prefill_kernel"        # a query block too tall for the decode kernels of this head dimension: the tiled forward
    elif plan.mode == 1:
        kernel_name = "decode_wave_kernel" if plan.num_workers > plan.num_wgs else "decode_balanced_kernel"
    else:
        kernel_name = "decode_paged_kernel"
    out = {
        "metric": "paged_decode_hbm_bandwidth", "value": total_bytes / (ms_per_step * 1e-3) / 1e9, "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{name}: {w['desc']}", "batch": w["B"], "q_heads": w["hq"], "kv_heads": w["hk"],
                   "headdim": w["d"], "page_block_size": w["page"], "sum_keys": int(w["lens"].sum()) + w["B"] * w["snew"],
                   "split_mode": "balanced" if plan.mode == 1 else "grid", "workgroups": plan.num_wgs, "workers": plan.num_workers,
                   "kv_splits": plan.nsplits, "split_keys": plan.split_keys, "cold_cache": f"{npools} pools rotated, {npools * attn_bytes / 2**20:.0f} MiB read per rotation (last-level cache 256 MiB)", "kv_layout": args.kv_layout},
        "us_per_call": ms_per_step * 1e3,
        "us_per_call_median": median(call_ms) * 1e3,     # HIP events in the same timed pass, `marks_every` calls apart
        "marks_every": every,
        "pct_of_hbm_peak": 100.0 * total_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "algorithmic_bytes": total_bytes,
        "roofline": {"bound": "hbm", "kernel": kernel_name, "achieved": achieved, "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
                     "traffic": traffic, "traffic_source": traffic_file,
                     "kernel_us": kern_ms * 1e3, "kernel_us_stat": "median of per-step HIP events",
                     "append_us": median(a_ms) * 1e3, "combine_us": median(c_ms) * 1e3,
                     "algorithmic_bytes_per_launch": attn_bytes},
    }
    if name == "c4":
        # arithmetic intensity of this config is above the ridge: report the matrix-core side too
        flops = 2.0 * w["hq"] * (w["d"] + w["dv"]) * float(w["lens"].sum())
        out["dtype"] = "int8 cache, bf16 MFMA"
        out["roofline_mfma"] = {"bound": "mfma", "achieved": flops / (kern_ms * 1e-3) / 1e12, "peak": MFMA_BF16_PEAK_TFLOPS,
                                "unit": "TFLOP/s", "frac": flops / (kern_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                                "algorithmic_flops": flops}
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_decode_baseline(w, budget_s=cpu_budget[0], min_s=cpu_budget[1])
    del calls, sets, w
    torch.cuda.empty_cache()
    return out


def prefill_workload(device, seed: int = 0):
    """BASELINE.json configs[4]: 16 sequences, lengths uniform in [512, 4096] rescaled to a total of
    32768 tokens (largest remainder), 32 q heads / 8 kv heads, d = 128, bf16, causal."""
    import torch
    g = torch.Generator(device="cpu").manual_seed(seed)
    raw = torch.randint(512, 4097, (16,), generator=g).double()
    scaled = raw * (32768.0 / raw.sum())
    lens = scaled.floor().long()
    rem = 32768 - int(lens.sum())
    order = torch.argsort(scaled - lens.double(), descending=True)
    lens[order[:rem]] += 1
    cu = torch.zeros(17, dtype=torch.int32)
    cu[1:] = lens.cumsum(0).to(torch.int32)
    gd = torch.Generator(device=device).manual_seed(seed + 1)

    def rn(*shape):
        return torch.randn(*shape, generator=gd, device=device, dtype=torch.float32).to(torch.bfloat16)

    return dict(lens=lens, cu=cu.to(device), q=rn(32768, 32, 128), k=rn(32768, 8, 128), v=rn(32768, 8, 128),
                max_len=int(lens.max()), hq=32, hk=8, d=128)


def run_prefill(args, cpu_budget_s: float = 20.0):
    import torch
    from flash_attn_npu import flash_attn_npu as ops
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    w = prefill_workload(dev)
    scale = w["d"] ** -0.5
    flops = sum(4.0 * int(l) * int(l) * w["d"] * w["hq"] / 2.0 for l in w["lens"])
    out = torch.empty_like(w["q"])

    def step():
        return ops.varlen_fwd(w["q"], w["k"], w["v"], out, w["cu"], w["cu"], None, None, None, None, w["max_len"],
                              w["max_len"], 0.0, scale, False, True, -1, -1, 0.0, False, None)

    warmup = warm_up(args, lambda i: step())
    # one timed pass: K calls between two device synchronisations; the call is a single kernel, so the events
    # between the calls give its duration as well
    ev = HipEvents(args.steps + 1)
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    t0 = time.perf_counter()
    ev.record(0, stream)
    for i in range(args.steps):
        step()
        ev.record(i + 1, stream)
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    kern_ms = median([ev.elapsed_ms(i, i + 1) for i in range(args.steps)])
    ev.close()
    achieved = flops / (kern_ms * 1e-3) / 1e12
    traffic, traffic_file = traffic_from_profile("c5")
    res = {
        "metric": "varlen_prefill_fwd_tflops", "value": flops / (ms_per_step * 1e-3) / 1e12, "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "c5: varlen prefill forward bf16, 16 sequences (lengths U[512,4096] rescaled to 32768 "
                               "tokens), 32q/8kv heads, d=128, causal", "seq_lens": [int(x) for x in w["lens"]],
                   "flop_count": "sum 4*S^2*d*Hq / 2"},
        "us_per_call": ms_per_step * 1e3, "us_per_call_median": kern_ms * 1e3, "algorithmic_flops": flops,
        "pct_of_mfma_peak": 100.0 * flops / (ms_per_step * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
        "roofline": {"bound": "mfma", "kernel": "prefill_kernel", "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": achieved / MFMA_BF16_PEAK_TFLOPS, "traffic": traffic,
                     "traffic_source": traffic_file, "kernel_us": kern_ms * 1e3,
                     "kernel_us_stat": "median of per-step HIP events"},
    }
    if not args.no_cpu:
        import fa_oracle as O
        q, k, v, cu = w["q"].cpu(), w["k"].cpu(), w["v"].cpu(), w["cu"].cpu()
        done_flops, secs, n = 0.0, 0.0, 0
        for b in range(16):
            a, e = int(cu[b]), int(cu[b + 1])
            c1 = torch.tensor([0, e - a], dtype=torch.int32)
            t1 = time.perf_counter()
            O.flash_attn_varlen(q[a:e], k[a:e], v[a:e], c1, c1, e - a, e - a, softmax_scale=scale, causal=True, mode="golden")
            secs += time.perf_counter() - t1
            done_flops += 4.0 * (e - a) * (e - a) * w["d"] * w["hq"] / 2.0
            n += 1
            if secs > cpu_budget_s:
                break
        res["cpu_baseline"] = dict(value=done_flops / secs / 1e12, unit="TFLOP/s", cores=torch.get_num_threads(), kind="port",
                                   sample=f"oracle blocked golden on the first {n} of 16 sequences, {secs:.2f} s on "
                                          f"{os.cpu_count()} host cpus, torch threads {torch.get_num_threads()}")
    del w, out
    torch.cuda.empty_cache()
    return res


def run_mixed(args):
    """Not a BASELINE.json config: a token-major serving step over a paged cache through the varlen call, 63 decode
    rows (contexts uniform in [1024, 8191]) and one 1024-token prompt chunk at the end of a 16384-key context,
    32 q / 8 kv heads, d = 128, bf16, causal.  The decode rows are bound by HBM, the chunk by the matrix pipe: the
    line reports the time against the sum of the two roofs."""
    import torch
    from flash_attn_npu import flash_attn_npu as ops
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    hq, hk, d, page = 32, 8, 128, 256
    g = torch.Generator(device="cpu").manual_seed(0)
    lens_k = torch.randint(1024, 8192, (63,), generator=g).tolist() + [16384]
    lens_q = [1] * 63 + [1024]
    pages = [(n + page - 1) // page for n in lens_k]
    pool = sum(pages)
    table = torch.zeros(64, max(pages), dtype=torch.int32)
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    o = 0
    for b in range(64):
        table[b, :pages[b]] = perm[o:o + pages[b]]
        o += pages[b]
    gd = torch.Generator(device=dev).manual_seed(1)

    def rn(*shape):
        return torch.randn(*shape, generator=gd, device=dev, dtype=torch.float32).to(torch.bfloat16)

    sets = [(rn(pool, page, hk, d), rn(pool, page, hk, d)) for _ in range(2)]     # two pools alternated: cold caches
    q = rn(sum(lens_q), hq, d)
    out = torch.empty_like(q)
    cu_q = torch.tensor([0] + torch.tensor(lens_q).cumsum(0).tolist(), dtype=torch.int32, device=dev)
    used = torch.tensor(lens_k, dtype=torch.int32, device=dev)
    table = table.to(dev)
    scale = d ** -0.5

    def step(i):
        kc, vc = sets[i & 1]
        return ops.varlen_fwd(q, kc, vc, out, cu_q, None, used, None, table, None, max(lens_q), max(lens_k), 0.0, scale,
                              False, True, -1, -1, 0.0, False, None)

    warmup = warm_up(args, step)
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    decode_bytes = sum(lens_k[:63]) * hk * d * 2 * 2
    chunk_flops = 4.0 * 1024 * (16384 - 1024 + 1024 / 2.0) * d * hq
    at_roofs_us = decode_bytes / (HBM_PEAK_GBPS * 1e9) * 1e6 + chunk_flops / (MFMA_BF16_PEAK_TFLOPS * 1e12) * 1e6
    return {"metric": "mixed_batch_step_us", "value": ms * 1e3, "unit": "us", "n_gpus": 1, "steps": args.steps,
            "warmup": warmup, "ms_per_step": ms, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "mixed: token-major step over a paged cache, 63 decode rows (contexts U[1024,8191]) + one "
                                   "1024-token chunk ending a 16384-key context, 32q/8kv d=128 page=256 causal",
                       "decode_bytes": decode_bytes, "chunk_flops": chunk_flops},
            "us_per_call": ms * 1e3, "us_at_both_roofs": at_roofs_us, "frac_of_both_roofs": at_roofs_us / (ms * 1e3)}


def run_copy(args):
    """Plain device copy of known size (1 GiB read + 1 GiB written per step): the calibration
    workload for the FETCH_SIZE / WRITE_SIZE counters and a practical bandwidth yardstick."""
    import torch
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device="cuda:0").random_(0, 255)
    dst = torch.empty_like(src)
    warmup = warm_up(args, lambda i: dst.copy_(src))
    t0 = time.perf_counter()
    for _ in range(args.steps):
        dst.copy_(src)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    return {"metric": "device_copy_bandwidth", "value": 2 * n / (ms * 1e-3) / 1e9, "unit": "GB/s", "n_gpus": 1,
            "steps": args.steps, "warmup": warmup, "ms_per_step": ms, "higher_is_better": True,
            "config": {"workload": "copy: 1 GiB torch copy_ (read 1 GiB + write 1 GiB per step)"}}


def sub_record(r):
    """What a sub-record of the default line keeps of a config's own line."""
    keep = ("metric", "value", "unit", "warmup", "ms_per_step", "us_per_call", "us_per_call_median", "marks_every", "dtype", "roofline",
            "roofline_mfma", "cpu_baseline", "algorithmic_bytes", "algorithmic_flops")
    d = {k: r[k] for k in keep if k in r}
    d["workload"] = r["config"]["workload"]
    if "cold_cache" in r["config"]:
        d["cold_cache"] = r["config"]["cold_cache"]
    return d


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=None,
                    help="untimed calls in front of the timed ones; default: at least 10 and at least 0.1 s of them")
    ap.add_argument("--config", default="all", help="all = c2 headline plus sub-records of every other baseline config")
    ap.add_argument("--num-splits", type=int, default=0, help="0 = balanced partition (default), n >= 1 = fixed splits")
    ap.add_argument("--kv-layout", default="nhd", choices=["nhd", "hnd"], help="memory layout of the paged caches")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU golden timing")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the hot path has no cross-GPU exchange and this build uses a single "
              "MI355X; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a ROCm GPU", file=sys.stderr)
        sys.exit(2)
    if args.config == "all":
        out = run_decode(args, "c2")
        subs = {}
        for name in ("c2_8k", "c3a", "c3b", "c4"):
            r = run_decode(args, name, cpu_budget=(4.0, 2.5))
            subs[name] = sub_record(r)
        subs["c5"] = sub_record(run_prefill(args, cpu_budget_s=3.0))
        out["configs"] = subs
    elif args.config in ("c2", "c2_8k", "c3a", "c3b", "c4", "mqa32", "mqa32_d256", "mqa32_d64", "g32k8", "g32k8_d64", "g32k8_d256", "g64k8", "g48k8", "g32k4", "g32k2") or args.config.startswith("c2_u"):
        out = run_decode(args, args.config)
    elif args.config == "c5":
        out = run_prefill(args)
    elif args.config == "mixed":
        out = run_mixed(args)
    elif args.config == "copy":
        out = run_copy(args)
    else:
        raise SystemExit(f"unknown config {args.config}")
    print(json.dumps(out))


if __name__ == "__main__":
    main()
