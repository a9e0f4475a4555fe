#!/usr/bin/env python3
"""Benchmark of the TPA forward hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2|c2u|c3|c3u|c4|c4pg|c4s|c5|c5u|c2n|c5n|c5r|c5rn|c5rp|c2f|c3f|c2fb|c4f|c2m|c3m|c5m|c2p|c3p|c2pu|c3pu|c2b|c3b|c2pb|ap1|ap2|ap3|copy] [--no-cpu] [--no-decode] [--no-backward]

A step is one forward pass over one batch of synthetic, seeded inputs that are resident in HBM
before the timed region starts.  The default workload is the prefill configuration the headline
metric is quoted on (c2: B=4, T=4096, H=16, D=128, Rq=6, Rk=Rv=2, bf16, causal); the same run
also times the decode configuration (c4: B=64, cache 8192, H=32, D=128) and reports it in the
"decode" object, the backward pass at the c2 shape ("backward"), and times the CPU oracle on a bounded
sample of c2 ("cpu_baseline").
One JSON line is printed on stdout; progress goes to stderr.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "tensor-product-attention-jax_amd"))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2516.6  # MI355X dense bf16 MFMA
PEAK_F32_TFLOPS = 157.3    # MI355X dense fp32 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E

WORKLOADS = {
    # name: (kind, B, lq, lk, H, D, rq, rk, causal)
    "c2": ("prefill", 4, 4096, 4096, 16, 128, 6, 2, True),
    "c3": ("prefill", 1, 32768, 32768, 32, 128, 6, 2, True),
    "c5": ("prefill", 8, 2048, 2048, 64, 64, 16, 8, False),
    # the same two without the optional workspace: the fused kernel that rebuilds every K/V tile from the
    # rank factors inside the flash loop (with the workspace these shapes reconstruct dense K, V once)
    "c2u": ("prefill", 4, 4096, 4096, 16, 128, 6, 2, True),
    "c3u": ("prefill", 1, 32768, 32768, 32, 128, 6, 2, True),
    "c5u": ("prefill", 8, 2048, 2048, 64, 64, 16, 8, False),
    # nomat=True (tpa/tpa.py:250): the order of operations that never forms K or V, at the c2 and c5 shapes
    "c2n": ("prefill", 4, 4096, 4096, 16, 128, 6, 2, True),
    "c5n": ("prefill", 8, 2048, 2048, 64, 64, 16, 8, False),
    # the c5 shape with the benchmark ranks 6 / 2: the default route (c5r), the split-key order (c5rn) and the
    # reference's rank-pair tables, tpa/tpa.py:333-359 (c5rp)
    "c5r": ("prefill", 8, 2048, 2048, 64, 64, 6, 2, False),
    "c5rn": ("prefill", 8, 2048, 2048, 64, 64, 6, 2, False),
    "c5rp": ("prefill", 8, 2048, 2048, 64, 64, 6, 2, False),
    "c4": ("decode", 64, 1, 8192, 32, 128, 6, 2, False),
    "c4pg": ("decode", 64, 1, 8192, 32, 128, 6, 2, False),  # the c4 cache as a pool of shuffled 64-token pages
    "c4s": ("decode", 64, 4, 8192, 32, 128, 6, 2, True),  # four appended tokens per sequence, each masked to its predecessors
    # dense flash attention (tpa/mha.py) at the prefill shapes: the same-shape baseline
    "c2m": ("dense", 4, 4096, 4096, 16, 128, 0, 0, True),
    "c3m": ("dense", 1, 32768, 32768, 32, 128, 0, 0, True),
    "c5m": ("dense", 8, 2048, 2048, 64, 64, 0, 0, False),
    # packed sequences (segment ids, tpa/tpa.py:369-375): the c2 / c3 shapes holding documents of DOC_LEN tokens
    # backward pass (tpa/tpa.py:168-214) at the c2 / c3 shapes: gradients of all six factor arrays
    "c2b": ("backward", 4, 4096, 4096, 16, 128, 6, 2, True),
    "c3b": ("backward", 1, 32768, 32768, 32, 128, 6, 2, True),
    "c2pb": ("backward", 4, 4096, 4096, 16, 128, 6, 2, True),   # packed documents, as c2p
    "c2p": ("prefill", 4, 4096, 4096, 16, 128, 6, 2, True),
    "c3p": ("prefill", 1, 32768, 32768, 32, 128, 6, 2, True),
    "c2pu": ("prefill", 4, 4096, 4096, 16, 128, 6, 2, True),     # packed documents without a workspace: the fused kernel
    "c3pu": ("prefill", 1, 32768, 32768, 32, 128, 6, 2, True),
    # fp32 inputs (the reference's default dtype) at the c2 shape and at a quarter of c3's length: the fp32 MFMA kernel
    "c2f": ("prefill", 4, 4096, 4096, 16, 128, 6, 2, True),
    "c3f": ("prefill", 1, 16384, 16384, 32, 128, 6, 2, True),
    "c2fb": ("backward", 4, 4096, 4096, 16, 128, 6, 2, True),
    "c4f": ("decode", 64, 1, 8192, 32, 128, 6, 2, False),
    # the producer step (tpa_cache_append): (kind, B, new tokens, cache length, H, D, rq, rk, -) with d_model = H * D:
    # one decode step of the c4 batch, and a prefill chunk of 4096 tokens for four sequences
    "ap1": ("append", 64, 1, 8192, 32, 128, 6, 2, False),
    "ap2": ("append", 4, 4096, 8192, 32, 128, 6, 2, False),
    "ap3": ("append", 4, 512, 8192, 32, 128, 6, 2, False),     # a chunk of 2048 tokens: 128 x 128 tiles
}
F32_WORKLOADS = ("c2f", "c3f", "c2fb", "c4f")
COPY_BYTES = 1 << 30  # --workload copy: bytes read (and bytes written) by each plain copy launch

TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "prefill_c2_decode_c4_hbm_bytes.txt")


def mfma_sustained_rate():
    """TFLOP/s that back-to-back bf16 MFMAs on N(0, 1) operands sustain on this device, all CUs busy, nothing
    else running: the stand-alone yardstick built beside the library (csrc/mfma_rate.hip), run as a child
    process.  The published peak stays the roofline's `peak`; this says how much of it the matrix cores
    deliver on non-zero data under the device's power limit.  None if the program is missing or fails."""
    import subprocess

    exe = os.path.join(ROOT, "tensor-product-attention-jax_amd", "lib", "mfma_rate")
    if not os.access(exe, os.X_OK):
        log(f"[bench] {exe} not built: no sustained MFMA rate")
        return None
    try:
        out = subprocess.run([exe, "2", "0", "256", "8192"], capture_output=True, text=True, timeout=120, check=True).stdout
        return float(json.loads(out.strip().splitlines()[-1])["tflops"])
    except Exception as e:  # a yardstick, not part of the measurement
        log(f"[bench] mfma_rate failed: {e}")
        return None


def hbm_sustained_rates():
    """GB/s that a plain read (16-byte non-temporal loads) and a plain copy of 2 GiB buffers sustain on this device:
    the stand-alone yardstick built beside the library (csrc/hbm_rate.hip), run as a child process.  None if the
    program is missing or fails."""
    import subprocess

    exe = os.path.join(ROOT, "tensor-product-attention-jax_amd", "lib", "hbm_rate")
    if not os.access(exe, os.X_OK):
        log(f"[bench] {exe} not built: no sustained HBM rates")
        return None
    try:
        out = subprocess.run([exe, "2048"], capture_output=True, text=True, timeout=120, check=True).stdout
        line = json.loads(out.strip().splitlines()[-1])
        return float(line["read_gbs"]), float(line["copy_gbs"])
    except Exception as e:  # a yardstick, not part of the measurement
        log(f"[bench] hbm_rate failed: {e}")
        return None


def add_hbm_sustained(roof):
    rates = hbm_sustained_rates()
    if rates:
        log(f"[bench] a plain read sustains {rates[0]:.0f} GB/s on this device, a plain copy {rates[1]:.0f} GB/s (read + written)")
        roof["hbm_sustained"] = dict(read=rates[0], copy=rates[1], unit="GB/s", frac_of_peak_read=rates[0] / PEAK_HBM_GBS,
                                     achieved_over_sustained_read=roof["achieved"] / rates[0],
                                     how="hbm_rate 2048: 2 GiB buffers, 16-byte loads (non-temporal for the read), 2 in flight per lane, 768 workgroups of 256")


TRAFFIC_KERNELS = {  # workload -> the kernels of one step, as rocprofv3 prints the start of their names
    "c2": ["recon_bf16_h8_kernel", "prefill_kernel<128, 2, false>"],
    "c2u": ["prefill_kernel<128, 0, false>"],
    "c4": ["decode_kernel<128, 2, false, 1>", "decode_merge_kernel<128, bf16"],
}


def measured_traffic(workload):
    """HBM bytes per launch of the workload's kernels, read from the committed rocprofv3 counter summary
    (FETCH_SIZE / WRITE_SIZE in KiB per dispatch, one table row per kernel), each counter scaled by what it
    reads for the 1 GiB device copy in the same table.  None where the summary has no row for the kernels.
    This is a figure from the profile run named in the summary's header, not from the run that prints it."""
    kernels = TRAFFIC_KERNELS.get(workload)
    if not kernels or not os.path.exists(TRAFFIC_PROFILE):
        return None
    rows = {}
    for line in open(TRAFFIC_PROFILE):
        parts = line.split()
        for k in kernels + ["__amd_rocclr_copyBuffer"]:
            if line.strip().startswith(k):
                nums = [float(x) for x in parts if x.replace(".", "", 1).isdigit() and "." in x]
                if len(nums) >= 2:
                    rows[k] = nums[-2:]
    if "__amd_rocclr_copyBuffer" not in rows or any(k not in rows for k in kernels):
        return None
    kib = COPY_BYTES / 1024
    fetch_scale, write_scale = kib / rows["__amd_rocclr_copyBuffer"][0], kib / rows["__amd_rocclr_copyBuffer"][1]
    return sum(fetch_scale * rows[k][0] + write_scale * rows[k][1] for k in kernels) * 1024


def traffic_source():
    """where `roofline.traffic` comes from: the summary file and the source commit its header names"""
    commit = None
    if os.path.exists(TRAFFIC_PROFILE):
        for line in open(TRAFFIC_PROFILE):
            if "git commit" in line:
                commit = line.split("git commit")[1].split()[0].strip(".,;:()")
                break
    return dict(file=os.path.relpath(TRAFFIC_PROFILE, ROOT), source_commit=commit,
                how="rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE per dispatch, scaled by a 1 GiB device copy; not measured in this run")


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_inputs(torch, device, B, lq, lk, H, D, rq, rk, seed, dtype=None):
    """Split factor arrays, i.i.d. N(0,1) / sqrt(R), bf16 unless `dtype` says otherwise, generated on the device."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)

    def draw(shape, r):
        return (torch.randn(shape, generator=g, device=device, dtype=torch.float32) / r**0.5).to(dtype or torch.bfloat16)

    return (
        draw((B, lq, rq, H), rq), draw((B, lq, rq, D), rq),
        draw((B, lk, rk, H), rk), draw((B, lk, rk, D), rk),
        draw((B, lk, rk, H), rk), draw((B, lk, rk, D), rk),
    )


DOC_LEN = {"c2p": 1024, "c3p": 4096, "c2pb": 1024, "c2pu": 1024, "c3pu": 4096}


def prefill_flops(B, lq, lk, H, D, causal):
    pairs = lq * lk / 2 if causal else lq * lk
    return 2.0 * B * H * (D + D) * pairs


def decode_bytes(B, lq, lk, H, D, rq, rk, elem=2):
    cache = B * lk * (rk + rk) * (H + D) * elem
    qf = B * lq * rq * (H + D) * elem
    out = B * lq * H * D * elem + B * H * lq * 4
    return cache + qf + out


PREHEAT_S = 0.4  # seconds of the step itself, untimed, before the counted warm-up (see time_steps)


def time_steps(torch, fn, steps, warmup, preheat_s=None):
    """Times `steps` calls of fn after `warmup` untimed ones.  Returns a dict: wall ms per step over the
    whole timed region, and mean / median / min ms per step from events on the launch stream.

    Before the counted warm-up the step is repeated for `preheat_s` seconds (untimed, reported): the first
    workload of a process otherwise meets a device that has not settled yet - lazily loaded code objects,
    first-touch page mappings of fresh allocations, and a clock that the power management has not yet
    brought to what it holds under this load - and a few warm-up steps of 0.3 ms do not cover that."""
    preheat_s = PREHEAT_S if preheat_s is None else preheat_s
    t0 = time.perf_counter()
    n_pre = 0
    while time.perf_counter() - t0 < preheat_s:
        for _ in range(8):
            fn(n_pre)
            n_pre += 1
        torch.cuda.synchronize()
    pre_ms = (time.perf_counter() - t0) * 1e3
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        starts[i].record()
        fn(i)
        ends[i].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ev = [s.elapsed_time(e) for s, e in zip(starts, ends)]
    srt = sorted(ev)
    med = srt[len(srt) // 2] if len(srt) % 2 else 0.5 * (srt[len(srt) // 2 - 1] + srt[len(srt) // 2])
    log("[bench]   per-step event ms: " + " ".join(f"{x:.4f}" for x in ev))
    return dict(wall_ms=wall_ms, kernel_ms=sum(ev) / len(ev), kernel_ms_median=med, kernel_ms_min=srt[0],
                preheat=dict(seconds=pre_ms / 1e3, steps=n_pre))


def launch_times(r):
    """event times per step for a roofline object: mean (what `achieved` is computed from), median, fastest"""
    return dict(ms_per_launch=r["kernel_ms"], ms_per_launch_median=r["kernel_ms_median"], ms_per_launch_min=r["kernel_ms_min"],
                preheat=r["preheat"])


def run_prefill(torch, tpa, device, name, steps, warmup):
    _, B, lq, lk, H, D, rq, rk, causal = WORKLOADS[name]
    x = make_inputs(torch, device, B, lq, lk, H, D, rq, rk, seed=0, dtype=torch.float32 if name in F32_WORKLOADS else None)
    scale = D**-0.5
    out = {}
    doc = DOC_LEN.get(name)
    seg = None
    if doc:
        seg = (torch.arange(lq, device=device, dtype=torch.int32) // doc).repeat(B, 1).contiguous()

    use_ws = not name.endswith("u")
    nomat = "pairs" if name.endswith("rp") else name.endswith("n")

    def step(i):
        out["o"], out["lse"] = tpa.tpa_factors(*x, seg, seg, sm_scale=scale, causal=causal, kernel=2, use_workspace=use_ws, nomat=nomat)

    t = time_steps(torch, step, steps, warmup)
    wall_ms, ev_ms, ev_min, ev_med = t["wall_ms"], t["kernel_ms"], t["kernel_ms_min"], t["kernel_ms_median"]
    # packed: only pairs inside a document count
    fl = prefill_flops(B * (lq // doc), doc, doc, H, D, causal) if doc else prefill_flops(B, lq, lk, H, D, causal)
    return dict(
        wall_ms=wall_ms, kernel_ms=ev_ms, kernel_ms_min=ev_min, kernel_ms_median=ev_med, preheat=t["preheat"], flops=fl,
        tflops_wall=fl / wall_ms / 1e9, tflops_kernel=fl / ev_ms / 1e9,
        shape=dict(B=B, lq=lq, lk=lk, H=H, D=D, rank_q=rq, rank_k=rk, causal=causal, **({"document_len": doc} if doc else {})),
        inputs=x, out=out,
    )


def run_dense_prefill(torch, mha, device, name, steps, warmup):
    """Dense multi-head flash attention (tpa/mha.py:23-37) on q, k, v [B, T, H, D] bf16."""
    _, B, lq, lk, H, D, _, _, causal = WORKLOADS[name]
    g = torch.Generator(device=device)
    g.manual_seed(5)
    draw = lambda l: torch.randn((B, l, H, D), generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)
    q, k, v = draw(lq), draw(lk), draw(lk)
    scale = D**-0.5

    def step(i):
        mha._mha_fwd(q, k, v, None, scale, causal=causal, kernel=2)

    t = time_steps(torch, step, steps, warmup)
    wall_ms, ev_ms, ev_min, ev_med = t["wall_ms"], t["kernel_ms"], t["kernel_ms_min"], t["kernel_ms_median"]
    fl = prefill_flops(B, lq, lk, H, D, causal)
    return dict(
        wall_ms=wall_ms, kernel_ms=ev_ms, kernel_ms_min=ev_min, kernel_ms_median=ev_med, preheat=t["preheat"], flops=fl,
        tflops_wall=fl / wall_ms / 1e9, tflops_kernel=fl / ev_ms / 1e9,
        shape=dict(B=B, lq=lq, lk=lk, H=H, D=D, causal=causal),
    )


def run_backward(torch, tpa, device, name, steps, warmup):
    """One step = one call of the backward entry point (all its kernels) on resident inputs, with
    the forward's o and lse computed once beforehand."""
    _, B, lq, lk, H, D, rq, rk, causal = WORKLOADS[name]
    dtype = torch.float32 if name in F32_WORKLOADS else torch.bfloat16
    x = make_inputs(torch, device, B, lq, lk, H, D, rq, rk, seed=0, dtype=dtype)
    scale = D**-0.5
    doc = DOC_LEN.get(name)
    seg = (torch.arange(lq, device=device, dtype=torch.int32) // doc).repeat(B, 1).contiguous() if doc else None
    o, lse = tpa.tpa_factors(*x, seg, seg, sm_scale=scale, causal=causal, kernel=2)
    g = torch.Generator(device=device)
    g.manual_seed(7)
    do = torch.randn(o.shape, generator=g, device=device, dtype=torch.float32).to(dtype)
    grads = tuple(torch.empty(t.shape, dtype=torch.float32, device=device) for t in x)
    ws = torch.empty(tpa.bwd_workspace_bytes(B, lq, lk, H, D, D) + 256, dtype=torch.uint8, device=device)

    def step(i):
        tpa.tpa_factors_bwd(*x, seg, seg, o, lse, do, scale, causal, grads=grads, workspace=ws, kernel=2)

    t = time_steps(torch, step, steps, warmup)
    wall_ms, ev_ms, ev_min, ev_med = t["wall_ms"], t["kernel_ms"], t["kernel_ms_min"], t["kernel_ms_median"]
    # five contractions against the forward's two; packed: only pairs inside a document count
    fl = 2.5 * (prefill_flops(B * (lq // doc), doc, doc, H, D, causal) if doc else prefill_flops(B, lq, lk, H, D, causal))
    return dict(
        wall_ms=wall_ms, kernel_ms=ev_ms, kernel_ms_min=ev_min, kernel_ms_median=ev_med, preheat=t["preheat"], flops=fl,
        tflops_wall=fl / wall_ms / 1e9, tflops_kernel=fl / ev_ms / 1e9,
        shape=dict(B=B, lq=lq, lk=lk, H=H, D=D, rank_q=rq, rank_k=rk, causal=causal, **({"document_len": doc} if doc else {})),
    )


def run_decode(torch, tpa, device, name, steps, warmup):
    _, B, lq, lk, H, D, rq, rk, causal = WORKLOADS[name]
    causal = tpa.CAUSAL_BOTTOM_RIGHT if causal else False
    # two distinct caches, alternated, so that no launch finds its cache in the 256 MB last-level cache
    f32 = name in F32_WORKLOADS
    xs = [make_inputs(torch, device, B, lq, lk, H, D, rq, rk, seed=s, dtype=torch.float32 if f32 else None) for s in (0, 1)]
    scale = D**-0.5
    ws = torch.empty(max(tpa.decode_workspace_bytes(B, lq, lk, H, D), 16), dtype=torch.uint8, device=device)
    out = {}
    table = None
    if name == "c4pg":
        page = 64
        g = torch.Generator(device=device)
        g.manual_seed(11)
        table = torch.randperm(B * lk // page, generator=g, device=device).to(torch.int32).reshape(B, lk // page)
        # a pool holds the same bytes; which page holds what does not matter for the timing
        xs = [x[:2] + tuple(t.reshape(B * lk // page, page, rk, t.shape[-1]) for t in x[2:]) for x in xs]

    def step(i):
        out["o"], out["lse"] = tpa.tpa_decode(*xs[i & 1], sm_scale=scale, workspace=ws, kernel=2, page_table=table, causal=causal)

    t = time_steps(torch, step, steps, warmup)
    wall_ms, ev_ms, ev_min, ev_med = t["wall_ms"], t["kernel_ms"], t["kernel_ms_min"], t["kernel_ms_median"]
    nbytes = decode_bytes(B, lq, lk, H, D, rq, rk, elem=4 if f32 else 2)
    return dict(
        wall_ms=wall_ms, kernel_ms=ev_ms, kernel_ms_min=ev_min, kernel_ms_median=ev_med, preheat=t["preheat"], bytes=nbytes,
        gbs_wall=nbytes / wall_ms / 1e6, gbs_kernel=nbytes / ev_ms / 1e6,
        shape=dict(B=B, lq=lq, lk=lk, H=H, D=D, rank_q=rq, rank_k=rk), inputs=xs[0], out=out,
    )


def run_append(torch, tpa, device, name, steps, warmup):
    """One step = one tpa_cache_append call: y = x W^T (M = B * n tokens, d_model = H * D inputs,
    rq (H + D) + 2 rk (H + D) outputs), rotary embedding, rows appended to a bf16 factored cache."""
    _, B, n, cache_len, H, D, rq, rk, _ = WORKLOADS[name]
    dm = H * D
    n_out = rq * (H + D) + 2 * rk * (H + D)
    g = torch.Generator(device=device)
    g.manual_seed(9)
    x = torch.randn((B, n, dm), generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)
    w = (torch.randn((n_out, dm), generator=g, device=device, dtype=torch.float32) / dm**0.5).to(torch.bfloat16)
    ang = torch.arange(cache_len, device=device, dtype=torch.float32)[:, None] * (10000.0 ** (-torch.arange(0, D, 2, device=device, dtype=torch.float32) / D))[None]
    cos, sin = torch.cos(ang), torch.sin(ang)
    caches = [torch.zeros((B, cache_len, rk, inner), dtype=torch.bfloat16, device=device) for inner in (H, D, H, D)]
    lengths = torch.full((B,), cache_len - n - 1, dtype=torch.int32, device=device)

    ws_bytes = tpa.cache_append_workspace_bytes(B, n, dm, H, D, rq, rk)  # decode steps split the contraction over workgroups
    ws = torch.empty(ws_bytes + 16, dtype=torch.uint8, device=device) if ws_bytes else None

    def step(i):
        tpa.tpa_cache_append(x, w, cos, sin, *caches, lengths, rank_q=rq, kernel=2, workspace=ws)

    t = time_steps(torch, step, steps, warmup)
    wall_ms, ev_ms, ev_min, ev_med = t["wall_ms"], t["kernel_ms"], t["kernel_ms_min"], t["kernel_ms_median"]
    fl = 2.0 * B * n * dm * n_out
    nbytes = (B * n * dm + n_out * dm + B * n * n_out) * 2
    return dict(wall_ms=wall_ms, kernel_ms=ev_ms, kernel_ms_min=ev_min, kernel_ms_median=ev_med, preheat=t["preheat"], flops=fl, bytes=nbytes,
                shape=dict(B=B, new_tokens=n, d_model=dm, H=H, D=D, rank_q=rq, rank_k=rk, outputs=n_out))


def run_dense_decode(torch, mha, device, name, steps, warmup):
    """Dense attention (tpa/mha.py) at the decode configuration: the baseline the factored cache is
    compared with.  K and V hold H*D values per token instead of R*(H+D)."""
    _, B, lq, lk, H, D, _, _, _ = WORKLOADS[name]
    g = torch.Generator(device=device)
    g.manual_seed(3)
    draw = lambda *shape: torch.randn(shape, generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)
    q = draw(B, lq, H, D)
    kvs = []
    for _ in range(2):  # two caches, alternated (each is far larger than the last-level cache anyway)
        kvs.append((torch.cat([draw(B // 4, lk, H, D) for _ in range(4)]), torch.cat([draw(B // 4, lk, H, D) for _ in range(4)])))
    scale = D**-0.5

    def step(i):
        k, v = kvs[i & 1]
        mha._mha_fwd(q, k, v, None, scale, kernel=2)

    t = time_steps(torch, step, steps, warmup)
    wall_ms, ev_ms, ev_min, ev_med = t["wall_ms"], t["kernel_ms"], t["kernel_ms_min"], t["kernel_ms_median"]
    nbytes = 2 * B * lk * H * D * 2 + B * lq * H * D * 2 * 2 + B * H * lq * 4
    return dict(wall_ms=wall_ms, kernel_ms=ev_ms, kernel_ms_min=ev_min, kernel_ms_median=ev_med, preheat=t["preheat"], bytes=nbytes, gbs_kernel=nbytes / ev_ms / 1e6)


def cpu_baseline_prefill(torch, inputs, shape, budget_s=12.0):
    """The numpy oracle on the prefill workload, one batch element (all heads) at a time, until the
    workload is done or `budget_s` seconds of CPU work have been spent.  Returns the figures and
    the oracle's output for batch element 0."""
    import numpy as np

    from oracle import tpa_oracle as orc

    D, H = shape["D"], shape["H"]
    dt, done, o0, lse0 = 0.0, 0, None, None
    for it in range(64 * shape["B"]):  # cycles through the batch elements until the budget is spent
        b = it % shape["B"]
        qa, qb, ka, kb, va, vb = (t[b : b + 1].float().cpu().numpy() for t in inputs)
        cat = lambda a, b_: np.concatenate([a, b_], axis=-1)
        q, k, v = cat(qa, qb), cat(ka, kb), cat(va, vb)
        t0 = time.perf_counter()
        o, lse = orc.tpa_reference(q, k, v, None, None, H, sm_scale=D**-0.5, causal=shape["causal"], dtype=np.float32)
        dt += time.perf_counter() - t0
        done += 1
        if it == 0:
            o0, lse0 = o, lse
        if dt >= budget_s:
            break
    fl = prefill_flops(done, shape["lq"], shape["lk"], H, D, shape["causal"])
    try:
        from threadpoolctl import threadpool_info

        threads = max([p.get("num_threads", 1) for p in threadpool_info()] + [1])
    except Exception:
        threads = os.cpu_count() or 1
    return dict(
        value=fl / dt / 1e12, unit="TFLOP/s", cores=threads, kind="port",
        sample=f"numpy fp32 oracle on {done} batch elements (all {H} heads; the workload has {shape['B']}, taken in turn), "
        f"{dt:.1f} s of CPU work; matmuls on {threads} BLAS threads of {os.cpu_count()} host cores, "
        f"the rest single-threaded; its flops counted as the kernel's are",
    ), o0, lse0


def main():
    global PREHEAT_S
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS) + ["copy"],
                    help="copy = a plain device copy of known size, the yardstick for the HBM byte counters")
    ap.add_argument("--preheat", type=float, default=PREHEAT_S,
                    help="seconds of untimed repetitions of a workload's step before its counted warm-up (0 = none)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-decode", action="store_true", help="skip the secondary decode measurement")
    ap.add_argument("--no-backward", action="store_true", help="skip the secondary backward measurement")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives are built); use --gpus 1")
    PREHEAT_S = max(0.0, args.preheat)

    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no HIP device visible")
    from tpa import tpa

    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.workload == "copy":
        src = torch.empty(COPY_BYTES, dtype=torch.uint8, device=device).random_(0, 255)
        dst = torch.empty_like(src)
        t = time_steps(torch, lambda i: dst.copy_(src), args.steps, args.warmup)
        wall_ms, ev_ms = t["wall_ms"], t["kernel_ms"]
        print(json.dumps(dict(metric="plain device copy", value=2 * COPY_BYTES / ev_ms / 1e6, unit="GB/s",
                              bytes_read_per_launch=COPY_BYTES, bytes_written_per_launch=COPY_BYTES,
                              ms_per_step=wall_ms, ms_per_launch=ev_ms, n_gpus=1, steps=args.steps,
                              warmup=args.warmup)), flush=True)
        return
    kind = WORKLOADS[args.workload][0]
    result = {}
    if kind == "prefill":
        log(f"[bench] prefill {args.workload}: warmup {args.warmup}, steps {args.steps}")
        f32 = args.workload in F32_WORKLOADS
        peak = PEAK_F32_TFLOPS if f32 else PEAK_BF16_TFLOPS
        r = run_prefill(torch, tpa, device, args.workload, args.steps, args.warmup)
        log(f"[bench] {r['kernel_ms']:.4f} ms/launch (min {r['kernel_ms_min']:.4f}), {r['tflops_kernel']:.1f} TFLOP/s")
        result.update(
            metric="TPA causal prefill forward throughput" if r["shape"]["causal"] else "TPA prefill forward throughput",
            value=r["tflops_wall"], unit="TFLOP/s", ms_per_step=r["wall_ms"],
            roofline=dict(bound="mfma", achieved=r["tflops_kernel"], peak=peak, unit="TFLOP/s",
                          frac=r["tflops_kernel"] / peak, traffic=measured_traffic(args.workload),
                          **({"traffic_source": traffic_source()} if measured_traffic(args.workload) else {}),
                          kernel="prefill_f32_kernel" if f32 else ("nomat_pairs_kernel" if args.workload.endswith("rp") else "decode_kernel + decode_merge_kernel per 64 query rows" if args.workload.endswith("n")
                                                                   else "prefill_kernel" if args.workload.endswith("u") else "recon_bf16_h8_kernel + prefill_kernel"),
                          **launch_times(r), algorithmic_flops_per_launch=r["flops"]),
            config=dict(workload=f"{args.workload}: TPA prefill" + (", fp32 inputs" if f32 else "") + (", nomat (rank-pair tables)" if args.workload.endswith("rp") else ", nomat" if args.workload.endswith("n") else ""), **r["shape"]),
        )
        if not args.no_decode and not f32:
            log("[bench] decode c4")
            d = run_decode(torch, tpa, device, "c4", args.steps, args.warmup)
            log(f"[bench] {d['kernel_ms']*1e3:.1f} us/launch (min {d['kernel_ms_min']*1e3:.1f}), {d['gbs_kernel']:.0f} GB/s")
            result["decode"] = dict(
                metric="TPA decode effective HBM bandwidth", value=d["gbs_wall"], unit="GB/s", ms_per_step=d["wall_ms"],
                roofline=dict(bound="hbm", achieved=d["gbs_kernel"], peak=PEAK_HBM_GBS, unit="GB/s",
                              frac=d["gbs_kernel"] / PEAK_HBM_GBS, traffic=measured_traffic("c4"),
                              **({"traffic_source": traffic_source()} if measured_traffic("c4") else {}),
                              kernel="decode_kernel + decode_merge_kernel",
                              **launch_times(d),
                              algorithmic_bytes_per_launch=d["bytes"]),
                config=dict(workload="c4: TPA decode over the factored KV cache", **d["shape"]),
            )
            add_hbm_sustained(result["decode"]["roofline"])
            log("[bench] dense decode at the c4 shape")
            from tpa import mha

            dd = run_dense_decode(torch, mha, device, "c4", max(10, args.steps // 5), 3)
            log(f"[bench] {dd['kernel_ms']*1e3:.1f} us/launch, {dd['gbs_kernel']:.0f} GB/s")
            result["decode"]["dense_mha_same_shape"] = dict(
                ms_per_launch=dd["kernel_ms"], achieved=dd["gbs_kernel"], unit="GB/s", frac=dd["gbs_kernel"] / PEAK_HBM_GBS,
                algorithmic_bytes_per_launch=dd["bytes"], speedup_of_factored_cache=dd["kernel_ms"] / d["kernel_ms"])
        if not args.no_backward and args.workload == "c2":
            log("[bench] backward at the c2 shape")
            bw = run_backward(torch, tpa, device, "c2b", max(10, args.steps // 2), 5)
            log(f"[bench] {bw['kernel_ms']:.4f} ms/call, {bw['tflops_kernel']:.1f} TFLOP/s")
            result["backward"] = dict(
                metric="TPA causal prefill backward throughput", value=bw["tflops_wall"], unit="TFLOP/s", ms_per_step=bw["wall_ms"],
                roofline=dict(bound="mfma", achieved=bw["tflops_kernel"], peak=PEAK_BF16_TFLOPS, unit="TFLOP/s",
                              frac=bw["tflops_kernel"] / PEAK_BF16_TFLOPS, traffic=None,
                              kernel="recon + delta + bwd_dq_kernel + bwd_dkv_kernel + project (whole call)",
                              **launch_times(bw),
                              algorithmic_flops_per_launch=bw["flops"]),
                config=dict(workload="c2b: TPA backward", **bw["shape"]),
            )
        if not args.no_cpu and args.workload == "c2":
            log("[bench] cpu baseline (numpy oracle on a sample)")
            base, o_ref, _ = cpu_baseline_prefill(torch, r["inputs"], r["shape"])
            result["cpu_baseline"] = base
            # the sample doubles as a parity check of the timed kernel's output
            err = float(abs(r["out"]["o"][:1].float().cpu().numpy() - o_ref).max())
            result["max_abs_err_vs_oracle_sample"] = err
            log(f"[bench] cpu {base['value']*1e3:.2f} GFLOP/s; max abs err vs oracle on the sample {err:.2e}")
    elif kind == "dense":
        from tpa import mha

        log(f"[bench] dense flash attention {args.workload}: warmup {args.warmup}, steps {args.steps}")
        r = run_dense_prefill(torch, mha, device, args.workload, args.steps, args.warmup)
        log(f"[bench] {r['kernel_ms']:.4f} ms/launch (min {r['kernel_ms_min']:.4f}), {r['tflops_kernel']:.1f} TFLOP/s")
        result.update(
            metric="dense flash attention forward throughput", value=r["tflops_wall"], unit="TFLOP/s", ms_per_step=r["wall_ms"],
            roofline=dict(bound="mfma", achieved=r["tflops_kernel"], peak=PEAK_BF16_TFLOPS, unit="TFLOP/s",
                          frac=r["tflops_kernel"] / PEAK_BF16_TFLOPS, traffic=None, kernel="prefill_kernel (dense loader)",
                          **launch_times(r),
                          algorithmic_flops_per_launch=r["flops"]),
            config=dict(workload=f"{args.workload}: dense flash attention (tpa/mha.py) at the prefill shape", **r["shape"]),
        )
    elif kind == "append":
        log(f"[bench] cache append {args.workload}: warmup {args.warmup}, steps {args.steps}")
        r = run_append(torch, tpa, device, args.workload, args.steps, args.warmup)
        # few tokens: the weights are read once (HBM); many: the product is bound by the matrix cores
        hbm = r["shape"]["new_tokens"] * r["shape"]["B"] <= 256
        ach = r["bytes"] / r["kernel_ms"] / 1e6 if hbm else r["flops"] / r["kernel_ms"] / 1e9
        log(f"[bench] {r['kernel_ms']*1e3:.1f} us/launch, {ach:.1f} {'GB/s' if hbm else 'TFLOP/s'}")
        result.update(
            metric="TPA cache append (factor projections + rotary embedding) throughput", value=(r["bytes"] / r["wall_ms"] / 1e6 if hbm else r["flops"] / r["wall_ms"] / 1e9),
            unit="GB/s" if hbm else "TFLOP/s", ms_per_step=r["wall_ms"],
            roofline=dict(bound="hbm" if hbm else "mfma", achieved=ach, peak=PEAK_HBM_GBS if hbm else PEAK_BF16_TFLOPS,
                          unit="GB/s" if hbm else "TFLOP/s", frac=ach / (PEAK_HBM_GBS if hbm else PEAK_BF16_TFLOPS), traffic=None,
                          kernel="append_fewrows_kernel + append_finish_kernel" if hbm else ("append_gemm_kernel<2>" if args.workload == "ap3" else "append_gemm_kernel<4>"), **launch_times(r),
                          algorithmic_flops_per_launch=r["flops"], algorithmic_bytes_per_launch=r["bytes"]),
            config=dict(workload=f"{args.workload}: TPA cache append", **r["shape"]),
        )
    elif kind == "backward":
        log(f"[bench] backward {args.workload}: warmup {args.warmup}, steps {args.steps}")
        r = run_backward(torch, tpa, device, args.workload, args.steps, args.warmup)
        log(f"[bench] {r['kernel_ms']:.4f} ms/call (min {r['kernel_ms_min']:.4f}), {r['tflops_kernel']:.1f} TFLOP/s")
        f32 = args.workload in F32_WORKLOADS
        peak = PEAK_F32_TFLOPS if f32 else PEAK_BF16_TFLOPS
        result.update(
            metric="TPA causal prefill backward throughput", value=r["tflops_wall"], unit="TFLOP/s", ms_per_step=r["wall_ms"],
            roofline=dict(bound="mfma", achieved=r["tflops_kernel"], peak=peak, unit="TFLOP/s",
                          frac=r["tflops_kernel"] / peak, traffic=None,
                          kernel=("recon + delta + bwd_f32_dq_kernel + bwd_f32_dkv_kernel + project (whole call)" if f32 else
                                  "recon + delta + bwd_dq_kernel + bwd_dkv_kernel + project (whole call)"),
                          **launch_times(r),
                          algorithmic_flops_per_launch=r["flops"]),
            config=dict(workload=f"{args.workload}: TPA backward" + (", fp32 inputs" if f32 else ""), **r["shape"]),
        )
    else:
        log(f"[bench] decode {args.workload}: warmup {args.warmup}, steps {args.steps}")
        d = run_decode(torch, tpa, device, args.workload, args.steps, args.warmup)
        log(f"[bench] {d['kernel_ms']*1e3:.1f} us/launch (min {d['kernel_ms_min']*1e3:.1f}), {d['gbs_kernel']:.0f} GB/s")
        result.update(
            metric="TPA decode effective HBM bandwidth", value=d["gbs_wall"], unit="GB/s", ms_per_step=d["wall_ms"],
            roofline=dict(bound="hbm", achieved=d["gbs_kernel"], peak=PEAK_HBM_GBS, unit="GB/s",
                          frac=d["gbs_kernel"] / PEAK_HBM_GBS, traffic=measured_traffic(args.workload),
                          **({"traffic_source": traffic_source()} if measured_traffic(args.workload) else {}),
                          kernel=("decode_f32_kernel" if args.workload in F32_WORKLOADS else "decode_kernel") + " + decode_merge_kernel",
                          **launch_times(d),
                          algorithmic_bytes_per_launch=d["bytes"]),
            config=dict(workload=f"{args.workload}: TPA decode over the factored KV cache" +
                        (", fp32 cache" if args.workload in F32_WORKLOADS else ""), **d["shape"]),
        )
    roof = result.get("roofline", {})
    if roof.get("bound") == "hbm" and kind == "decode":
        add_hbm_sustained(roof)
    if roof.get("bound") == "mfma" and args.workload not in F32_WORKLOADS:
        rate = mfma_sustained_rate()
        if rate:
            log(f"[bench] back-to-back bf16 MFMAs on N(0,1) operands sustain {rate:.0f} TFLOP/s on this device ({rate / PEAK_BF16_TFLOPS:.2f} of the published peak)")
            roof["mfma_sustained"] = dict(value=rate, unit="TFLOP/s", frac_of_peak=rate / PEAK_BF16_TFLOPS,
                                          achieved_over_sustained=roof["achieved"] / rate,
                                          how="mfma_rate 2 0 256 8192: 8 independent v_mfma_f32_32x32x16_bf16 chains per wave, 2 waves per SIMD, 256 workgroups, no memory traffic")
    result.update(
        n_gpus=1, steps=args.steps, warmup=args.warmup, higher_is_better=True, scaling="weak",
        vs_baseline=None, dtype="f32" if args.workload in F32_WORKLOADS else "bf16", data="synthetic",
    )
    # the yardstick children have been waited for (subprocess.run); release the device memory before the line is
    # printed, so that the process is gone right after it
    r = d = bw = None
    import gc

    gc.collect()
    torch.cuda.empty_cache()
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
