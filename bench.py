#!/usr/bin/env python3
"""Benchmark of the block-sparse attention forward on one MI355X.

One "step" is one forward launch over the whole synthetic batch of the workload, called
through the C ABI with q/k/v and the block-mask metadata already resident in HBM.
Prints ONE JSON line.  `value` is effective TFLOP/s: 4*QB*KB*D flops per listed
(non-empty) block -- CAUSAL and PARTIAL blocks count as full tiles, softmax flops are
not counted, EMPTY blocks count nothing -- divided by the wall time per step.

Before the W counted warm-up launches the bench keeps the GPU under this same load for a
fixed time (--clock-settle-ms, reported as `clock_settle`): from idle the shader clock takes
some tens of milliseconds of load to reach the level it then holds, and a short run would
time that ramp instead of the kernel.  K and W are exactly what was passed.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline]
    python bench.py --sweep-bands     # runtime against the number of listed blocks (fixed shape)
    python bench.py --kernel-source-hash   # hash that ties a traffic measurement to the kernel sources
"""
import argparse
import hashlib
import json
import os
import re
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(ROOT, "omni-attention_amd")
for _p in (ROOT, PKG):
    if _p not in sys.path:
        sys.path.insert(0, _p)

METRIC = "effective TFLOP/s (non-empty blocks) + % bf16 MFMA peak, 8K interleaved mask"
MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 / fp16 MFMA

# HBM bytes per launch come from two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE), each scaled
# by what the same counter reads for a plain copy of known size.  The figures live in a tracked
# summary under profiles/, in a table row per workload that also records the hash of the kernel
# sources the run was made with; a figure whose hash is not the hash of the sources in this tree
# describes another kernel and is not reported.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "fwd_kernel_hbm_traffic.md")
KERNEL_SOURCES = ("omni_attn_fwd_kernel.hpp", "omni_attn_fwd_inst.hip", "omni_attn_capi.hip")


def kernel_source_hash() -> str:
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(PKG, "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def read_traffic_profile(path: str = TRAFFIC_PROFILE):
    """Rows `| workload | FETCH_SIZE KiB | fetch factor | WRITE_SIZE KiB | write factor | hash |`
    of the tracked summary -> {workload: {"bytes": ..., "kernel_source_hash": ...}}."""
    out = {}
    if not os.path.exists(path):
        return out
    row = re.compile(r"^\|\s*(\w+)\s*\|\s*([\d.]+)\s*\|\s*([\d.]+)\s*\|\s*([\d.]+)\s*\|\s*([\d.]+)\s*\|\s*([0-9a-f]{16})\s*\|")
    with open(path) as f:
        for line in f:
            m = row.match(line)
            if m:
                fetch, ff, write, wf = (float(m.group(i)) for i in range(2, 6))
                out[m.group(1)] = {"bytes": int((fetch * ff + write * wf) * 1024),
                                   "kernel_source_hash": m.group(6)}
    return out


def traffic_for(workload: str):
    """(bytes or None, provenance dict) for the roofline object."""
    rec = read_traffic_profile().get(workload)
    here = kernel_source_hash()
    if rec is None:
        return None, {"source": None, "measured_at_head": False, "kernel_source_hash": here}
    fresh = rec["kernel_source_hash"] == here
    return (rec["bytes"] if fresh else None), {
        "source": os.path.relpath(TRAFFIC_PROFILE, ROOT), "measured_at_head": fresh,
        "kernel_source_hash": here, "profile_kernel_source_hash": rec["kernel_source_hash"],
        "stale_bytes": None if fresh else rec["bytes"]}


def measure_mfma_peak(dev, dtype_code: int, target_ms: float = 60.0):
    """TFLOP/s of the library's pure matrix-instruction loop (two waves per SIMD, operands in
    registers), timed with events on the launch stream after the clock has settled under it."""
    import torch

    import omni_attn_capi

    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream(dev)
    iters = 20000
    t_end = time.perf_counter() + 0.25
    while time.perf_counter() < t_end:  # settle the clock under this load
        for _ in range(5):
            omni_attn_capi.mfma_peak_probe(dtype_code, iters, sink, stream.cuda_stream)
        torch.cuda.synchronize()
    best = 0.0
    for _ in range(5):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(stream)
        flops = omni_attn_capi.mfma_peak_probe(dtype_code, iters, sink, stream.cuda_stream)
        b.record(stream)
        torch.cuda.synchronize()
        best = max(best, flops / (a.elapsed_time(b) * 1e-3) / 1e12)
    return best


def cpu_baseline(w, budget_s: float):
    """The fp32 dense oracle timed on the host cores over a bounded sample of (b, h) slabs."""
    import torch
    from oracle.dense_oracle import attention_dense_fp32, prefix_mask

    B, H, S, D = w.q.shape
    m = w.block_mask
    per_block = 4.0 * m.Q_BLOCK_SIZE * m.KV_BLOCK_SIZE * D
    slabs = [(b, h) for h in range(H) for b in range(B)]
    done, flops = 0, 0.0
    t0 = time.perf_counter()
    for b, h in slabs:
        attention_dense_fp32(w.q[b, h], w.k[b, h], w.v[b, h], prefix_mask(w.prefix_len[b], S))
        flops += per_block * float(m.kv_num_blocks[b, h].sum().item())
        done += 1
        if time.perf_counter() - t0 >= budget_s:
            break
    dt = time.perf_counter() - t0
    return {
        "value": flops / dt / 1e12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{done} of {B * H} (batch, head) slabs of the same workload, dense fp32 "
                  f"[S,S] scores per slab, {dt:.1f} s; effective flops of those slabs / time",
        "ms_per_slab": dt / done * 1e3,
    }


def band_sweep(dev, steps, warmup):
    """Kernel time against the number of listed blocks at the fixed shape of c2_interleaved
    (B=2, H=32, S=4096, D=128, bf16, 128/128): banded masks, query block i lists the FULL
    blocks max(0, i-w+1) .. i, for band widths w = 1, 2, 4, ... Tk.  Least-squares fit
    t = a + b * N_ne; returns the fit and the points."""
    import torch

    import omni_attn_capi

    B, H, S, D, QB, KB = 2, 32, 4096, 128, 128, 128
    Tq, Tk = S // QB, S // KB
    g = torch.Generator(device="cpu").manual_seed(0)
    q, k, v = (torch.randn(B, H, S, D, generator=g).to(torch.bfloat16).to(dev) for _ in range(3))
    o = torch.empty_like(q)
    stream = torch.cuda.current_stream(dev)
    points = []
    # settle the shader clock first (dense mask, some tens of milliseconds of load)
    nb_w = torch.full((B, H, Tq), Tk, dtype=torch.int32, device=dev)
    idx_w = torch.arange(Tk, dtype=torch.int32).expand(B, H, Tq, Tk).contiguous().to(dev)
    tys_w = torch.full((B, H, Tq, Tk), 2, dtype=torch.int32, device=dev)
    for _ in range(100):
        omni_attn_capi.fwd(q, k, v, o, None, nb_w, idx_w, tys_w, QB, KB, S, None, None,
                           stream=stream.cuda_stream)
    torch.cuda.synchronize()
    w = 1
    while w <= Tk:
        nb = torch.zeros(Tq, dtype=torch.int32)
        idx = torch.zeros(Tq, Tk, dtype=torch.int32)
        for i in range(Tq):
            lo = max(0, i - w + 1)
            nb[i] = i - lo + 1
            idx[i, : i - lo + 1] = torch.arange(lo, i + 1, dtype=torch.int32)
        tys = torch.full((Tq, Tk), 2, dtype=torch.int32)
        nb_d = nb.expand(B, H, Tq).contiguous().to(dev)
        idx_d = idx.expand(B, H, Tq, Tk).contiguous().to(dev)
        tys_d = tys.expand(B, H, Tq, Tk).contiguous().to(dev)

        def step():
            omni_attn_capi.fwd(q, k, v, o, None, nb_d, idx_d, tys_d, QB, KB, S, None, None,
                               stream=stream.cuda_stream)

        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
        ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
        for i in range(steps):
            starts[i].record(stream)
            step()
            ends[i].record(stream)
        torch.cuda.synchronize()
        ms = statistics.median(a.elapsed_time(b) for a, b in zip(starts, ends))
        n_ne = int(nb.sum()) * B * H
        points.append({"band_blocks": w, "nonempty_blocks": n_ne, "kernel_ms_median": ms,
                       "tflops": 4.0 * QB * KB * D * n_ne / (ms * 1e-3) / 1e12})
        w *= 2
    xs = [p["nonempty_blocks"] for p in points]
    ys = [p["kernel_ms_median"] for p in points]
    n = len(xs)
    mx, my = sum(xs) / n, sum(ys) / n
    sxx = sum((x - mx) ** 2 for x in xs)
    sxy = sum((x - mx) * (y - my) for x, y in zip(xs, ys))
    b = sxy / sxx
    a = my - b * mx
    ss_res = sum((y - (a + b * x)) ** 2 for x, y in zip(xs, ys))
    ss_tot = sum((y - my) ** 2 for y in ys)
    return {
        "sweep": "banded FULL masks, B=2 H=32 S=4096 D=128 bf16, Q_BLOCK=KV_BLOCK=128",
        "fit": {"ms_fixed": a, "ns_per_block": b * 1e6, "r2": 1.0 - ss_res / ss_tot,
                "max_rel_residual": max(abs(y - (a + b * x)) / y for x, y in zip(xs, ys))},
        "points": points,
    }


def fixed_cost_study(dev, seed, steps, warmup):
    """Where the time of c2_interleaved goes besides the per-block work: the same launch with
    every list repeated 2x and 3x (same workgroups, 2x / 3x the steps: r*T1 - Tr is r - 1 times the
    part that does not grow with the lists), with all block types FULL (no mask work), with the
    same number of blocks spread evenly over the query blocks (no imbalance), and the dense and
    plain causal controls of the same shape.  Kernel times are medians of HIP-event brackets."""
    import torch

    import omni_attn_capi
    from baseline_configs import make_workload

    w = make_workload("c2_interleaved", seed=seed)
    m = w.block_mask
    B, H, S, D = w.q.shape
    QB, KB = m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE
    q, k, v = (t.to(dev) for t in (w.q, w.k, w.v))
    o = torch.empty_like(q)
    lse = torch.empty(B, H, S, dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream(dev)
    per_block = 4.0 * QB * KB * D
    nb0, idx0, tys0 = m.kv_num_blocks, m.kv_indices, m.block_mask_types
    Tq, MB = nb0.shape[2], idx0.shape[3]

    def run(nb, idx, tys, what):
        nbd, idxd, tysd = (t.to(dev).contiguous() for t in (nb, idx, tys))

        def step():
            omni_attn_capi.fwd(q, k, v, o, lse, nbd, idxd, tysd, QB, KB, S, None, None, stream=stream.cuda_stream)

        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        st = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
        en = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
        for i in range(steps):
            st[i].record(stream)
            step()
            en[i].record(stream)
        torch.cuda.synchronize()
        ms = statistics.median(a.elapsed_time(b) for a, b in zip(st, en))
        blocks = int(nb.sum().item())
        return {"case": what, "listed_blocks": blocks, "kernel_us": ms * 1e3,
                "tflops": per_block * blocks / (ms * 1e-3) / 1e12, "ns_per_block": ms * 1e6 / blocks}

    t_end = time.perf_counter() + 0.25  # settle the clock under this load
    nbd, idxd, tysd = (t.to(dev) for t in (nb0, idx0, tys0))
    while time.perf_counter() < t_end:
        for _ in range(10):
            omni_attn_capi.fwd(q, k, v, o, lse, nbd, idxd, tysd, QB, KB, S, None, None, stream=stream.cuda_stream)
        torch.cuda.synchronize()
    rows = [run(nb0, idx0, tys0, "c2_interleaved as it is")]
    T1 = rows[0]["kernel_us"]
    ar = torch.arange(MB * 3)
    for r in (2, 3):
        idx = torch.zeros(B, H, Tq, MB * r, dtype=torch.int32)
        tys = torch.zeros(B, H, Tq, MB * r, dtype=torch.int32)
        for b in range(B):
            src = (ar[: MB * r].view(1, -1) % nb0[b, 0].clamp(min=1).view(-1, 1)).long()
            idx[b] = torch.gather(idx0[b, 0], 1, src).unsqueeze(0).expand(H, -1, -1)
            tys[b] = torch.gather(tys0[b, 0], 1, src).unsqueeze(0).expand(H, -1, -1)
        row = run(nb0 * r, idx, tys, f"every list repeated {r}x")
        row["fixed_us_estimate"] = (r * T1 - row["kernel_us"]) / (r - 1)
        rows.append(row)
    rows.append(run(nb0, idx0, torch.where(tys0 == 1, torch.full_like(tys0, 2), tys0), "all listed blocks FULL"))
    tot = int(nb0.sum().item())
    per = tot // (B * H * Tq)
    nbb = torch.full((B, H, Tq), per, dtype=torch.int32)
    nbb.view(-1)[: tot - per * B * H * Tq] += 1
    idxb = torch.arange(MB, dtype=torch.int32).expand(B, H, Tq, MB).contiguous()
    tysb = torch.full((B, H, Tq, MB), 2, dtype=torch.int32)
    rows.append(run(nbb, idxb, tysb, "same total, spread evenly over the query blocks"))
    rows.append(run(torch.full((B, H, Tq), MB, dtype=torch.int32), idxb, tysb, "dense control"))
    nbc = (torch.arange(Tq, dtype=torch.int32) + 1).expand(B, H, Tq).contiguous()
    tysc = tysb.clone()
    for i in range(Tq):
        tysc[:, :, i, i] = 1
    rows.append(run(nbc, idxb, tysc, "plain causal"))
    return {"study": "c2_interleaved: fixed cost, mask cost, imbalance (B=2 H=32 S=4096 D=128 bf16, 128/128)",
            "rows": rows}


def power_study(dev, seed, steps, warmup):
    """What the clock does to the figures.  (1) The library's matrix-instruction loop with eight
    operand sets, alone and with the forward kernel's LDS operand reads and softmax vector work
    beside it: rate and the shader clock one of its waves saw.  (2) The forward kernel on
    c2_interleaved with its real operands, with V zero and with all operands zero: the same
    instructions in the same order, but matrix cores and data paths that toggle fewer bits draw less
    power and the device grants a higher clock."""
    import torch

    import omni_attn_capi
    from baseline_configs import make_workload

    stream = torch.cuda.current_stream(dev)
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    ticks = torch.zeros(2, dtype=torch.int64, device=dev)
    names = {0: "mfma only, eight operand sets in turn", 1: "mfma + A operand from LDS",
             2: "mfma + softmax vector work", 3: "mfma + A operand from LDS + softmax vector work"}
    mixes = []
    for mix in range(4):
        iters = 20000
        t_end = time.perf_counter() + 0.25
        while time.perf_counter() < t_end:
            for _ in range(3):
                omni_attn_capi.mfma_mix_probe(mix, iters, sink, None, stream.cuda_stream)
            torch.cuda.synchronize()
        best = None
        for _ in range(3):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(stream)
            flops = omni_attn_capi.mfma_mix_probe(mix, iters, sink, ticks, stream.cuda_stream)
            b.record(stream)
            torch.cuda.synchronize()
            tf = flops / (a.elapsed_time(b) * 1e-3) / 1e12
            cyc, rt = (int(x) for x in ticks.tolist())
            if best is None or tf > best["tflops"]:
                best = {"mix": names[mix], "tflops": tf, "shader_clock_mhz": 100.0 * cyc / max(rt, 1),
                        "frac_of_rated_peak": tf / MFMA_PEAK_TFLOPS}
        best["mfma_busy_at_that_clock"] = best["tflops"] / (MFMA_PEAK_TFLOPS * best["shader_clock_mhz"] / 2400.0)
        mixes.append(best)

    w = make_workload("c2_interleaved", seed=seed)
    m = w.block_mask
    B, H, S, D = w.q.shape
    nb, idx, tys = (t.to(dev) for t in (m.kv_num_blocks, m.kv_indices, m.block_mask_types))
    o = torch.empty(w.q.shape, dtype=w.dtype, device=dev)
    lse = torch.empty(B, H, S, dtype=torch.float32, device=dev)
    rows = []
    for what in ("operands as in the benchmark (standard normal)", "V zero", "Q, K and V zero"):
        q, k, v = (t.to(dev) for t in (w.q, w.k, w.v))
        if what != "operands as in the benchmark (standard normal)":
            v = torch.zeros_like(v)
        if what == "Q, K and V zero":
            q, k = torch.zeros_like(q), torch.zeros_like(k)

        def step():
            omni_attn_capi.fwd(q, k, v, o, lse, nb, idx, tys, m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE, S, None, None,
                               stream=stream.cuda_stream)

        t_end = time.perf_counter() + 0.25
        while time.perf_counter() < t_end:
            for _ in range(10):
                step()
            torch.cuda.synchronize()
        st = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
        en = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
        for i in range(steps):
            st[i].record(stream)
            step()
            en[i].record(stream)
        torch.cuda.synchronize()
        ms = statistics.median(a.elapsed_time(b) for a, b in zip(st, en))
        tf = w.effective_flops / (ms * 1e-3) / 1e12
        rows.append({"operands": what, "kernel_us": ms * 1e3, "tflops": tf, "frac_of_rated_peak": tf / MFMA_PEAK_TFLOPS})
    return {"study": "clock under load: instruction mixes of the probe loop, and the forward kernel on "
                     "c2_interleaved (B=2 H=32 S=4096 D=128 bf16) with operands that toggle fewer bits",
            "probe_mixes": mixes, "forward_c2_interleaved": rows}


def issue_study(dev):
    """How much softmax vector work fits under a matrix instruction on one SIMD: the issue probe
    (one workgroup on one compute unit; groups of one bf16 32x32x16 MFMA + n v_fma_f32 + e v_exp_f32
    on registers of their own) at one and two waves per SIMD.  Cycles per group and SIMD; a matrix
    instruction alone takes 32."""
    import torch

    import omni_attn_capi

    ticks = torch.zeros(17, dtype=torch.int64, device=dev)
    iters = 2048
    rows = []
    for n_exp in (0, 1, 2):
        for n_plain in (0, 2, 4, 6, 8):
            row = {"v_fma_f32_per_mfma": n_plain, "v_exp_f32_per_mfma": n_exp}
            for waves in (1, 2):
                best = None
                for _ in range(3):
                    omni_attn_capi.issue_probe(n_plain, n_exp, waves, iters, ticks)
                    torch.cuda.synchronize()
                    t = ticks.tolist()
                    span = max(t[2 * w + 1] for w in range(4 * waves)) - min(t[2 * w] for w in range(4 * waves))
                    cyc = span / (4.0 * iters * waves)
                    best = cyc if best is None else min(best, cyc)
                row["cycles_per_group_per_simd_%dw" % waves] = best
            rows.append(row)
    return {"study": "vector work beside the matrix instructions of one SIMD (issue probe)", "rows": rows}


def extra_workload(name, seed, dev, steps, warmup, backward=False, settle_ms=150.0):
    """Kernel time of another workload, or of the backward of a workload (HIP events on the launch
    stream, after `settle_ms` of the same load)."""
    import torch

    import omni_attn_capi
    from baseline_configs import make_workload

    w = make_workload(name, seed=seed)
    m = w.block_mask
    B, H, S, D = w.q.shape
    q, k, v = (t.to(dev) for t in (w.q, w.k, w.v))
    o = torch.empty_like(q)
    lse = torch.empty(B, H, S, dtype=torch.float32, device=dev)
    nb, idx, tys = (t.to(dev) for t in (m.kv_num_blocks, m.kv_indices, m.block_mask_types))
    pidx = None if m.partial_block_mask_indices is None else m.partial_block_mask_indices.to(dev)
    pm = None if m.partial_block_masks is None else m.partial_block_masks.to(dev)
    stream = torch.cuda.current_stream(dev)

    def step():
        omni_attn_capi.fwd(q, k, v, o, lse, nb, idx, tys, m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE, S, pidx, pm,
                           stream=stream.cuda_stream)

    if backward:
        step()
        g = torch.Generator(device="cpu").manual_seed(seed + 1)
        dout = torch.randn(w.q.shape, generator=g).to(w.dtype).to(dev)
        dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
        ws = torch.empty(omni_attn_capi.load_library().omni_attn_bwd_workspace_bytes(B, H, S), dtype=torch.uint8,
                         device=dev)

        def step():  # noqa: F811
            omni_attn_capi.bwd(q, k, v, o, dout, lse, dq, dk, dv, nb, idx, tys, m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE,
                               S, pidx, pm, None, workspace=ws, stream=stream.cuda_stream)

    # the workload was built on the host while the GPU sat idle: bring the clock back under this
    # load before the counted launches (the main workload's settle phase, shorter)
    t_end = time.perf_counter() + settle_ms * 1e-3
    while settle_ms > 0 and time.perf_counter() < t_end:
        for _ in range(5):
            step()
        torch.cuda.synchronize()
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    for i in range(steps):
        starts[i].record(stream)
        step()
        ends[i].record(stream)
    torch.cuda.synchronize()
    ms = sum(a.elapsed_time(b) for a, b in zip(starts, ends)) / steps
    tf = w.effective_flops * (2.5 if backward else 1.0) / (ms * 1e-3) / 1e12
    out = {"workload": f"{name}: B={B} H={H} S={S} D={D}", "nonempty_blocks": w.nonempty_blocks,
           "kernel_ms_avg": ms, "tflops": tf, "frac": tf / MFMA_PEAK_TFLOPS}
    if backward:
        out["pass"] = "backward (dQ kernel + dK/dV kernel), 10*QB*KB*D flop per listed block"
    return out


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=100, help="untimed launches before the timed ones")
    ap.add_argument("--clock-settle-ms", type=float, default=250.0,
                    help="keep the GPU under the benchmark's own load for this long before the warm-up "
                         "launches (from idle the shader clock needs some tens of milliseconds to settle)")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the measured MFMA peak, the c2_interleaved_8k figure and the backward figure")
    ap.add_argument("--kernel-source-hash", action="store_true", help="print the hash and exit")
    ap.add_argument("--backward", action="store_true",
                    help="time the backward (dQ kernel + dK/dV kernel) instead of the forward; effective "
                         "flops are 10*QB*KB*D per listed block (five products)")
    ap.add_argument("--packed-tiles", action="store_true",
                    help="pack the PARTIAL tiles once with the pre-pass kernel and time the forward on "
                         "packed tiles; also reports the pre-pass kernel against the HBM roofline")
    ap.add_argument("--workload", default="c2_interleaved")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-budget-s", type=float, default=12.0)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 256 MiB device copy, so that a counter run of this "
                         "command shows what FETCH_SIZE / WRITE_SIZE read for a known traffic")
    ap.add_argument("--fixed-cost", action="store_true",
                    help="instead of the workload: c2_interleaved with its lists repeated, its types all "
                         "FULL, its blocks spread evenly (fixed cost / mask cost / imbalance of a launch)")
    ap.add_argument("--power-study", action="store_true",
                    help="instead of the workload: the probe loop with the forward kernel's LDS reads and "
                         "vector work beside the matrix instructions (rate and shader clock), and the forward "
                         "kernel with zero operands")
    ap.add_argument("--issue-study", action="store_true",
                    help="instead of the workload: cycles per matrix instruction and SIMD with 0..8 plain and "
                         "0..2 transcendental vector instructions issued beside each (one compute unit)")
    ap.add_argument("--sweep-bands", action="store_true",
                    help="instead of the workload: kernel time against the number of listed blocks")
    args = ap.parse_args(argv)
    if args.kernel_source_hash:
        print(kernel_source_hash())
        return 0
    if args.gpus != 1:
        print("bench.py measures one GPU: (batch, head) slabs are independent, so more GPUs would "
              "only run disjoint slices of the same kernel; run with --gpus 1.", file=sys.stderr)
        return 2

    import torch

    import omni_attn_capi
    from baseline_configs import make_workload

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 1
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    omni_attn_capi.load_library()  # fail loudly when the HIP library is missing
    if args.sweep_bands:
        print(json.dumps(band_sweep(dev, min(args.steps, 30), min(args.warmup, 5))))
        return 0
    if args.issue_study:
        print(json.dumps(issue_study(dev)))
        return 0
    if args.power_study:
        print(json.dumps(power_study(dev, args.seed, min(args.steps, 60), min(args.warmup, 10))))
        return 0
    if args.fixed_cost:
        print(json.dumps(fixed_cost_study(dev, args.seed, min(args.steps, 60), min(args.warmup, 10))))
        return 0

    w = make_workload(args.workload, seed=args.seed)
    m = w.block_mask
    B, H, S, D = w.q.shape
    q, k, v = (t.to(dev) for t in (w.q, w.k, w.v))
    o = torch.empty_like(q)
    lse = torch.empty(B, H, S, dtype=torch.float32, device=dev)
    nb, idx, tys = (t.to(dev) for t in (m.kv_num_blocks, m.kv_indices, m.block_mask_types))
    pidx = None if m.partial_block_mask_indices is None else m.partial_block_mask_indices.to(dev)
    pm = None if m.partial_block_masks is None else m.partial_block_masks.to(dev)
    stream = torch.cuda.current_stream(dev)

    bits = None
    pack_report = None
    if args.packed_tiles and pm is not None and pm.numel() > 0:
        bits = omni_attn_capi.pack_partial_masks(pm, stream.cuda_stream)
        torch.cuda.synchronize()
        # the pre-pass against the HBM roofline: bytes read + words written per launch
        reps = 50
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(10):
            omni_attn_capi.pack_partial_masks(pm, stream.cuda_stream)
        a.record(stream)
        for _ in range(reps):
            omni_attn_capi.pack_partial_masks(pm, stream.cuda_stream)
        b.record(stream)
        torch.cuda.synchronize()
        us = a.elapsed_time(b) * 1e3 / reps
        nbytes = pm.numel() + pm.numel() // 8
        pack_report = {"bound": "hbm", "achieved": nbytes / (us * 1e-6) / 1e9, "peak": 8000.0, "unit": "GB/s",
                       "frac": nbytes / (us * 1e-6) / 1e9 / 8000.0, "bytes_per_launch": nbytes,
                       "us_per_launch": us, "tiles": int(pm.shape[0]),
                       "note": "launch plus allocation of the output by the caller's allocator included"}

    bwd_state = None
    if args.backward:
        g = torch.Generator(device="cpu").manual_seed(args.seed + 1)
        dout = torch.randn(w.q.shape, generator=g).to(w.dtype).to(dev)
        omni_attn_capi.fwd(q, k, v, o, lse, nb, idx, tys, m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE, S, pidx,
                           None if bits is not None else pm, stream=stream.cuda_stream, partial_bits=bits)
        dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
        ws = torch.empty(omni_attn_capi.load_library().omni_attn_bwd_workspace_bytes(B, H, S), dtype=torch.uint8,
                         device=dev)
        bwd_state = (dout, dq, dk, dv, ws)

    def step():
        if bwd_state is not None:
            dout, dq, dk, dv, ws = bwd_state
            omni_attn_capi.bwd(q, k, v, o, dout, lse, dq, dk, dv, nb, idx, tys, m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE,
                               S, pidx, None if bits is not None else pm, bits, workspace=ws,
                               stream=stream.cuda_stream)
        elif bits is not None:
            omni_attn_capi.fwd(q, k, v, o, lse, nb, idx, tys, m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE, S, pidx, None,
                               stream=stream.cuda_stream, partial_bits=bits)
        else:
            omni_attn_capi.fwd(q, k, v, o, lse, nb, idx, tys, m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE, S, pidx, pm,
                               stream=stream.cuda_stream)

    # clock settle: the same launches, for a fixed time, not counted as warm-up or steps
    settle_launches = 0
    t_settle = time.perf_counter()
    while (time.perf_counter() - t_settle) * 1e3 < args.clock_settle_ms:
        for _ in range(10):
            step()
        settle_launches += 10
        torch.cuda.synchronize()
    settle_ms = (time.perf_counter() - t_settle) * 1e3

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    # timed region: exactly K steps, synchronised on both sides; events on the launch stream
    # bracket every launch so that the kernel's own duration is measured in the same region
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        starts[i].record(stream)
        step()
        ends[i].record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    if args.calibrate_copy:
        src = torch.ones(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()

    kernel_ms = [s.elapsed_time(e) for s, e in zip(starts, ends)]
    avg_kernel_ms = sum(kernel_ms) / len(kernel_ms)
    med_kernel_ms = statistics.median(kernel_ms)
    ms_per_step = wall / args.steps * 1e3
    flops = w.effective_flops * (2.5 if args.backward else 1.0)
    value = flops / (ms_per_step * 1e-3) / 1e12
    achieved = flops / (avg_kernel_ms * 1e-3) / 1e12
    traffic, traffic_provenance = traffic_for(args.workload)

    out = {
        "metric": METRIC,
        "value": value,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": {"bfloat16": "bf16", "float16": "f16"}.get(w.info["dtype"], w.info["dtype"]),
        "data": "synthetic",
        "config": {
            "workload": f"{w.name}: B={B} H={H} S={S} D={D} {w.info['dtype']}, Q_BLOCK={m.Q_BLOCK_SIZE} "
                        f"KV_BLOCK={m.KV_BLOCK_SIZE}, seed {args.seed}, image spans per batch element "
                        f"{[len(s) for s in w.spans]}",
            "nonempty_blocks": w.nonempty_blocks,
            "total_blocks": B * H * m.num_q_blocks * m.num_kv_blocks,
            "effective_gflop_per_step": flops / 1e9,
        },
        "clock_settle": {"ms": settle_ms, "launches": settle_launches},
        "pct_of_mfma_peak": 100.0 * value / MFMA_PEAK_TFLOPS,
        "kernel_ms_median": med_kernel_ms,
        "roofline": {
            "bound": "mfma",
            "achieved": achieved,
            "peak": MFMA_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved / MFMA_PEAK_TFLOPS,
            "traffic": traffic,
            "traffic_provenance": traffic_provenance,
            "kernel_ms_avg": avg_kernel_ms,
        },
    }
    if args.backward:
        out["config"]["pass"] = "backward (dQ kernel + dK/dV kernel), 10*QB*KB*D flop per listed block"
    if pack_report is not None:
        out["mask_pack"] = pack_report
        out["config"]["partial_tiles"] = "packed once by the pre-pass kernel"
    if not args.no_extras:
        dtype_code = omni_attn_capi.DTYPE_BF16 if w.dtype == torch.bfloat16 else omni_attn_capi.DTYPE_F16
        peak = measure_mfma_peak(dev, dtype_code)
        out["roofline"]["measured_mfma_peak"] = peak
        out["roofline"]["frac_of_measured_peak"] = achieved / peak
        if args.workload == "c2_interleaved":
            out["c2_interleaved_8k"] = extra_workload("c2_interleaved_8k", args.seed, dev, steps=args.steps,
                                                      warmup=max(args.warmup, 5))
            if not args.backward:
                out["c2_interleaved_backward"] = extra_workload("c2_interleaved", args.seed, dev,
                                                                steps=min(args.steps, 50), warmup=5, backward=True)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w, args.cpu_budget_s)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
