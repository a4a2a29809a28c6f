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
Extra fields of the line: `from_idle` (the same K steps with no settle phase), `operator` (host time
per call of the Python operator next to the bare C-ABI call and the kernel), `c2_interleaved_8k`,
`c2_interleaved_backward`.
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


def visited_pairs(m) -> int:
    """(query row, key) pairs the scalar-semantics kernel visits: all of a FULL or PARTIAL block, the
    keys up to the row's own position of a CAUSAL one."""
    import torch
    QB, KB = m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE
    nb = m.kv_num_blocks.cpu().long()
    slot = torch.arange(m.kv_indices.shape[-1]).view(1, 1, 1, -1)
    live = slot < nb.unsqueeze(-1)
    ty = m.block_mask_types.cpu().long()
    kv0 = m.kv_indices.cpu().long() * KB
    q0 = (torch.arange(nb.shape[2]) * QB).view(1, 1, -1, 1)
    rows = torch.arange(QB).view(1, 1, 1, 1, -1)
    causal = ((q0.unsqueeze(-1) + rows) - kv0.unsqueeze(-1) + 1).clamp(min=0, max=KB).sum(-1)
    per_slot = torch.where(ty == 1, causal, torch.full_like(causal, QB * KB))
    per_slot = torch.where(live & (ty != 0), per_slot, torch.zeros_like(per_slot))
    return int(per_slot.sum().item())


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


def operator_overhead(name, seed, dev, calls=200):
    """What the operator level adds to a launch: host time per call of omni_attention_shared_kv_swizzle
    (wrapper + module `omni_attn` + C ABI; the mask already on the GPU) and of the bare C-ABI call
    with preallocated output, both as the wall time of `calls` back-to-back asynchronous calls between
    two synchronisations, next to the kernel's own duration (HIP events)."""
    import torch

    import omni_attn_capi
    import omni_attn_torch
    from baseline_configs import make_workload

    w = make_workload(name, seed=seed)
    m = w.block_mask.to(dev)
    B, H, S, D = w.q.shape
    q, k, v = (t.to(dev) for t in (w.q, w.k, w.v))
    o = torch.empty_like(q)
    stream = torch.cuda.current_stream(dev)

    def op():
        return omni_attn_torch.omni_attention_shared_kv_swizzle(q, k, v, m)

    def capi():
        omni_attn_capi.fwd(q, k, v, o, None, m.kv_num_blocks, m.kv_indices, m.block_mask_types, m.Q_BLOCK_SIZE,
                           m.KV_BLOCK_SIZE, S, m.partial_block_mask_indices, m.partial_block_masks,
                           stream=stream.cuda_stream)

    def wall(fn):
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(calls):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t) / calls * 1e3

    t_end = time.perf_counter() + 0.1
    while time.perf_counter() < t_end:
        for _ in range(10):
            capi()
        torch.cuda.synchronize()
    op_ms, capi_ms = wall(op), wall(capi)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record(stream)
    for _ in range(calls):
        capi()
    b.record(stream)
    torch.cuda.synchronize()
    kernel_ms = a.elapsed_time(b) / calls
    return {"operator_ms_per_call": op_ms, "capi_ms_per_call": capi_ms, "kernel_ms": kernel_ms,
            "operator_minus_kernel_us": (op_ms - kernel_ms) * 1e3,
            "what": "omni_attention_shared_kv_swizzle(query, key, value, block_mask) vs omni_attn_fwd_gfx950"}


# The reference's published grid (omni-attn-mma/logs/printed_mask.md:186-237): B=1, H=8, head_dim 64,
# fp16, sequence / block size as below; the figures are its swizzle kernel's "TFLOPS" on an NVIDIA
# GPU it does not name -- context, not a baseline for this metric.
REFERENCE_GRID_PUBLISHED = {
    "causal": {(512, 64): 4.57, (512, 128): 4.35, (1024, 64): 14.39, (1024, 128): 12.47,
               (2048, 64): 31.69, (2048, 128): 32.27},
    "interleaved": {(512, 64): 4.62, (512, 128): 3.38, (1024, 64): 13.19, (1024, 128): 12.24,
                    (2048, 64): 28.17, (2048, 128): 33.60},
}


def reference_dense_flops(B: int, H: int, N: int, D: int) -> float:
    """The flop count behind the reference's "TFLOPS": every one of the N x N score positions,
    softmax and scaling included, whatever the mask leaves out
    (omni-attn-mma/test_with_debug_data.py:35-54, compute_dense_attn_tflops)."""
    qk = B * H * N * N * (2 * D - 1)
    softmax = B * H * N * (N - 1) + 3 * B * H * N * N + B * H * N * (N - 1)
    scaling = B * H * N * N
    pv = B * H * N * D * (2 * N - 1)
    return float(qk + softmax + scaling + pv)


def reference_grid(dev, seed: int):
    """The shapes of the reference's published table, timed the reference's way -- one wall-clock
    sample around a call of the swizzle wrapper plus a synchronise, after one untimed call
    (test_with_debug_data.py:152-162) -- and with HIP events around the kernel (median of 30)."""
    import torch

    import omni_attn_capi
    import omni_attn_torch as oat

    B, H, D = 1, 8, 64
    rows = []
    for kind in ("causal", "interleaved"):
        for S in (512, 1024, 2048):
            for blk in (64, 128):
                gen = torch.Generator().manual_seed(seed)
                q, k, v = (torch.randn(B, H, S, D, generator=gen).to(torch.float16).to(dev) for _ in range(3))
                if kind == "causal":
                    m = oat.create_causal_omni_block_mask(B, H, S, S, blk, blk, device=dev)
                else:  # three segments: text, an image span that ends off the block grid, text
                    pos = torch.tensor([[[0, S // 4, S // 4 + S // 8 + 5]]], dtype=torch.int64)
                    m = oat.create_omni_block_mask_from_modality_positions(pos, B, H, S, S, blk, blk, device=dev)
                oat.omni_attention_shared_kv_swizzle(q, k, v, m)
                torch.cuda.synchronize()
                t0 = time.time()
                oat.omni_attention_shared_kv_swizzle(q, k, v, m)
                torch.cuda.synchronize()
                wall_ms = (time.time() - t0) * 1e3
                o = torch.empty_like(q)
                stream = torch.cuda.current_stream(dev)

                def launch():
                    omni_attn_capi.fwd(q, k, v, o, None, m.kv_num_blocks, m.kv_indices, m.block_mask_types, blk, blk,
                                       S, m.partial_block_mask_indices, m.partial_block_masks,
                                       stream=stream.cuda_stream)

                for _ in range(20):
                    launch()
                ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(30)]
                for a, b in ev:
                    a.record(stream)
                    launch()
                    b.record(stream)
                torch.cuda.synchronize()
                kernel_ms = sorted(a.elapsed_time(b) for a, b in ev)[15]
                dense = reference_dense_flops(B, H, S, D)
                listed = int(m.kv_num_blocks.sum().item())
                rows.append({"mask": kind, "seq_len": S, "block": blk, "listed_blocks": listed,
                             "wall_ms_one_call": wall_ms, "kernel_ms_median": kernel_ms,
                             "dense_equivalent_tflops_wall": dense / (wall_ms * 1e-3) / 1e12,
                             "dense_equivalent_tflops_kernel": dense / (kernel_ms * 1e-3) / 1e12,
                             "effective_tflops_kernel": 4.0 * blk * blk * D * listed / (kernel_ms * 1e-3) / 1e12,
                             "reference_published_swizzle_tflops": REFERENCE_GRID_PUBLISHED[kind][(S, blk)]})
    return {"grid": "the reference's published shapes: B=1 H=8 head_dim 64 fp16, seq_len / block as listed",
            "note": "dense-equivalent TFLOPS by the reference's formula (all N x N positions, softmax included); "
                    "the published figures are from an NVIDIA GPU the reference does not name",
            "rows": rows}


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=100, help="untimed launches before the timed ones")
    ap.add_argument("--clock-settle-ms", type=float, default=250.0,
                    help="keep the GPU under the benchmark's own load for this long before the warm-up "
                         "launches (from idle the shader clock needs some tens of milliseconds to settle)")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the measured MFMA peak, the c2_interleaved_8k figure, the backward figure and "
                         "the operator-level timing")
    ap.add_argument("--kernel-source-hash", action="store_true", help="print the hash and exit")
    ap.add_argument("--backward", action="store_true",
                    help="time the backward (dQ kernel + dK/dV kernel) instead of the forward; effective "
                         "flops are 10*QB*KB*D per listed block (five products)")
    ap.add_argument("--generic-kernel", action="store_true",
                    help="time the scalar-semantics forward (any block size, head_dim <= 256) instead of the MFMA "
                         "kernel; adds its key-row traffic per launch and the rate it is read at")
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
    ap.add_argument("--sweep-bands", action="store_true",
                    help="instead of the workload: kernel time against the number of listed blocks")
    ap.add_argument("--reference-grid", action="store_true",
                    help="instead of the workload: the shapes of the reference's published table, timed its way")
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
    if args.reference_grid:
        print(json.dumps(reference_grid(dev, args.seed)))
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
        # the same kernel where it is bound by HBM and not by the launch: 65536 random tiles of this
        # workload's shape, more than the 256 MB of last-level cache hold (kernel time from events,
        # output preallocated through the raw entry point)
        NBIG = 65536
        big = torch.rand(NBIG, pm.shape[1], pm.shape[2], device=dev) < 0.5
        words = torch.empty(NBIG, pm.shape[1], pm.shape[2] // 32, dtype=torch.int32, device=dev)
        lib = omni_attn_capi.load_library()

        def pack_big():
            rc = lib.omni_attn_pack_partial_masks_gfx950(big.data_ptr(), words.data_ptr(), NBIG, pm.shape[1],
                                                         pm.shape[2], stream.cuda_stream)
            assert rc == 0, rc

        for _ in range(5):
            pack_big()
        a.record(stream)
        for _ in range(20):
            pack_big()
        b.record(stream)
        torch.cuda.synchronize()
        us_big = a.elapsed_time(b) * 1e3 / 20
        nbytes_big = big.numel() + big.numel() // 8
        pack_report["large"] = {"tiles": NBIG, "bytes_per_launch": nbytes_big, "us_per_launch": us_big,
                                "achieved": nbytes_big / (us_big * 1e-6) / 1e9, "unit": "GB/s",
                                "frac": nbytes_big / (us_big * 1e-6) / 1e9 / 8000.0}
        del big, words

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
        elif args.generic_kernel:
            omni_attn_capi.fwd(q, k, v, o, lse, nb, idx, tys, m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE, S, pidx, pm,
                               stream=stream.cuda_stream, generic=True)
        elif bits is not None:
            omni_attn_capi.fwd(q, k, v, o, lse, nb, idx, tys, m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE, S, pidx, None,
                               stream=stream.cuda_stream, partial_bits=bits)
        else:
            omni_attn_capi.fwd(q, k, v, o, lse, nb, idx, tys, m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE, S, pidx, pm,
                               stream=stream.cuda_stream)

    def timed_steps(n):
        """Wall time of exactly n launches between two synchronisations (nothing else is enqueued or
        recorded inside the region)."""
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(n):
            step()
        torch.cuda.synchronize()
        return time.perf_counter() - t

    # From idle: W warm-up launches and K timed ones straight after the uploads, before the GPU has
    # been under load for any length of time (the shader clock is still settling: reported beside the
    # headline, never as `value`).
    from_idle = None
    if args.clock_settle_ms > 0:
        for _ in range(args.warmup):
            step()
        wall_idle = timed_steps(args.steps)
        from_idle = {"ms_per_step": wall_idle / args.steps * 1e3, "steps": args.steps, "warmup": args.warmup}

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
    # timed region: exactly K bare launches, synchronised on both sides
    wall = timed_steps(args.steps)
    # the kernel's own duration: a second pass of the same K launches, each bracketed by events on
    # the launch stream (kept out of the host-timed region: two event records cost about 6 us a step)
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    for i in range(args.steps):
        starts[i].record(stream)
        step()
        ends[i].record(stream)
    torch.cuda.synchronize()

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
        "from_idle": None if from_idle is None else dict(
            from_idle, value=flops / (from_idle["ms_per_step"] * 1e-3) / 1e12,
            note="the same K steps after the same W warm-ups with no clock-settle phase before them"),
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
    if args.generic_kernel:
        # Every query row reads the K row (twice: maximum pass and weight pass) and the V row of every
        # key it visits; nothing is shared between rows except through the caches.
        pairs = visited_pairs(m)
        nbytes = pairs * 3 * D * 2
        out["config"]["kernel"] = "fwd_generic_kernel (one wave per query row, two passes, fp32)"
        out["generic_kernel"] = {"bound": "l2", "row_key_pairs": pairs, "algorithmic_bytes": nbytes,
                                 "achieved": nbytes / (avg_kernel_ms * 1e-3) / 1e9, "unit": "GB/s",
                                 "note": "K (two passes) and V rows per visited (query row, key) pair; served by "
                                         "L2 and L1, compulsory HBM bytes are 4*B*H*S*D*2"}
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
        out["operator"] = {name: operator_overhead(name, args.seed, dev) for name in ("c1_causal", "c2_interleaved")}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w, args.cpu_budget_s)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
