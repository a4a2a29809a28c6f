#!/usr/bin/env python3
"""Console check of the five operator entry points on one workload, in the shape of the
reference's fixed-data script (omni-attn-mma/test_with_debug_data.py:317-369): every entry
point is run on the same Q/K/V and block mask, compared with dense PyTorch attention on the
GPU, and reported as PASSED / FAILED with its time and TFLOPS.

Differences from the reference script:
  * the data is a tensor-only fixture (safetensors: q, k, v, the block-mask tensors and five
    integers) or one of the seeded workloads of baseline_configs -- no pickled objects
    (the reference stores a pickled OmniBlockMask, generate_debug_data.py:127-140);
  * next to the dense-equivalent TFLOPS the reference prints (4*B*H*S*S*D / t,
    test_with_debug_data.py: compute_dense_attn_tflops) the effective TFLOPS over the
    listed blocks is shown, which is what the kernel actually computes;
  * the comparison kernel is dense PyTorch attention, not FlexAttention.

    python omni-attention_amd/console_harness.py --workload c1_causal
    python omni-attention_amd/console_harness.py --save-fixture /tmp/c1.safetensors --workload c1_causal
    python omni-attention_amd/console_harness.py --fixture /tmp/c1.safetensors

Per-kernel times from the profiler, for the same run:

    rocprofv3 --kernel-trace --stats --output-format csv -d /tmp/prof -o run \
        -- python3 omni-attention_amd/console_harness.py --workload c2_interleaved
    python omni-attention_amd/console_harness.py --rocprof-summary /tmp/prof
"""
import argparse
import os
import sys
import time

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
if HERE not in sys.path:
    sys.path.insert(0, HERE)

import omni_attn_torch as oat  # noqa: E402
from omni_attn_torch import OmniBlockMask  # noqa: E402

ENTRY_POINTS = (
    ("Simple", "omni_attention_simple"),
    ("Cp_async", "omni_attention_cp_async"),
    ("Prefetch", "omni_attention_preftech"),
    ("Shared_kv", "omni_attention_shared_kv"),
    ("Swizzle", "omni_attention_shared_kv_swizzle"),
)


def save_fixture(path, q, k, v, block_mask: OmniBlockMask, seq_len: int) -> None:
    """Tensor-only fixture: everything needed to rebuild the call, nothing executable."""
    from safetensors.torch import save_file

    m = block_mask
    tensors = {
        "q": q.contiguous().cpu(), "k": k.contiguous().cpu(), "v": v.contiguous().cpu(),
        "kv_num_blocks": m.kv_num_blocks.contiguous().cpu(),
        "kv_indices": m.kv_indices.contiguous().cpu(),
        "block_mask_types": m.block_mask_types.contiguous().cpu(),
        "ints": torch.tensor([m.q_len, m.kv_len, m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE, seq_len], dtype=torch.int64),
    }
    if m.partial_block_mask_indices is not None and m.partial_block_masks is not None:
        tensors["partial_block_mask_indices"] = m.partial_block_mask_indices.contiguous().cpu()
        tensors["partial_block_masks"] = m.partial_block_masks.to(torch.uint8).contiguous().cpu()
    save_file(tensors, path)


def load_fixture(path):
    from safetensors.torch import load_file

    t = load_file(path)
    q_len, kv_len, QB, KB, seq_len = (int(x) for x in t["ints"])
    pidx = t.get("partial_block_mask_indices")
    pm = t.get("partial_block_masks")
    m = OmniBlockMask(kv_num_blocks=t["kv_num_blocks"], kv_indices=t["kv_indices"],
                      block_mask_types=t["block_mask_types"], q_len=q_len, kv_len=kv_len,
                      Q_BLOCK_SIZE=QB, KV_BLOCK_SIZE=KB, partial_block_mask_indices=pidx,
                      partial_block_masks=None if pm is None else pm.bool())
    return t["q"], t["k"], t["v"], m, seq_len


def _time_gpu(fn, warmup: int, iters: int) -> float:
    """Seconds per call: events on the current stream around `iters` calls."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e-3 / iters


def run(q, k, v, block_mask: OmniBlockMask, device="cuda:0", warmup=3, iters=10, out=sys.stdout):
    """Runs every entry point; returns {label: (passed, seconds)}."""
    q, k, v = (t.to(device) for t in (q, k, v))
    m = block_mask.to(device)
    B, H, S, D = q.shape
    listed = int(m.kv_num_blocks.sum())
    eff_flops = 4.0 * m.Q_BLOCK_SIZE * m.KV_BLOCK_SIZE * D * listed
    dense_flops = 4.0 * B * H * S * S * D
    atol = 2e-3 if q.dtype == torch.float16 else 1e-2

    print(f"Q shape: {tuple(q.shape)} {q.dtype}; blocks {m.Q_BLOCK_SIZE}/{m.KV_BLOCK_SIZE}; "
          f"listed blocks {listed}; Sparsity: {m.sparsity():.4f}", file=out)
    # dense reference in fp32 on the same (already rounded) inputs; rows without any allowed key
    # give NaN in the dense form and 0 in the kernels, as in the reference's kernels
    score_mask = m.to_score_mask()[..., :S, :S]
    t0 = time.perf_counter()
    ref = oat.naive_attention_with_dense_mask(q.float(), k.float(), v.float(), score_mask)
    torch.cuda.synchronize()
    ref_time = time.perf_counter() - t0
    ref = torch.nan_to_num(ref, nan=0.0)

    results = {}
    for label, fn_name in ENTRY_POINTS:
        fn = getattr(oat, fn_name)
        try:
            o = fn(q, k, v, m)
            passed = oat.check_correctness(ref, o, rtol=0.0, atol=atol, name=fn_name)
            secs = _time_gpu(lambda: fn(q, k, v, m), warmup, iters)
        except Exception as e:  # the console shape of the reference: report and go on
            print(f"✗ Error in {fn_name}: {e}", file=out)
            passed, secs = False, float("nan")
        results[label] = (passed, secs)

    print("=" * 60, file=out)
    for label, (passed, secs) in results.items():
        print(f"  {label}: {'PASSED' if passed else 'FAILED'}, time: {secs * 1e3:.3f}ms, "
              f"TFLOPS: {dense_flops / secs / 1e12:.2f} dense-equivalent, "
              f"{eff_flops / secs / 1e12:.2f} effective, speedup: {ref_time / secs:.1f}x", file=out)
    print(f"  Dense PyTorch fp32: time: {ref_time * 1e3:.3f}ms, TFLOPS: {dense_flops / ref_time / 1e12:.2f}",
          file=out)
    return results


def rocprof_summary(path, out=sys.stdout, top=12):
    """Print the per-kernel table of a `rocprofv3 --kernel-trace --stats --output-format csv` run:
    ``path`` is a `*_kernel_stats.csv` file or a directory that holds some (searched recursively).
    Returns the rows as (name, calls, average microseconds, percent of the traced kernel time)."""
    import csv
    import glob

    files = [path] if os.path.isfile(path) else sorted(
        glob.glob(os.path.join(path, "**", "*kernel_stats.csv"), recursive=True))
    if not files:
        raise FileNotFoundError(f"no *_kernel_stats.csv under {path}")
    rows = []
    for f in files:
        with open(f, newline="") as fh:
            for r in csv.DictReader(fh):
                rows.append((r["Name"], int(r["Calls"]), float(r["AverageNs"]) * 1e-3, float(r["TotalDurationNs"])))
    total = sum(r[3] for r in rows) or 1.0
    rows.sort(key=lambda r: -r[3])
    print(f"rocprofv3 kernel summary ({len(files)} file(s), {sum(r[1] for r in rows)} dispatches):", file=out)
    result = []
    for name, calls, avg_us, tot in rows[:top]:
        short = name if len(name) <= 72 else name[:69] + "..."
        print(f"  {100.0 * tot / total:6.2f}%  {calls:7d} x {avg_us:10.1f} us  {short}", file=out)
        result.append((name, calls, avg_us, 100.0 * tot / total))
    return result


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--workload", default="c1_causal")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--fixture", help="safetensors fixture to run instead of a workload")
    ap.add_argument("--save-fixture", help="write the workload as a safetensors fixture and exit")
    ap.add_argument("--iters", type=int, default=10)
    ap.add_argument("--rocprof-summary", metavar="PATH",
                    help="print the per-kernel table of a rocprofv3 --kernel-trace --stats csv run and exit")
    args = ap.parse_args(argv)

    if args.rocprof_summary:
        rocprof_summary(args.rocprof_summary)
        return 0

    if args.fixture:
        q, k, v, m, _ = load_fixture(args.fixture)
        print(f"Testing with data: {args.fixture} ...")
    else:
        from baseline_configs import make_workload

        w = make_workload(args.workload, seed=args.seed)
        q, k, v, m = w.q, w.k, w.v, w.block_mask
        if args.save_fixture:
            save_fixture(args.save_fixture, q, k, v, m, q.shape[2])
            print(f"wrote {args.save_fixture}")
            return 0
        print(f"Testing with workload: {args.workload} (seed {args.seed}) ...")
    if not torch.cuda.is_available():
        print("the console harness needs a GPU", file=sys.stderr)
        return 1
    results = run(q, k, v, m, iters=args.iters)
    return 0 if all(p for p, _ in results.values()) else 1


if __name__ == "__main__":
    sys.exit(main())
