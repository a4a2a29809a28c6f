"""Parity of the gfx950 kernel with the CPU oracle, called through the C ABI.

Bars (written here, enforced in helpers.compare_with_oracle): max-abs on the output
2e-3 for fp16 and 1e-2 for bf16, 1e-3 on the logsumexp, rows with no allowed key
exactly 0 / -inf.  Inputs are rounded to the 16-bit type once; kernel and oracle see
the same rounded values.
"""
import os

import numpy as np
import pytest
import torch

import omni_attn_capi
from baseline_configs import make_workload
from helpers import (HERE, TOL_LSE, TOL_O, compare_with_oracle, random_block_metadata)
from oracle.block_walk import attention_block_walk
from oracle.dense_oracle import attention_dense_fp32, dense_mask_from_blocks, prefix_mask

pytestmark = pytest.mark.gpu


def _dev(t, device):
    return None if t is None else t.to(device).contiguous()


def run_kernel(q, k, v, nb, idx, tys, QB, KB, seqlen, pidx=None, pm=None, device="cuda:0",
               want_lse=True, stream=None):
    """One forward through the C ABI.  O and LSE start as NaN so that any element the
    kernel does not write shows up."""
    qd, kd, vd = (_dev(t, device) for t in (q, k, v))
    o = torch.full_like(qd, float("nan"))
    lse = torch.full(qd.shape[:3], float("nan"), dtype=torch.float32, device=device) if want_lse else None
    omni_attn_capi.fwd(qd, kd, vd, o, lse, _dev(nb, device), _dev(idx, device), _dev(tys, device), QB, KB,
                       seqlen, _dev(pidx, device), _dev(pm, device), stream=stream)
    torch.cuda.synchronize()
    return o, lse


def run_workload(w, device, **kw):
    m = w.block_mask
    return run_kernel(w.q, w.k, w.v, m.kv_num_blocks, m.kv_indices, m.block_mask_types, m.Q_BLOCK_SIZE,
                      m.KV_BLOCK_SIZE, w.q.shape[2], m.partial_block_mask_indices, m.partial_block_masks,
                      device=device, **kw)


def test_c1_causal_full_parity(gpu_device):
    w = make_workload("c1_causal", seed=0)
    o, lse = run_workload(w, gpu_device)
    S = 512
    ro, rl = attention_dense_fp32(w.q, w.k, w.v, prefix_mask(w.prefix_len, S).unsqueeze(1))
    compare_with_oracle(o, lse, ro, rl, torch.float16, "c1 vs dense oracle")
    m = w.block_mask
    wo, wl = attention_block_walk(w.q, w.k, w.v, m.kv_num_blocks, m.kv_indices, m.block_mask_types, 128, 128, S)
    compare_with_oracle(o, lse, wo, wl, torch.float16, "c1 vs block walk")
    gold = np.load(os.path.join(HERE, "golden", "c1_causal_seed0.npz"))
    assert abs(float(gold["q_checksum"]) - w.q.double().sum().item()) < 1e-9, "inputs differ from the fixture's"
    compare_with_oracle(o, lse, torch.from_numpy(gold["o"]), torch.from_numpy(gold["lse"]), torch.float16,
                        "c1 vs committed fixture")
    # causal row 0 attends key 0 only: O = V[0] bit for bit, lse = q0.k0/sqrt(D)
    assert torch.equal(o[0, :, 0].cpu(), w.v[0, :, 0])


def _merge_property(w, o, lse, device):
    """Size-independent check over every head at full size: attention over a block list
    equals the logsumexp-weighted merge of attention over its two halves."""
    m = w.block_mask
    nb = m.kv_num_blocks
    half = nb // 2
    max_blocks = m.kv_indices.shape[-1]
    slot = torch.arange(max_blocks).view(1, 1, 1, -1)
    # second half: shift the slots left by `half`
    src = (slot + half.unsqueeze(-1).long()).clamp(max=max_blocks - 1)
    def shifted(t):
        return None if t is None else torch.gather(t, -1, src).contiguous()
    QB, KB, S = m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE, w.q.shape[2]
    oa, la = run_kernel(w.q, w.k, w.v, half.contiguous(), m.kv_indices, m.block_mask_types, QB, KB, S,
                        m.partial_block_mask_indices, m.partial_block_masks, device=device)
    ob, lb = run_kernel(w.q, w.k, w.v, (nb - half).contiguous(), shifted(m.kv_indices),
                        shifted(m.block_mask_types), QB, KB, S, shifted(m.partial_block_mask_indices),
                        m.partial_block_masks, device=device)
    l_merged = torch.logaddexp(la, lb)
    wa = torch.exp(la - l_merged).nan_to_num(0.0).unsqueeze(-1)
    wb = torch.exp(lb - l_merged).nan_to_num(0.0).unsqueeze(-1)
    o_merged = wa * oa.float() + wb * ob.float()
    live = ~torch.isinf(lse)
    assert torch.equal(torch.isinf(l_merged), torch.isinf(lse))
    assert (l_merged[live] - lse[live]).abs().max().item() <= TOL_LSE
    # three roundings to the 16-bit type are involved instead of one
    assert (o_merged - o.float()).abs().max().item() <= 2 * TOL_O[w.dtype]


def _oracle_slabs(name, B, H):
    """(batch, head) slabs checked against the dense oracle.  The headline configurations
    (c2, its 8K variant, c3) are checked on every slab; the two largest ones on at least 8
    slabs that cover every distinct batch layout (heads of a batch element share their mask,
    so the slabs of one batch element differ in q/k/v only)."""
    if name in ("c2_interleaved", "c2_interleaved_8k", "c3_partial"):
        return [(b, h) for b in range(B) for h in range(H)]
    if name == "c4_long":
        return [(0, h) for h in range(0, H, 4)]                  # 8 of 32 heads, one layout
    if name == "c5_batched":
        return [(b, (5 * b + 1) % H) for b in range(B)]           # all 8 layouts, different heads
    return [(b, (3 * b) % H) for b in range(B)]                   # c5_full_control: 8 slabs


@pytest.mark.parametrize("name", ["c2_interleaved", "c2_interleaved_8k", "c3_partial", "c4_long",
                                  "c5_batched", "c5_full_control"])
def test_config_full_size(name, gpu_device):
    """Full-size run against the dense oracle (slabs: see _oracle_slabs), plus the merge
    property on all heads."""
    w = make_workload(name, seed=0)
    B, H, S, D = w.q.shape
    o, lse = run_workload(w, gpu_device)
    assert not torch.isnan(o).any() and not torch.isnan(lse).any()
    o_cpu, lse_cpu = o.cpu(), lse.cpu()
    masks = {}
    for b, h in _oracle_slabs(name, B, H):
        if b not in masks:
            masks = {b: prefix_mask(w.prefix_len[b], S)}
        ro, rl = attention_dense_fp32(w.q[b, h], w.k[b, h], w.v[b, h], masks[b])
        compare_with_oracle(o_cpu[b, h], lse_cpu[b, h], ro, rl, w.dtype, f"{name} slab ({b},{h})")
    _merge_property(w, o, lse, gpu_device)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("QB,KB", [(128, 128), (128, 64), (64, 128), (64, 64)])
def test_random_metadata_all_slot_kinds(dtype, D, QB, KB, gpu_device):
    """FULL / CAUSAL (on and off the diagonal) / PARTIAL with bits / PARTIAL without bits /
    MASKED slots, unordered kv_indices, empty query blocks, fully masked rows inside
    listed blocks, for every (Q_BLOCK, KV_BLOCK, head_dim, dtype) instance."""
    gen = torch.Generator().manual_seed(1000 * D + 10 * QB + KB)
    B, H, S = 2, 2, 512
    q, k, v = (torch.randn(B, H, S, D, generator=gen).to(dtype) for _ in range(3))
    nb, idx, tys, pidx, pm = random_block_metadata(gen, B, H, S // QB, S // KB, QB, KB, shuffle=True)
    for seqlen in (S, S - 45):
        o, lse = run_kernel(q, k, v, nb, idx, tys, QB, KB, seqlen, pidx, pm, device=gpu_device)
        dense = dense_mask_from_blocks(nb, idx, tys, QB, KB, S, S, pidx, pm, seqlen_orig=seqlen)
        ro, rl = attention_dense_fp32(q, k, v, dense)
        compare_with_oracle(o, lse, ro, rl, dtype, f"dense oracle seqlen={seqlen}")
        wo, wl = attention_block_walk(q, k, v, nb, idx, tys, QB, KB, seqlen, pidx, pm)
        compare_with_oracle(o, lse, wo, wl, dtype, f"block walk seqlen={seqlen}")
        assert (o[:, :, seqlen:] == 0).all()


def test_lse_pointer_is_optional(gpu_device):
    w = make_workload("c1_causal", seed=1)
    o1, _ = run_workload(w, gpu_device)
    o2, none = run_workload(w, gpu_device, want_lse=False)
    assert none is None and torch.equal(o1, o2)


def test_sequence_not_a_multiple_of_the_block(gpu_device):
    """S_pad = 500 handed to the C ABI as it is (Tq = ceil(500/128) = 4): loads are clamped,
    keys and rows beyond 500 do not exist."""
    gen = torch.Generator().manual_seed(11)
    S, D, QB, KB = 500, 64, 128, 64
    q, k, v = (torch.randn(1, 3, S, D, generator=gen).to(torch.bfloat16) for _ in range(3))
    from omni_attn_torch import create_causal_omni_block_mask
    m = create_causal_omni_block_mask(1, 3, S, S, QB, KB, device="cpu")
    o, lse = run_kernel(q, k, v, m.kv_num_blocks, m.kv_indices, m.block_mask_types, QB, KB, S, device=gpu_device)
    ro, rl = attention_dense_fp32(q, k, v, torch.tril(torch.ones(S, S, dtype=torch.bool)))
    compare_with_oracle(o, lse, ro, rl, torch.bfloat16, "ragged S")


def test_out_of_range_metadata_is_clamped(gpu_device):
    """kv_num_blocks beyond max_blocks and kv_indices beyond the last block are clamped."""
    gen = torch.Generator().manual_seed(12)
    S, D = 256, 64
    q, k, v = (torch.randn(1, 1, S, D, generator=gen).to(torch.float16) for _ in range(3))
    nb = torch.tensor([[[7, 2]]], dtype=torch.int32)            # max_blocks is 2
    idx = torch.tensor([[[[0, 99], [-5, 1]]]], dtype=torch.int32)
    tys = torch.full((1, 1, 2, 2), 2, dtype=torch.int32)
    o, lse = run_kernel(q, k, v, nb, idx, tys, 128, 128, S, device=gpu_device)
    nb2 = torch.tensor([[[2, 2]]], dtype=torch.int32)
    idx2 = torch.tensor([[[[0, 1], [0, 1]]]], dtype=torch.int32)
    o2, lse2 = run_kernel(q, k, v, nb2, idx2, tys, 128, 128, S, device=gpu_device)
    assert torch.equal(o, o2) and torch.equal(lse, lse2)


def test_partial_index_beyond_the_stored_tiles_skips_the_slot(gpu_device):
    """A PARTIAL slot whose index is >= the number of stored tiles has no bits: it is
    skipped like a negative index, and nothing beyond the tile array is read.  Tiles are
    laid out so that memory right behind the array is another, all-ones tensor: a kernel
    that read tile P would attend everything and differ from the expected result."""
    gen = torch.Generator().manual_seed(21)
    S, D, QB, KB = 512, 64, 128, 128
    q, k, v = (torch.randn(1, 2, S, D, generator=gen).to(torch.bfloat16) for _ in range(3))
    Tq = Tk = S // QB
    nb = torch.full((1, 2, Tq), Tk, dtype=torch.int32)
    idx = torch.arange(Tk, dtype=torch.int32).expand(1, 2, Tq, Tk).contiguous()
    tys = torch.full((1, 2, Tq, Tk), 3, dtype=torch.int32)
    tys[..., 0] = 2  # one FULL slot per row so that no row is empty
    P = 3
    tiles = torch.rand(P, QB, KB, generator=gen) < 0.5
    pidx = torch.randint(0, P, (1, 2, Tq, Tk), generator=gen, dtype=torch.int32)
    bad = pidx.clone()
    bad[0, 0, 1, 2] = P            # first index past the end
    bad[0, 1, 2, 1] = 1 << 20      # far past the end
    bad[0, 1, 3, 3] = 2 ** 31 - 1
    skip = pidx.clone()
    for pos in ((0, 0, 1, 2), (0, 1, 2, 1), (0, 1, 3, 3)):
        skip[pos] = -1
    backing = torch.ones(P + 4, QB, KB, dtype=torch.bool)  # tile P and beyond: all ones
    backing[:P] = tiles
    backing_d = backing.to(gpu_device)
    o_bad, lse_bad = run_kernel(q, k, v, nb, idx, tys, QB, KB, S, bad, backing_d[:P], device=gpu_device)
    o_skip, lse_skip = run_kernel(q, k, v, nb, idx, tys, QB, KB, S, skip, backing_d[:P], device=gpu_device)
    assert torch.equal(o_bad, o_skip) and torch.equal(lse_bad, lse_skip)
    wo, wl = attention_block_walk(q, k, v, nb, idx, tys, QB, KB, S, bad, tiles)
    compare_with_oracle(o_bad, lse_bad, wo, wl, torch.bfloat16, "out-of-range partial index")


def test_any_non_zero_mask_byte_means_attend(gpu_device):
    """partial_block_masks is read as bytes: the reference's kernels test `!mask[...]`
    (attn_naive.cu:151), so 2, 0x80 or 0xff attend like 1."""
    gen = torch.Generator().manual_seed(22)
    S, D, QB, KB = 256, 64, 128, 64
    q, k, v = (torch.randn(1, 1, S, D, generator=gen).to(torch.float16) for _ in range(3))
    Tq, Tk = S // QB, S // KB
    nb = torch.full((1, 1, Tq), Tk, dtype=torch.int32)
    idx = torch.arange(Tk, dtype=torch.int32).expand(1, 1, Tq, Tk).contiguous()
    tys = torch.full((1, 1, Tq, Tk), 3, dtype=torch.int32)
    pidx = torch.arange(Tq * Tk, dtype=torch.int32).view(1, 1, Tq, Tk)
    bits = torch.rand(Tq * Tk, QB, KB, generator=gen) < 0.6
    values = torch.tensor([1, 2, 4, 0x10, 0x80, 0xfe, 0xff, 3], dtype=torch.uint8)
    pick = torch.randint(0, len(values), bits.shape, generator=gen)
    as_bytes = torch.where(bits, values[pick], torch.zeros((), dtype=torch.uint8))
    o1, l1 = run_kernel(q, k, v, nb, idx, tys, QB, KB, S, pidx, bits, device=gpu_device)
    o2, l2 = run_kernel(q, k, v, nb, idx, tys, QB, KB, S, pidx, as_bytes, device=gpu_device)
    assert torch.equal(o1, o2) and torch.equal(l1, l2)
    wo, wl = attention_block_walk(q, k, v, nb, idx, tys, QB, KB, S, pidx, as_bytes)
    compare_with_oracle(o2, l2, wo, wl, torch.float16, "non-zero mask bytes")


def test_non_default_stream(gpu_device):
    w = make_workload("c1_causal", seed=2)
    o_ref, lse_ref = run_workload(w, gpu_device)
    s = torch.cuda.Stream(device=gpu_device)
    with torch.cuda.stream(s):
        o, lse = run_workload(w, gpu_device, stream=s.cuda_stream)
    s.synchronize()
    assert torch.equal(o, o_ref) and torch.equal(lse, lse_ref)


def test_runs_are_bitwise_reproducible(gpu_device):
    w = make_workload("c3_partial", seed=5, H=2, S=2048)
    a = run_workload(w, gpu_device)
    b = run_workload(w, gpu_device)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


@pytest.mark.parametrize("QB,KB,D", [(64, 64, 32), (128, 64, 64)])
def test_more_than_64_listed_blocks_per_query_block(QB, KB, D, gpu_device):
    """Lists longer than 64 and 128 blocks (the kernel keeps 64 blocks of metadata in
    registers and fetches the next 64 when the walk gets there), random slot kinds."""
    gen = torch.Generator().manual_seed(77 + D)
    B, H, S = 1, 2, 64 * 134
    dtype = torch.float16
    q, k, v = (torch.randn(B, H, S, D, generator=gen).to(dtype) for _ in range(3))
    nb, idx, tys, pidx, pm = random_block_metadata(gen, B, H, S // QB, S // KB, QB, KB, p_empty=0.05,
                                                   shuffle=True)
    assert int(nb.max()) > 128
    o, lse = run_kernel(q, k, v, nb, idx, tys, QB, KB, S - 10, pidx, pm, device=gpu_device)
    wo, wl = attention_block_walk(q, k, v, nb, idx, tys, QB, KB, S - 10, pidx, pm)
    compare_with_oracle(o, lse, wo, wl, dtype, "block walk, long lists")


def test_runtime_is_linear_in_listed_blocks(gpu_device):
    """Kernel time against the number of listed blocks at a fixed shape (banded masks of
    width 1, 2, 4 ... 32 blocks): a straight line, t = a + b * N_ne."""
    import bench

    r = bench.band_sweep(torch.device(gpu_device), steps=30, warmup=10)
    assert r["fit"]["r2"] > 0.98, r
    assert r["fit"]["ns_per_block"] > 0


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("gain", [4.0, 12.0])
def test_wide_score_range_moves_the_reference_often(dtype, gain, D, gpu_device):
    """Scores whose running maximum keeps jumping by far more than 2^6 (the kernel's
    lazy reference point has to move, and O and l have to be rescaled, on many steps),
    rows that stay without any allowed key for several steps, and very negative scores."""
    gen = torch.Generator().manual_seed(int(gain) * 7 + (dtype == torch.float16))
    B, H, S, QB, KB = 1, 3, 1536, 128, 128
    q = (torch.randn(B, H, S, D, generator=gen) * gain).to(dtype)
    k = torch.randn(B, H, S, D, generator=gen).to(dtype)
    v = torch.randn(B, H, S, D, generator=gen).to(dtype)
    k[:, 1] -= 0.5 * q[:, 1].float().mean(2, keepdim=True).to(dtype)  # head 1: mostly negative scores
    nb, idx, tys, pidx, pm = random_block_metadata(gen, B, H, S // QB, S // KB, QB, KB, p_empty=0.2,
                                                   shuffle=True)
    o, lse = run_kernel(q, k, v, nb, idx, tys, QB, KB, S, pidx, pm, device=gpu_device)
    wo, wl = attention_block_walk(q, k, v, nb, idx, tys, QB, KB, S, pidx, pm)
    # Peaked softmax rows return single V entries, up to |O| ~ 4.5, where rounding the output to
    # the 16-bit type alone costs up to half an ulp (bf16: 2^-9 relative = 0.016 at 4..8): the
    # absolute bar is widened by one ulp of the reference value; everything else as usual.
    o32, ref = o.float().cpu(), wo.float()
    assert torch.isfinite(o32).all()
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    excess = ((o32 - ref).abs() - ulp * ref.abs()).max().item()
    assert excess <= TOL_O[dtype], f"gain {gain}: max(|dO| - ulp|O|) = {excess:.3e}"
    empty = torch.isinf(wl) & (wl < 0)
    l32 = lse.float().cpu()
    assert torch.equal(torch.isinf(l32) & (l32 < 0), empty)
    assert (o32[empty] == 0).all()
    rel_l = ((l32[~empty] - wl[~empty]).abs() / wl[~empty].abs().clamp(min=1.0)).max().item()
    assert rel_l <= TOL_LSE, f"gain {gain}: LSE relative error {rel_l:.3e}"


def sparse_rows_bf16_case():
    """B=2 H=9 S=1152 D=128 128/128 bf16, standard-normal operands, 80 % of the blocks left out
    and shuffled lists: many rows attend one, two or a handful of keys, so outputs are single V
    entries of magnitude 2 .. 4.7 instead of averages near 0."""
    gen = torch.Generator().manual_seed(19073)
    B, H, S, D, QB, KB = 2, 9, 1152, 128, 128, 128
    q, k, v = (torch.randn(B, H, S, D, generator=gen).to(torch.bfloat16) for _ in range(3))
    meta = random_block_metadata(gen, B, H, S // QB, S // KB, QB, KB, p_empty=0.8, shuffle=True)
    return (q, k, v) + tuple(meta) + (QB, KB, S)


def two_rounding_bound(q, k, v, dense, dtype):
    """What the two roundings to the 16-bit type can cost an output element: the weights P are
    rounded before the PV product while the row sum keeps the unrounded ones (relative error u
    per weight: at most u * sum_j p_j |v_j| / l), and the result is rounded once more (u * |O|);
    u = 2^-8 for bf16 (8 significant bits), 2^-11 for fp16."""
    u = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    ref, _ = attention_dense_fp32(q, k, v, dense)
    mean_abs, _ = attention_dense_fp32(q, k, v.float().abs(), dense)
    return ref, u * (mean_abs + ref.abs()) + 1e-4


def test_bf16_error_on_rows_with_few_keys_is_the_two_roundings(gpu_device):
    """With bf16 the north-star bar of 1e-2 is an absolute one, and an output of magnitude 2 .. 4
    already moves by up to 2^-7 = 0.0078 when it is rounded to bf16; rounding P before the PV
    product (as the reference does, omni_attn_shared_kv.cu:450-453) adds up to 2^-8 * |V|.  On this
    input the largest deviation is 0.0114 (row 634 of slab (0, 2): keys 949 and 964, weights 0.0745
    and 0.9255, V = 0.516 and -2.781; the walk meets the small weight first, so the large one is
    12.416 -> 12.4375 in bf16 against a row sum of 13.416: -2.53999, which rounds to -2.546875;
    fp32 gives -2.535505).  Asserted: every element within the bound of the two roundings; the
    plain bar wherever that bound is below it; LSE and empty rows as everywhere."""
    q, k, v, nb, idx, tys, pidx, pm, QB, KB, S = sparse_rows_bf16_case()
    o, lse = run_kernel(q, k, v, nb, idx, tys, QB, KB, S, pidx, pm, device=gpu_device)
    dense = dense_mask_from_blocks(nb, idx, tys, QB, KB, S, S, pidx, pm, seqlen_orig=S)
    ref, bound = two_rounding_bound(q, k, v, dense, torch.bfloat16)
    _, rl = attention_dense_fp32(q, k, v, dense)
    o32, l32 = o.float().cpu(), lse.float().cpu()
    err = (o32 - ref).abs()
    assert (err <= bound).all(), f"max excess over the rounding bound {(err - bound).max().item():.3e}"
    inside = bound <= TOL_O[torch.bfloat16]
    assert inside.float().mean().item() > 0.9 and err[inside].max().item() <= TOL_O[torch.bfloat16]
    assert err.max().item() <= TOL_O[torch.bfloat16] + 2.0 ** -8 * v.float().abs().max().item()
    empty = torch.isinf(rl) & (rl < 0)
    assert torch.equal(torch.isinf(l32) & (l32 < 0), empty) and (o32[empty] == 0).all()
    assert (l32[~empty] - rl[~empty]).abs().max().item() <= TOL_LSE


def test_the_forward_can_be_captured_in_a_graph(gpu_device):
    """No entry point allocates or keeps state: a captured launch replays with new contents
    of the same buffers.  Replays are interleaved with eager work and synchronisations and
    every replay is checked against the eager result."""
    w = make_workload("c3_partial", seed=11, H=2, S=1024)
    m = w.block_mask
    dev = gpu_device
    q, k, v = (t.to(dev).clone() for t in (w.q, w.k, w.v))
    o = torch.zeros_like(q)
    lse = torch.zeros(q.shape[:3], dtype=torch.float32, device=dev)
    nb, idx, tys, pidx, pm = (t.to(dev).contiguous() for t in (m.kv_num_blocks, m.kv_indices, m.block_mask_types,
                                                                m.partial_block_mask_indices, m.partial_block_masks))
    S = q.shape[2]

    def launch(stream_ptr=None):
        omni_attn_capi.fwd(q, k, v, o, lse, nb, idx, tys, m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE, S, pidx, pm,
                           stream=stream_ptr)

    launch()
    torch.cuda.synchronize()
    side = torch.cuda.Stream(device=dev)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        launch(side.cuda_stream)  # warm-up on the capture stream
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            launch(torch.cuda.current_stream(dev).cuda_stream)
    gen = torch.Generator().manual_seed(5)
    for rep in range(4):
        q.copy_(torch.randn(q.shape, generator=gen).to(q.dtype))
        k.copy_(torch.randn(k.shape, generator=gen).to(k.dtype))
        torch.cuda.synchronize()
        o.fill_(float("nan"))
        lse.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        o_graph, lse_graph = o.clone(), lse.clone()
        o.fill_(float("nan"))
        launch()
        torch.cuda.synchronize()
        assert torch.equal(o_graph, o) and torch.equal(lse_graph, lse), f"replay {rep}"
