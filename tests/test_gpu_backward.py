"""Parity of the backward kernels with autograd through the fp32 dense oracle, through the C ABI.

The reference has no backward and north_star states no bar for gradients.  The bars used here:
each gradient tensor is compared on the inputs the kernels saw (q, k, v, dO already rounded to
the 16-bit type), normalised by the largest reference entry of that tensor:
    max|d - d_ref| <= TOL * max(1, max|d_ref|),   TOL = 4e-3 (fp16), 3e-2 (bf16)
(the kernels round P and dS to the 16-bit type before the second products of a step, as the
forward rounds P: 2^-11 resp. 2^-8 relative per term).  Rows and keys beyond the sequence, and
keys nobody attends, get exactly zero.
"""
import pytest
import torch

import omni_attn_capi
from baseline_configs import make_workload
from helpers import random_block_metadata
from oracle.dense_oracle import (attention_dense_fp32, attention_dense_grads, attention_dense_grads_chunked,
                                 dense_mask_from_blocks, prefix_mask)

pytestmark = pytest.mark.gpu

TOL_GRAD = {torch.float16: 4e-3, torch.bfloat16: 3e-2}


def run_fwd_bwd(q, k, v, dout, nb, idx, tys, QB, KB, seqlen, pidx=None, pm=None, device="cuda:0", packed=False,
                softcap=0.0):
    dev = lambda t: None if t is None else t.to(device).contiguous()
    qd, kd, vd, dod = dev(q), dev(k), dev(v), dev(dout)
    nbd, idxd, tysd, pidxd, pmd = dev(nb), dev(idx), dev(tys), dev(pidx), dev(pm)
    bits = omni_attn_capi.pack_partial_masks(pmd) if (packed and pmd is not None) else None
    o = torch.full_like(qd, float("nan"))
    lse = torch.full(qd.shape[:3], float("nan"), dtype=torch.float32, device=device)
    if bits is not None:
        omni_attn_capi.fwd(qd, kd, vd, o, lse, nbd, idxd, tysd, QB, KB, seqlen, pidxd, None, partial_bits=bits,
                           softcap=softcap)
    else:
        omni_attn_capi.fwd(qd, kd, vd, o, lse, nbd, idxd, tysd, QB, KB, seqlen, pidxd, pmd, softcap=softcap)
    dq, dk, dv = (torch.full_like(qd, float("nan")) for _ in range(3))
    omni_attn_capi.bwd(qd, kd, vd, o, dod, lse, dq, dk, dv, nbd, idxd, tysd, QB, KB, seqlen, pidxd,
                       None if bits is not None else pmd, bits, softcap=softcap)
    torch.cuda.synchronize()
    return dq, dk, dv, o, lse


def check_grads(got, ref, dtype, what):
    for name, a, b in zip(("dQ", "dK", "dV"), got, ref):
        a = a.float().cpu()
        assert torch.isfinite(a).all(), f"{what}: non-finite {name}"
        err = (a - b).abs().max().item()
        bar = TOL_GRAD[dtype] * max(1.0, b.abs().max().item())
        assert err <= bar, f"{what}: max|d{name}| error {err:.3e} > {bar:.3e} (max|ref| {b.abs().max().item():.3f})"


def test_c1_causal_backward(gpu_device):
    w = make_workload("c1_causal", seed=0)
    m = w.block_mask
    gen = torch.Generator().manual_seed(100)
    dout = torch.randn(w.q.shape, generator=gen).to(w.dtype)
    S = w.q.shape[2]
    got = run_fwd_bwd(w.q, w.k, w.v, dout, m.kv_num_blocks, m.kv_indices, m.block_mask_types, 128, 128, S,
                      device=gpu_device)
    ref = attention_dense_grads(w.q, w.k, w.v, prefix_mask(w.prefix_len, S).unsqueeze(1), dout)
    check_grads(got[:3], ref, w.dtype, "c1")


@pytest.mark.parametrize("packed", [False, True], ids=["bytes", "bits"])
def test_c3_partial_shrunk_backward(packed, gpu_device):
    w = make_workload("c3_partial", seed=2, H=2, S=2048)
    m = w.block_mask
    gen = torch.Generator().manual_seed(101)
    dout = torch.randn(w.q.shape, generator=gen).to(w.dtype)
    S = w.q.shape[2]
    got = run_fwd_bwd(w.q, w.k, w.v, dout, m.kv_num_blocks, m.kv_indices, m.block_mask_types, m.Q_BLOCK_SIZE,
                      m.KV_BLOCK_SIZE, S, m.partial_block_mask_indices, m.partial_block_masks,
                      device=gpu_device, packed=packed)
    ref = attention_dense_grads(w.q, w.k, w.v, prefix_mask(w.prefix_len, S).unsqueeze(1), dout)
    check_grads(got[:3], ref, w.dtype, "c3 shrunk")


@pytest.mark.parametrize("softcap", [0.0, 2.0, 50.0], ids=["nocap", "cap2", "cap50"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("QB,KB", [(128, 128), (128, 64), (64, 128), (64, 64)])
def test_random_metadata_backward(dtype, D, QB, KB, softcap, gpu_device):
    """Every instance of both backward kernels, plain and soft-capped (byte tiles, every slot kind,
    a sequence that ends inside a block)."""
    gen = torch.Generator().manual_seed(7000 + 10 * D + QB + KB // 64)
    B, H, S = 2, 2, 512
    q, k, v, dout = (torch.randn(B, H, S, D, generator=gen).to(dtype) for _ in range(4))
    nb, idx, tys, pidx, pm = random_block_metadata(gen, B, H, S // QB, S // KB, QB, KB, shuffle=True)
    for seqlen in (S, S - 45):
        got = run_fwd_bwd(q, k, v, dout, nb, idx, tys, QB, KB, seqlen, pidx, pm, device=gpu_device, softcap=softcap)
        dense = dense_mask_from_blocks(nb, idx, tys, QB, KB, S, S, pidx, pm, seqlen_orig=seqlen)
        ref = attention_dense_grads(q, k, v, dense, dout, softcap=softcap)
        check_grads(got[:3], ref, dtype, f"random metadata seqlen={seqlen} softcap={softcap}")
        for t in got[:3]:
            assert (t[:, :, seqlen:] == 0).all(), "rows beyond the sequence must get zero gradients"


def test_padding_rows_are_never_read(gpu_device):
    """Rows at or beyond seqlen_orig of q, k, v and dO may hold anything (here NaN): the outputs
    are the same bits as with zeros there, finite everywhere and zero on the padding."""
    gen = torch.Generator().manual_seed(108)
    B, H, S, seqlen = 1, 3, 384, 300
    for dtype, D, QB, KB in ((torch.bfloat16, 128, 128, 128), (torch.float16, 64, 128, 64), (torch.bfloat16, 32, 64, 64)):
        q, k, v, dout = (torch.randn(B, H, S, D, generator=gen).to(dtype) for _ in range(4))
        nb, idx, tys, pidx, pm = random_block_metadata(gen, B, H, S // QB, S // KB, QB, KB, shuffle=True)
        clean = []
        for t in (q, k, v, dout):
            t[:, :, seqlen:] = 0
            clean.append(t.clone())
        ref = run_fwd_bwd(*clean, nb, idx, tys, QB, KB, seqlen, pidx, pm, device=gpu_device)
        for t in (q, k, v, dout):
            t[:, :, seqlen:] = float("nan")
        got = run_fwd_bwd(q, k, v, dout, nb, idx, tys, QB, KB, seqlen, pidx, pm, device=gpu_device)
        for name, a, b in zip(("dQ", "dK", "dV", "O", "LSE"), got, ref):
            assert name == "LSE" or torch.isfinite(a).all(), f"non-finite {name}"
            assert not torch.isnan(a).any() and torch.equal(a, b), f"{name} depends on the padding rows"
        for t in got[:4]:
            assert (t[:, :, seqlen:] == 0).all()


def test_sequences_of_length_zero_and_one(gpu_device):
    """seqlen_orig = 0: nothing is attended, everything is zero (LSE -inf).  seqlen_orig = 1: row 0
    attends key 0 alone, so O[0] = V[0], dV[0] = dO[0] and the softmax of one element has no
    gradient with respect to its score."""
    gen = torch.Generator().manual_seed(107)
    B, H, S, D = 1, 2, 256, 64
    q, k, v, dout = (torch.randn(B, H, S, D, generator=gen).to(torch.float16) for _ in range(4))
    nb = torch.tensor([[[1, 2]]] * 1, dtype=torch.int32).expand(B, H, 2).contiguous()
    idx = torch.tensor([[0, 0], [0, 1]], dtype=torch.int32).expand(B, H, 2, 2).contiguous()
    tys = torch.tensor([[1, 0], [2, 1]], dtype=torch.int32).expand(B, H, 2, 2).contiguous()
    dq, dk, dv, o, lse = run_fwd_bwd(q, k, v, dout, nb, idx, tys, 128, 128, 0, device=gpu_device)
    for t in (dq, dk, dv, o):
        assert (t == 0).all()
    assert (lse == float("-inf")).all()
    dq, dk, dv, o, lse = run_fwd_bwd(q, k, v, dout, nb, idx, tys, 128, 128, 1, device=gpu_device)
    assert torch.equal(o[:, :, 0].cpu(), v[:, :, 0]) and (o[:, :, 1:] == 0).all()
    assert torch.equal(dv[:, :, 0].cpu(), dout[:, :, 0]) and (dv[:, :, 1:] == 0).all()
    # (dP and delta are the same sum in two summation orders: zero up to fp32 rounding)
    assert dq.abs().max().item() <= 1e-3 and dk.abs().max().item() <= 1e-3
    assert (dq[:, :, 1:] == 0).all() and (dk[:, :, 1:] == 0).all()
    expect = (q[:, :, 0].float() * k[:, :, 0].float()).sum(-1) / 8.0
    assert (lse[:, :, 0].cpu() - expect).abs().max().item() <= 1e-3 and (lse[:, :, 1:] == float("-inf")).all()


def test_slab_counts_that_do_not_divide_over_the_xcds(gpu_device):
    """15 and 9 slabs: the kernels deal slabs to the 8 XCDs round-robin, so some XCDs get one slab
    more than others (forward and backward)."""
    for B, H in ((3, 5), (1, 9)):
        gen = torch.Generator().manual_seed(106 + B)
        S, D, QB, KB = 384, 64, 128, 128
        q, k, v, dout = (torch.randn(B, H, S, D, generator=gen).to(torch.bfloat16) for _ in range(4))
        nb, idx, tys, pidx, pm = random_block_metadata(gen, B, H, S // QB, S // KB, QB, KB, shuffle=True)
        got = run_fwd_bwd(q, k, v, dout, nb, idx, tys, QB, KB, S - 7, pidx, pm, device=gpu_device)
        dense = dense_mask_from_blocks(nb, idx, tys, QB, KB, S, S, pidx, pm, seqlen_orig=S - 7)
        check_grads(got[:3], attention_dense_grads(q, k, v, dense, dout), torch.bfloat16, f"{B * H} slabs")
        fwd_ref, _ = attention_dense_fp32(q, k, v, dense)
        assert (got[3].float().cpu() - fwd_ref).abs().max().item() <= 1e-2


def scattered_lists(gen, H, S, QB, KB, W):
    """Metadata of H heads whose lists are W slots wide, nearly all MASKED padding, with the real
    blocks (FULL, CAUSAL and PARTIAL, about three quarters of the KV blocks) at random slots."""
    Tq, Tk = S // QB, S // KB
    nb = torch.zeros(1, H, Tq, dtype=torch.int32)
    idx = torch.randint(0, Tk, (1, H, Tq, W), generator=gen, dtype=torch.int32)
    tys = torch.zeros(1, H, Tq, W, dtype=torch.int32)  # MASKED
    pidx = torch.full((1, H, Tq, W), -1, dtype=torch.int32)
    tiles = []
    for h in range(H):
        for qb in range(Tq):
            cols = [kb for kb in range(Tk) if torch.rand((), generator=gen).item() > 0.25]
            slots = sorted(torch.randperm(W, generator=gen)[:len(cols)].tolist())
            if qb == 1:
                slots[-1] = W - 1  # the last slot of the list
            if qb == 2 and len(slots) > 1:
                slots[0], slots[1] = 63, 64  # either side of a word boundary
            nb[0, h, qb] = W if qb != 3 else slots[-1] + 1
            for s, kb in zip(slots, cols):
                idx[0, h, qb, s] = kb
                ty = (2, 1, 3)[int(torch.randint(0, 3, (), generator=gen))]
                tys[0, h, qb, s] = ty
                if ty == 3:
                    pidx[0, h, qb, s] = len(tiles)
                    tiles.append(torch.rand(QB, KB, generator=gen) < 0.5)
    return nb, idx, tys, pidx, torch.stack(tiles).to(torch.uint8)


def test_wide_block_lists_backward(gpu_device):
    """Lists wider than 64 and 128 slots (most of them MASKED padding, the real blocks scattered over
    the whole width): the metadata of a query block then spans several 64-slot words, in the dQ
    kernel's register chunks and in the dK/dV kernel's match bitmap alike."""
    gen = torch.Generator().manual_seed(105)
    B, H, S, D, QB, KB, W = 1, 2, 512, 64, 128, 64, 150
    q, k, v, dout = (torch.randn(B, H, S, D, generator=gen).to(torch.float16) for _ in range(4))
    nb, idx, tys, pidx, pm = scattered_lists(gen, H, S, QB, KB, W)
    got = run_fwd_bwd(q, k, v, dout, nb, idx, tys, QB, KB, S, pidx, pm, device=gpu_device)
    dense = dense_mask_from_blocks(nb, idx, tys, QB, KB, S, S, pidx, pm, seqlen_orig=S)
    ref = attention_dense_grads(q, k, v, dense, dout)
    check_grads(got[:3], ref, torch.float16, "wide lists")
    fwd_ref, _ = attention_dense_fp32(q, k, v, dense)
    assert (got[3].float().cpu() - fwd_ref).abs().max().item() <= 2e-3


@pytest.mark.parametrize("dtype,D,QB,KB,S,W,windows", [
    (torch.bfloat16, 128, 128, 128, 2048, 64 * 400, 3),   # 16 x 400 = 6400 words, 2602 held at a time
    (torch.float16, 64, 64, 64, 1024, 64 * 300, 2),       # 16 x 300 = 4800 words, 4096 at a time
    (torch.float16, 128, 64, 64, 1024, 64 * 300, 2),
])
def test_metadata_beyond_one_bitmap_window(dtype, D, QB, KB, S, W, windows, gpu_device):
    """More 64-slot words of metadata per slab than the dK/dV kernel's match bitmap holds in LDS:
    the kernel scans and walks them window by window (the boundaries fall inside a query block's
    list), and the gradients are those of the same blocks in a narrow list."""
    gen = torch.Generator().manual_seed(115)
    H = 2
    words = (S // QB) * (W // 64)
    assert windows == -(-words // (2602 if (D, KB) == (128, 128) else 4096))
    q, k, v, dout = (torch.randn(1, H, S, D, generator=gen).to(dtype) for _ in range(4))
    nb, idx, tys, pidx, pm = scattered_lists(gen, H, S, QB, KB, W)
    got = run_fwd_bwd(q, k, v, dout, nb, idx, tys, QB, KB, S - 5, pidx, pm, device=gpu_device, softcap=0.0)
    dense = dense_mask_from_blocks(nb, idx, tys, QB, KB, S, S, pidx, pm, seqlen_orig=S - 5)
    check_grads(got[:3], attention_dense_grads(q, k, v, dense, dout), dtype, f"{words} words of metadata")
    fwd_ref, _ = attention_dense_fp32(q, k, v, dense)
    assert (got[3].float().cpu() - fwd_ref).abs().max().item() <= (1e-2 if dtype == torch.bfloat16 else 2e-3)
    # the same blocks packed to the front of a list one window holds: bit-identical gradients
    order = torch.argsort((tys == 0).to(torch.int8), dim=-1, stable=True)[..., :S // KB]
    narrow = [torch.gather(t, -1, order).contiguous() for t in (idx, tys, pidx)]
    nb2 = (tys != 0).sum(-1).to(torch.int32)
    got2 = run_fwd_bwd(q, k, v, dout, nb2, narrow[0], narrow[1], QB, KB, S - 5, narrow[2], pm, device=gpu_device)
    for name, a, b in zip(("dQ", "dK", "dV"), got[:3], got2[:3]):
        assert torch.equal(a, b), f"{name} differs between the wide and the narrow list"


def test_c2_full_size_backward_on_sampled_slabs(gpu_device):
    w = make_workload("c2_interleaved", seed=0)
    m = w.block_mask
    B, H, S, D = w.q.shape
    gen = torch.Generator().manual_seed(102)
    dout = torch.randn(w.q.shape, generator=gen).to(w.dtype)
    got = run_fwd_bwd(w.q, w.k, w.v, dout, m.kv_num_blocks, m.kv_indices, m.block_mask_types, 128, 128, S,
                      device=gpu_device)
    cpu = [t.float().cpu() for t in got[:3]]
    for b, h in ((0, 0), (1, 17), (1, 31)):
        mask = prefix_mask(w.prefix_len[b], S)
        ref = attention_dense_grads(w.q[b, h], w.k[b, h], w.v[b, h], mask, dout[b, h])
        check_grads([t[b, h] for t in cpu], ref, w.dtype, f"c2 slab ({b},{h})")


FULL_SIZE_SLABS = {
    "c3_partial": [(0, 0), (0, 5), (0, 10), (0, 15)],
    "c4_long": [(0, 0), (0, 9), (0, 18), (0, 27)],
    "c5_batched": [(b, (5 * b + 1) % 16) for b in range(8)],  # every batch layout
}


@pytest.mark.parametrize("name,packed", [("c3_partial", False), ("c3_partial", True), ("c4_long", False),
                                         ("c5_batched", False)],
                         ids=["c3_partial-bytes", "c3_partial-bits", "c4_long", "c5_batched"])
def test_config_full_size_backward_on_sampled_slabs(name, packed, gpu_device):
    """BASELINE configurations 3, 4 and 5 at full size: the whole backward runs on the GPU, sampled
    (batch, head) slabs are compared with the closed-form fp32 gradients of the dense oracle."""
    w = make_workload(name, seed=0)
    m = w.block_mask
    B, H, S, D = w.q.shape
    gen = torch.Generator().manual_seed(109)
    dout = torch.randn(w.q.shape, generator=gen).to(w.dtype)
    got = run_fwd_bwd(w.q, w.k, w.v, dout, m.kv_num_blocks, m.kv_indices, m.block_mask_types, m.Q_BLOCK_SIZE,
                      m.KV_BLOCK_SIZE, S, m.partial_block_mask_indices, m.partial_block_masks,
                      device=gpu_device, packed=packed)
    for t in got[:3]:
        assert torch.isfinite(t).all()
    for b, h in FULL_SIZE_SLABS[name]:
        mask = prefix_mask(w.prefix_len[b], S)
        ref = attention_dense_grads_chunked(w.q[b, h], w.k[b, h], w.v[b, h], mask, dout[b, h])
        check_grads([t[b, h] for t in got[:3]], ref, w.dtype, f"{name} slab ({b},{h})")


def test_duplicate_and_clamped_block_indices_backward(gpu_device):
    """The forward clamps block indices and visits a block as often as it is listed; the backward
    differentiates exactly that (a block listed twice counts twice in the softmax)."""
    gen = torch.Generator().manual_seed(103)
    S, D = 256, 64
    q, k, v, dout = (torch.randn(1, 1, S, D, generator=gen).to(torch.float16) for _ in range(4))
    nb = torch.tensor([[[2, 3]]], dtype=torch.int32)
    idx = torch.tensor([[[[0, 99, 0], [-5, 1, 1]]]], dtype=torch.int32)  # 99 -> 1, -5 -> 0; row 1 lists block 1 twice
    tys = torch.full((1, 1, 2, 3), 2, dtype=torch.int32)
    got = run_fwd_bwd(q, k, v, dout, nb, idx, tys, 128, 128, S, device=gpu_device)
    # reference: keys of a twice-listed block appear twice
    kk = torch.cat([k, k[:, :, 128:]], dim=2)
    vv = torch.cat([v, v[:, :, 128:]], dim=2)
    mask = torch.zeros(S, S + 128, dtype=torch.bool)
    mask[:128, :256] = True
    mask[128:, :] = True
    dq, dkk, dvv = attention_dense_grads(q[0, 0], kk[0, 0], vv[0, 0], mask, dout[0, 0])
    dk = dkk[:256].clone(); dk[128:] += dkk[256:]
    dv = dvv[:256].clone(); dv[128:] += dvv[256:]
    check_grads([t[0, 0] for t in got[:3]], (dq, dk, dv), torch.float16, "duplicates")


def test_backward_is_bitwise_reproducible_and_checks_its_workspace(gpu_device):
    w = make_workload("c3_partial", seed=5, H=2, S=1024)
    m = w.block_mask
    gen = torch.Generator().manual_seed(104)
    dout = torch.randn(w.q.shape, generator=gen).to(w.dtype)
    args = (w.q, w.k, w.v, dout, m.kv_num_blocks, m.kv_indices, m.block_mask_types, m.Q_BLOCK_SIZE,
            m.KV_BLOCK_SIZE, 1024, m.partial_block_mask_indices, m.partial_block_masks)
    a = run_fwd_bwd(*args, device=gpu_device)
    b = run_fwd_bwd(*args, device=gpu_device)
    for x, y in zip(a[:3], b[:3]):
        assert torch.equal(x, y)
    lib = omni_attn_capi.load_library()
    assert lib.omni_attn_bwd_workspace_bytes(1, 2, 1024) == 1 * 2 * 1024 * 2 * 4
    small = torch.empty(16, dtype=torch.uint8, device=gpu_device)
    q = w.q.to(gpu_device)
    with pytest.raises(RuntimeError, match="workspace"):
        omni_attn_capi.bwd(q, q, q, q, q, torch.zeros(q.shape[:3], device=gpu_device), q.clone(), q.clone(), q.clone(),
                           m.kv_num_blocks.to(gpu_device), m.kv_indices.to(gpu_device),
                           m.block_mask_types.to(gpu_device), m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE, 1024,
                           workspace=small)


def test_autograd_operator_matches_oracle_gradients(gpu_device):
    """omni_attn_torch.omni_attention: forward + backward kernels behind torch.autograd, on a
    sequence that is not a multiple of the block (the wrapper pads, gradients of padding are dropped)."""
    import omni_attn_torch as oat
    from omni_attn_torch import create_omni_block_mask_from_prefix_lengths, modality_prefix_lengths
    gen = torch.Generator().manual_seed(105)
    B, H, S, D = 1, 2, 500, 64
    S_pad = 512
    mp = torch.tensor([[[1, 100, 150], [1, 300, 90]]], dtype=torch.long)
    prefix = modality_prefix_lengths(mp, S_pad)
    mask = create_omni_block_mask_from_prefix_lengths(prefix, H, S_pad, S_pad, 128, 128)
    q, k, v = (torch.randn(B, H, S, D, generator=gen).to(torch.bfloat16) for _ in range(3))
    dout = torch.randn(B, H, S, D, generator=gen).to(torch.bfloat16)
    qd, kd, vd = (t.to(gpu_device).requires_grad_(True) for t in (q, k, v))
    for m in (mask.to(gpu_device), mask.to(gpu_device).pack_partial_masks()):
        for t in (qd, kd, vd):
            t.grad = None
        out = oat.omni_attention(qd, kd, vd, m)
        assert out.shape == (B, H, S, D)
        out.backward(dout.to(gpu_device))
        dense = prefix_mask(prefix[:, :S], S_pad)[..., :S].unsqueeze(1)
        ref = attention_dense_grads(q, k, v, dense, dout)
        check_grads((qd.grad, kd.grad, vd.grad), ref, torch.bfloat16, "autograd operator")
