"""Tensors beyond 2^31 elements (4 GiB and more per operand): forward and backward through the C ABI.

Every slab offset of the kernels is a 64-bit quantity; this test pins that.  264 (batch, head)
slabs of 65 536 rows at head_dim 128 in bf16 are 2.2e9 elements = 4.4e9 bytes per tensor, so slab
128 starts at byte 2^31 and slab 256 at byte 2^32.  The mask is a two-block sliding window (block
i - 1 FULL, block i CAUSAL), which keeps the launch short and makes every checked quantity
depend on three neighbouring blocks only: a 384-row extract of a slab is judged by the dense
oracle.  Bars as everywhere: O 1e-2, LSE 1e-3 (bf16); gradients 3e-2 of max(1, max|reference|).
"""
import pytest
import torch

import omni_attn_capi
from oracle.dense_oracle import attention_dense_fp32, attention_dense_grads

pytestmark = pytest.mark.gpu

B, H, S, D, BLK = 3, 88, 65536, 128, 128
TQ = S // BLK


def window_metadata(device):
    """Query block i lists [i - 1 (FULL), i (CAUSAL)]; block 0 only itself."""
    i = torch.arange(TQ, dtype=torch.int32)
    idx = torch.stack([torch.clamp(i - 1, min=0), i], dim=1)
    tys = torch.tensor([2, 1], dtype=torch.int32).repeat(TQ, 1)
    idx[0] = torch.tensor([0, 0], dtype=torch.int32)
    tys[0] = torch.tensor([1, 0], dtype=torch.int32)
    nb = torch.full((TQ,), 2, dtype=torch.int32)
    nb[0] = 1
    expand = lambda t: t.unsqueeze(0).unsqueeze(0).expand(B, H, *t.shape).contiguous().to(device)
    return expand(nb), expand(idx), expand(tys)


def extract_mask():
    """Dense mask of three neighbouring blocks under the window rule (first block: itself only)."""
    n = 3 * BLK
    r = torch.arange(n)
    causal = r[:, None] >= r[None, :]
    rb, cb = r[:, None] // BLK, r[None, :] // BLK
    return (causal & ((cb == rb) | (cb == rb - 1))).view(1, 1, n, n)


def test_forward_and_backward_on_tensors_beyond_four_gib(gpu_device):
    free, _ = torch.cuda.mem_get_info(gpu_device)
    need = 8 * B * H * S * D * 2 + (1 << 30)
    if free < need:
        pytest.skip("needs %.0f GiB of free device memory" % (need / 2**30))
    assert B * H * S * D > 2**31
    gen = torch.Generator(device=gpu_device).manual_seed(2024)
    shape = (B, H, S, D)
    q, k, v, dout = (torch.randn(shape, device=gpu_device, dtype=torch.bfloat16, generator=gen) for _ in range(4))
    o, dq, dk, dv = (torch.full(shape, float("nan"), device=gpu_device, dtype=torch.bfloat16) for _ in range(4))
    lse = torch.full((B, H, S), float("nan"), device=gpu_device, dtype=torch.float32)
    nb, idx, tys = window_metadata(gpu_device)
    omni_attn_capi.fwd(q, k, v, o, lse, nb, idx, tys, BLK, BLK, S)
    omni_attn_capi.bwd(q, k, v, o, dout, lse, dq, dk, dv, nb, idx, tys, BLK, BLK, S)
    torch.cuda.synchronize()

    mask = extract_mask()
    mid = slice(BLK, 3 * BLK)       # rows whose keys all lie inside the extract
    own = slice(BLK, 2 * BLK)       # keys whose queries all lie inside the extract
    # first and last slab, and the slabs on either side of byte 2^31 and byte 2^32
    for bh in (0, 127, 128, 255, 256, B * H - 1):
        b, h = divmod(bh, H)
        for i in (1, TQ // 2, TQ - 2):
            rows = slice((i - 1) * BLK, (i + 2) * BLK)
            ex = lambda t: t[b, h, rows].unsqueeze(0).unsqueeze(0).cpu()
            qe, ke, ve, de = ex(q), ex(k), ex(v), ex(dout)
            ro, rl = attention_dense_fp32(qe, ke, ve, mask)
            what = "slab %d query block %d" % (bh, i)
            eo = (ex(o).float()[..., mid, :] - ro[..., mid, :]).abs().max().item()
            el = (lse[b, h, rows].cpu()[mid] - rl[0, 0, mid]).abs().max().item()
            assert eo <= 1e-2 and el <= 1e-3, "%s: max|dO| %.3e max|dLSE| %.3e" % (what, eo, el)
            rq, rk, rv = attention_dense_grads(qe, ke, ve, mask, de)
            for name, got, ref, part in (("dQ", dq, rq, mid), ("dK", dk, rk, own), ("dV", dv, rv, own)):
                g = ex(got).float()[..., part, :]
                r = ref[..., part, :]
                assert torch.isfinite(g).all(), "%s: non-finite %s" % (what, name)
                err = (g - r).abs().max().item()
                bar = 3e-2 * max(1.0, r.abs().max().item())
                assert err <= bar, "%s: %s error %.3e > %.3e" % (what, name, err, bar)
    del q, k, v, dout, o, dq, dk, dv, lse
    torch.cuda.empty_cache()
