"""The scalar-semantics forward for shapes without an MFMA instance (any block size, head_dim up
to 256, as the reference's omni_attn_simple_kernel, attn_naive.cu:189-190 and :305-408), against
both CPU oracles.  Bars: max-abs 2e-3 (fp16) / 1e-2 (bf16) on the output, 1e-3 on the logsumexp."""
import pytest
import torch

import omni_attn_capi
from helpers import compare_with_oracle, random_block_metadata
from oracle.block_walk import attention_block_walk
from oracle.dense_oracle import attention_dense_fp32, dense_mask_from_blocks

pytestmark = pytest.mark.gpu


def run_generic(q, k, v, nb, idx, tys, QB, KB, seqlen, pidx, pm, device, softcap=0.0):
    dev = lambda t: None if t is None else t.to(device).contiguous()
    qd = dev(q)
    o = torch.full_like(qd, float("nan"))
    lse = torch.full(qd.shape[:3], float("nan"), dtype=torch.float32, device=device)
    omni_attn_capi.fwd(qd, dev(k), dev(v), o, lse, dev(nb), dev(idx), dev(tys), QB, KB, seqlen, dev(pidx), dev(pm),
                       generic=True, softcap=softcap)
    torch.cuda.synchronize()
    return o, lse


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("QB,KB,D", [(32, 32, 96), (16, 48, 256), (128, 64, 128), (100, 20, 40), (64, 256, 8)])
def test_generic_kernel_any_block_size_and_head_dim(dtype, QB, KB, D, gpu_device):
    gen = torch.Generator().manual_seed(QB * 1000 + KB * 10 + D)
    B, H = 1, 2
    S = 3 * max(QB, KB) if max(QB, KB) % min(QB, KB) == 0 else QB * KB // 10  # a multiple of both
    assert S % QB == 0 and S % KB == 0
    q, k, v = (torch.randn(B, H, S, D, generator=gen).to(dtype) for _ in range(3))
    nb, idx, tys, pidx, pm = random_block_metadata(gen, B, H, S // QB, S // KB, QB, KB, p_empty=0.2, shuffle=True)
    for seqlen in (S, S - 7):
        o, lse = run_generic(q, k, v, nb, idx, tys, QB, KB, seqlen, pidx, pm, gpu_device)
        dense = dense_mask_from_blocks(nb, idx, tys, QB, KB, S, S, pidx, pm, seqlen_orig=seqlen)
        ro, rl = attention_dense_fp32(q, k, v, dense)
        compare_with_oracle(o, lse, ro, rl, dtype, f"generic vs dense oracle, seqlen={seqlen}")
        wo, wl = attention_block_walk(q, k, v, nb, idx, tys, QB, KB, seqlen, pidx, pm)
        compare_with_oracle(o, lse, wo, wl, dtype, f"generic vs block walk, seqlen={seqlen}")


def test_generic_kernel_agrees_with_the_mfma_kernel_where_both_exist(gpu_device):
    gen = torch.Generator().manual_seed(5)
    B, H, S, D, QB, KB = 1, 2, 512, 64, 128, 64
    q, k, v = (torch.randn(B, H, S, D, generator=gen).to(torch.float16) for _ in range(3))
    nb, idx, tys, pidx, pm = random_block_metadata(gen, B, H, S // QB, S // KB, QB, KB, shuffle=True)
    og, lg = run_generic(q, k, v, nb, idx, tys, QB, KB, S, pidx, pm, gpu_device, softcap=3.0)
    dev = lambda t: t.to(gpu_device).contiguous()
    om = torch.empty_like(og)
    lm = torch.empty_like(lg)
    omni_attn_capi.fwd(dev(q), dev(k), dev(v), om, lm, dev(nb), dev(idx), dev(tys), QB, KB, S, dev(pidx), dev(pm),
                       softcap=3.0)
    torch.cuda.synchronize()
    assert (og.float() - om.float()).abs().max().item() <= 2e-3
    live = ~torch.isinf(lm)
    assert torch.equal(torch.isinf(lg), torch.isinf(lm)) and (lg[live] - lm[live]).abs().max().item() <= 1e-3


def test_simple_wrapper_takes_shapes_the_other_wrappers_refuse(gpu_device):
    import omni_attn_torch as oat
    from omni_attn_torch import create_causal_omni_block_mask
    gen = torch.Generator().manual_seed(6)
    S, D, blk = 192, 80, 32
    q, k, v = (torch.randn(1, 2, S, D, generator=gen).to(torch.float16).to(gpu_device) for _ in range(3))
    mask = create_causal_omni_block_mask(1, 2, S, S, blk, blk, device=gpu_device)
    out = oat.omni_attention_simple(q, k, v, mask)
    ref, _ = attention_dense_fp32(q.cpu(), k.cpu(), v.cpu(), torch.tril(torch.ones(S, S, dtype=torch.bool)))
    assert (out.float().cpu() - ref).abs().max().item() <= 2e-3
    with pytest.raises(ValueError, match="head_dim"):
        oat.omni_attention_shared_kv_swizzle(q, k, v, mask)
