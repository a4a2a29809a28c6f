"""The Transfusion-side shim: block masks from modality positions, the soft-capped operator.

CPU: the masks represent exactly the token rule of transfusion_pytorch/transfusion.py:496-515.
GPU: omni_flex_attention (forward and backward, with and without softcap) against the fp32 dense
oracle with the reference's softclamp (transfusion.py:298-299) on the scaled scores.  Bars: the
forward's (max-abs 2e-3 fp16 / 1e-2 bf16 on the output) and the backward's (test_gpu_backward).
"""
import pytest
import torch

import transfusion_shim as shim
from helpers import TOL_O
from oracle.dense_oracle import (attention_dense_fp32, attention_dense_grads, transfusion_mask_bruteforce)


def test_masks_represent_the_token_rule():
    mp = torch.tensor([[[1, 37, 90], [2, 200, 41]], [[1, 0, 130], [0, 0, 0]]], dtype=torch.long)
    seq_len = 250
    m = shim.create_transfusion_block_mask(mp, heads=3, seq_len=seq_len, Q_BLOCK_SIZE=128, KV_BLOCK_SIZE=64,
                                           device="cpu")
    assert m.q_len == 256 and m.kv_num_blocks.shape == (2, 3, 2)
    dense = m.to_dense_mask()
    for b, spans in enumerate([[(37, 90), (200, 41)], [(0, 130)]]):
        brute = transfusion_mask_bruteforce(256, spans)
        for h in range(3):
            assert torch.equal(dense[b, h], brute)
    c = shim.create_causal_block_mask(2, 3, seq_len, device="cpu")
    assert torch.equal(c.to_dense_mask()[1, 2], torch.tril(torch.ones(256, 256, dtype=torch.bool)))
    # the score_mod is the reference's function of the score
    sm = shim.softcap_score_mod(50.0)
    x = torch.linspace(-200, 200, 11)
    assert torch.allclose(sm(x, 0, 0, 0, 0), torch.tanh(x / 50.0) * 50.0)
    with pytest.raises(TypeError):
        shim.omni_flex_attention(x, x, x, block_mask=c, score_mod=lambda s, *a: s)


@pytest.mark.gpu
@pytest.mark.parametrize("softcap", [0.0, 50.0, 2.0])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
def test_flex_replacement_forward_and_backward(dtype, softcap, gpu_device):
    from test_gpu_backward import check_grads
    gen = torch.Generator().manual_seed(int(softcap) + 17)
    B, H, S, D = 2, 2, 700, 64
    mp = torch.tensor([[[1, 100, 256], [1, 500, 77]], [[1, 3, 300], [0, 0, 0]]], dtype=torch.long)
    # softcap 2 with scaled scores of several units: the cap bites (checked below); softcap 50 is
    # the model's default, where it only bends the largest scores
    gain = 3.0 if softcap == 2.0 else 1.0
    q = (torch.randn(B, H, S, D, generator=gen) * gain).to(dtype)
    k, v, dout = (torch.randn(B, H, S, D, generator=gen).to(dtype) for _ in range(3))
    mask = shim.create_transfusion_block_mask(mp.to(gpu_device), heads=H, seq_len=S)
    assert mask.partial_block_bits is not None
    qd, kd, vd = (t.to(gpu_device).requires_grad_(True) for t in (q, k, v))
    out = shim.omni_flex_attention(qd, kd, vd, block_mask=mask,
                                   score_mod=shim.softcap_score_mod(softcap) if softcap else None)
    out.backward(dout.to(gpu_device))
    dense = torch.stack([transfusion_mask_bruteforce(S, [(o, l) for _, o, l in mp[b].tolist() if l > 0])
                         for b in range(B)]).unsqueeze(1)
    ro, _ = attention_dense_fp32(q, k, v, dense, softcap=softcap)
    err = (out.detach().float().cpu() - ro).abs().max().item()
    assert err <= TOL_O[dtype], f"forward softcap={softcap}: max|dO| = {err:.3e}"
    ref = attention_dense_grads(q, k, v, dense, dout, softcap=softcap)
    check_grads((qd.grad, kd.grad, vd.grad), ref, dtype, f"softcap={softcap}")
    if softcap == 2.0:
        # the cap changes the answer (this case would pass with the hook switched off otherwise)
        ro_plain, _ = attention_dense_fp32(q, k, v, dense)
        assert (ro - ro_plain).abs().max().item() > 0.05


@pytest.mark.gpu
def test_softcap_through_the_c_abi_all_block_shapes(gpu_device):
    """Soft-capped forward on random metadata for every (Q_BLOCK, KV_BLOCK), logsumexp included."""
    import omni_attn_capi
    from helpers import compare_with_oracle, random_block_metadata
    from oracle.dense_oracle import dense_mask_from_blocks
    for QB, KB in ((128, 128), (128, 64), (64, 128), (64, 64)):
        gen = torch.Generator().manual_seed(QB + KB)
        B, H, S, D = 1, 2, 512, 128
        q = (torch.randn(B, H, S, D, generator=gen) * 2).to(torch.bfloat16)
        k, v = (torch.randn(B, H, S, D, generator=gen).to(torch.bfloat16) for _ in range(2))
        nb, idx, tys, pidx, pm = random_block_metadata(gen, B, H, S // QB, S // KB, QB, KB, shuffle=True)
        dev = lambda t: t.to(gpu_device).contiguous()
        o = torch.full_like(dev(q), float("nan"))
        lse = torch.full((B, H, S), float("nan"), dtype=torch.float32, device=gpu_device)
        omni_attn_capi.fwd(dev(q), dev(k), dev(v), o, lse, dev(nb), dev(idx), dev(tys), QB, KB, S - 30, dev(pidx),
                           dev(pm), softcap=5.0)
        torch.cuda.synchronize()
        dense = dense_mask_from_blocks(nb, idx, tys, QB, KB, S, S, pidx, pm, seqlen_orig=S - 30)
        ro, rl = attention_dense_fp32(q, k, v, dense, softcap=5.0)
        compare_with_oracle(o, lse, ro, rl, torch.bfloat16, f"softcap 5, blocks {QB}/{KB}")
