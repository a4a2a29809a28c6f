"""The operator surface on the GPU: the `omni_attn` module and the five wrappers."""
import pytest
import torch

import omni_attn_torch as oat
from baseline_configs import make_workload
from helpers import compare_with_oracle
from omni_attn_torch import (create_causal_omni_block_mask, create_omni_block_mask_from_modality_positions,
                             naive_attn_mask, omni_attention_cp_async, omni_attention_forward,
                             omni_attention_preftech, omni_attention_shared_kv,
                             omni_attention_shared_kv_swizzle, omni_attention_simple)
from oracle.dense_oracle import attention_dense_fp32



pytestmark = pytest.mark.gpu

WRAPPERS = [omni_attention_simple, omni_attention_cp_async, omni_attention_preftech,
            omni_attention_shared_kv, omni_attention_shared_kv_swizzle]


def test_five_wrappers_agree_and_match_oracle_on_ragged_length(gpu_device):
    """S = 500 is zero padded to 512 by the wrapper and sliced back, as in the reference."""
    gen = torch.Generator().manual_seed(21)
    S, D = 500, 64
    q, k, v = (torch.randn(2, 4, S, D, generator=gen).to(torch.float16) for _ in range(3))
    mp = torch.tensor([[[1, 100, 150], [1, 300, 128]], [[1, 17, 60], [0, 0, 0]]])
    mask = create_omni_block_mask_from_modality_positions(mp, 2, 4, S, S, 128, 128, device="cpu")
    ro, rl = attention_dense_fp32(q, k, v, naive_attn_mask(S, mp).unsqueeze(1))
    outs = [f(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), mask) for f in WRAPPERS]
    torch.cuda.synchronize()
    for out in outs:
        assert out.shape == (2, 4, S, D) and out.dtype == torch.float16
        assert torch.equal(out, outs[0])
    o, lse = omni_attention_forward(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), mask)
    assert torch.equal(o, outs[0]) and lse.shape == (2, 4, S)
    compare_with_oracle(o, lse, ro, rl, torch.float16, "wrappers, ragged")


def test_wrapper_keeps_bf16_and_unequal_blocks(gpu_device):
    w = make_workload("c3_partial", seed=3, H=2, S=1024)
    q, k, v = (t.to(gpu_device) for t in (w.q, w.k, w.v))
    out = omni_attention_shared_kv_swizzle(q, k, v, w.block_mask)
    assert out.dtype == torch.bfloat16
    from oracle.dense_oracle import prefix_mask
    ro, rl = attention_dense_fp32(w.q, w.k, w.v, prefix_mask(w.prefix_len, 1024).unsqueeze(1))
    o, lse = omni_attention_forward(q, k, v, w.block_mask)
    compare_with_oracle(o, lse, ro, rl, torch.bfloat16, "c3 small via wrapper")
    assert torch.equal(o, out)


def test_partial_types_without_tensors_are_skipped(gpu_device):
    """has_partial = False with PARTIAL slots present: the slots contribute nothing."""
    gen = torch.Generator().manual_seed(22)
    q, k, v = (torch.randn(1, 1, 256, 64, generator=gen).to(torch.float16).to(gpu_device) for _ in range(3))
    mask = create_causal_omni_block_mask(1, 1, 256, 256, 128, 128, device="cpu")
    mask.block_mask_types[0, 0, 1, 0] = 3   # the off-diagonal FULL block becomes a bitless PARTIAL
    out = omni_attention_simple(q, k, v, mask)
    ref_mask = torch.tril(torch.ones(256, 256, dtype=torch.bool))
    ref_mask[128:, :128] = False
    ro, _ = attention_dense_fp32(q.cpu(), k.cpu(), v.cpu(), ref_mask)
    assert (out.float().cpu() - ro).abs().max().item() <= 2e-3


def test_module_errors_on_gpu_tensors(gpu_device):
    import omni_attn
    q = torch.zeros(1, 2, 256, 64, dtype=torch.float16, device=gpu_device)
    nb = torch.ones(1, 2, 2, dtype=torch.int32, device=gpu_device)
    idx = torch.zeros(1, 2, 2, 2, dtype=torch.int32, device=gpu_device)
    e_i = torch.empty(0, dtype=torch.int32, device=gpu_device)
    e_b = torch.empty(0, dtype=torch.bool, device=gpu_device)
    ok = lambda **kw: None
    with pytest.raises(RuntimeError, match="num_q_blocks"):
        omni_attn.omni_attn_simple_kernel(q, q, q, q.clone(), nb, idx, idx, 64, 64, 256, e_i, e_b, False)
    with pytest.raises(RuntimeError, match="contiguous"):
        omni_attn.omni_attn_simple_kernel(q.transpose(1, 2).contiguous().transpose(1, 2), q, q, q.clone(),
                                          nb, idx, idx, 128, 128, 256, e_i, e_b, False)
    with pytest.raises(RuntimeError, match="int32"):
        omni_attn.omni_attn_simple_kernel(q, q, q, q.clone(), nb.long(), idx, idx, 128, 128, 256, e_i, e_b, False)
    with pytest.raises(RuntimeError, match="dtype"):
        omni_attn.omni_attn_simple_kernel(q, q.bfloat16(), q, q.clone(), nb, idx, idx, 128, 128, 256, e_i, e_b, False)
    with pytest.raises(RuntimeError, match="torch.bool"):
        omni_attn.omni_attn_simple_kernel(q, q, q, q.clone(), nb, idx, idx, 128, 128, 256, idx,
                                          torch.zeros(1, 128, 128, dtype=torch.uint8, device=gpu_device), True)
    # the matrix-core entry points take head_dim 32 / 64 / 128 only; the simple one (scalar-semantics
    # kernel behind it) any head_dim up to 256
    q96 = torch.zeros(1, 2, 256, 96, dtype=torch.float16, device=gpu_device)
    with pytest.raises(RuntimeError, match="head_dim"):
        omni_attn.omni_attn_cp_async(q96, q96, q96, q96.clone(), nb, idx, idx, 128, 128, 256, e_i, e_b, False)
    omni_attn.omni_attn_simple_kernel(q96, q96, q96, q96.clone(), nb, idx, torch.full_like(idx, 2), 128, 128, 256,
                                      e_i, e_b, False)
    q264 = torch.zeros(1, 2, 256, 264, dtype=torch.float16, device=gpu_device)
    with pytest.raises(RuntimeError, match="head_dim"):
        omni_attn.omni_attn_simple_kernel(q264, q264, q264, q264.clone(), nb, idx, idx, 128, 128, 256, e_i, e_b, False)
    # and a good call still works afterwards
    omni_attn.omni_attn_simple_kernel(q, q, q, q.clone(), nb, idx, torch.full_like(idx, 2), 128, 128, 256, e_i, e_b, False)
    torch.cuda.synchronize()


def test_mask_builders_run_on_the_gpu_and_agree_with_the_cpu(gpu_device):
    """The Transfusion-rule builder is plain tensor algebra: built on the GPU from
    modality positions it gives the metadata the CPU build gives, and the wrapper accepts
    it as is (no host round trip of the mask)."""
    import time

    S, H = 16384, 4
    mp = torch.tensor([[[1, 700, 1024], [1, 5000, 900], [1, 9000, 1500], [0, 0, 0]],
                       [[1, 128, 1024], [1, 4096, 2048], [1, 12000, 1111], [1, 15000, 1384]]])
    cpu = oat.create_omni_block_mask_from_modality_positions(mp, 2, H, S, S, 128, 128, device="cpu")
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    gpu = oat.create_omni_block_mask_from_modality_positions(mp, 2, H, S, S, 128, 128, device=gpu_device)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    for name in ("kv_num_blocks", "kv_indices", "block_mask_types", "partial_block_mask_indices",
                 "partial_block_masks"):
        a, b = getattr(cpu, name), getattr(gpu, name)
        assert b.is_cuda and torch.equal(a, b.cpu()), name
    assert dt < 5.0, f"GPU mask build took {dt:.2f} s"
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(2, H, 2048, 64, generator=g).to(torch.float16).to(gpu_device) for _ in range(3))
    small = oat.create_omni_block_mask_from_modality_positions(mp[:, :1] // 8 * 2, 2, H, 2048, 2048, 64, 64,
                                                               device=gpu_device)
    o = oat.omni_attention_shared_kv(q, k, v, small)
    ref = torch.nan_to_num(oat.naive_attention(q.float(), k.float(), v.float(), small), nan=0.0)
    assert (o.float() - ref).abs().max().item() <= 2e-3
