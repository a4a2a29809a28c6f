"""Seeded workload generators (CPU): determinism, layout rules, block counts."""
import pytest
import torch

from baseline_configs import SPECS, make_workload
from oracle.dense_oracle import dense_mask_from_blocks, prefix_mask, transfusion_mask_bruteforce


def test_c1_is_the_causal_configuration():
    w = make_workload("c1_causal", seed=0)
    assert w.q.shape == (1, 8, 512, 64) and w.q.dtype == torch.float16
    assert w.nonempty_blocks == 80 and w.effective_flops == 4 * 128 * 128 * 64 * 80
    assert torch.equal(prefix_mask(w.prefix_len, 512)[0], torch.tril(torch.ones(512, 512, dtype=torch.bool)))


def test_seed_determinism_and_variation():
    a = make_workload("c2_interleaved", seed=3, H=1, with_qkv=True)
    b = make_workload("c2_interleaved", seed=3, H=1, with_qkv=True)
    c = make_workload("c2_interleaved", seed=4, H=1, with_qkv=True)
    assert torch.equal(a.q, b.q) and torch.equal(a.v, b.v) and a.spans == b.spans
    assert torch.equal(a.block_mask.kv_indices, b.block_mask.kv_indices)
    assert not torch.equal(a.q, c.q)


def test_c2_layout_rules_and_block_count():
    w = make_workload("c2_interleaved", seed=0, with_qkv=False)
    assert w.block_mask.partial_block_masks is None  # aligned 1024-token images: F / C only
    for b, spans in enumerate(w.spans):
        prev_end = 0
        for off, ln in spans:
            assert ln == 1024 and off % 128 == 0 and off + ln <= 4096
            assert 128 <= off - prev_end <= 512 + 127
            prev_end = off + ln
        # causal: 32*33/2 = 528 blocks; each 8-block image adds its strict upper triangle, 28
        assert int(w.block_mask.kv_num_blocks[b, 0].sum()) == 528 + 28 * len(spans)
    assert (w.block_mask.kv_num_blocks[:, 0:1] == w.block_mask.kv_num_blocks).all()


@pytest.mark.parametrize("name", ["c3_partial", "c4_long"])
def test_unaligned_configs_represent_the_token_rule(name):
    S = 1024 if name == "c3_partial" else 2048
    w = make_workload(name, seed=1, H=1, S=S, with_qkv=False)
    QB, KB = w.block_mask.Q_BLOCK_SIZE, w.block_mask.KV_BLOCK_SIZE
    brute = transfusion_mask_bruteforce(S, w.spans[0]) if S <= 1024 else None
    dense = dense_mask_from_blocks(w.block_mask.kv_num_blocks, w.block_mask.kv_indices,
                                   w.block_mask.block_mask_types, QB, KB, S, S,
                                   w.block_mask.partial_block_mask_indices, w.block_mask.partial_block_masks)
    assert torch.equal(dense[0, 0], prefix_mask(w.prefix_len, S)[0])
    if brute is not None:
        assert torch.equal(dense[0, 0], brute)
    assert len(w.spans[0]) >= 1
    if name == "c3_partial":
        assert (w.block_mask.block_mask_types == 3).any()
        assert all(200 <= ln <= 1100 for _, ln in w.spans[0])


def test_c5_mixes_layouts_and_control_is_dense():
    w = make_workload("c5_batched", seed=0, H=1, S=2048, with_qkv=False)
    per_b = w.block_mask.kv_num_blocks[:, 0].sum(-1).tolist()
    assert w.info["layouts"][:3] == ["causal", "full", "interleaved"]
    assert per_b[0] == 16 * 17 // 2 and per_b[1] == 256
    ctl = make_workload("c5_full_control", seed=0, H=1, S=2048, with_qkv=False)
    assert (ctl.block_mask.kv_num_blocks == 16).all() and (ctl.block_mask.block_mask_types == 2).all()


def test_all_specs_build_at_full_size_without_qkv():
    for name, (B, H, S, D, dtype, QB, KB) in SPECS.items():
        w = make_workload(name, seed=0, with_qkv=False)
        assert w.block_mask.kv_num_blocks.shape == (B, H, S // QB)
        assert w.block_mask.kv_indices.shape == (B, H, S // QB, S // KB)
        assert w.nonempty_blocks > 0
