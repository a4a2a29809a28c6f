"""Block-mask data structure and builders (host logic, CPU)."""
import pytest
import torch

from helpers import load_printed_masks, random_block_metadata
from omni_attn_torch import (BlockMaskType, OmniBlockMask, block_pattern_rows,
                             build_partial_block_data, create_causal_omni_block_mask,
                             create_omni_block_mask_from_dense,
                             create_omni_block_mask_from_modality_positions,
                             create_omni_block_mask_from_prefix_lengths, modality_prefix_lengths,
                             naive_attn_mask, _pad_to_block_size)
from oracle.dense_oracle import dense_mask_from_blocks, transfusion_mask_bruteforce


def _rows_compact(mask):
    return [r.replace(" ", "x")[::2].replace("x", ".") for r in block_pattern_rows(mask)]


def _segment_dense(kind, S, segments):
    """Dense masks of the reference's generators, from their definitions
    (generate_attn_data.py:176-187 interleaved, :304-308 document)."""
    ends = [sum(segments[: i + 1]) for i in range(len(segments))]
    m = torch.zeros(S, S, dtype=torch.bool)
    if kind == "causal":
        return torch.tril(torch.ones(S, S, dtype=torch.bool)), [0, S]
    if kind == "document":
        start = 0
        for e in ends:
            m[start:e, start:e] = True
            start = e
    elif kind == "interleaved":
        s1, s2 = ends[0], ends[1]
        for qi in range(S):
            if qi < s1:
                m[qi, : qi + 1] = True
            elif qi < s2:
                m[qi, :s2] = True
            else:
                m[qi, : qi + 1] = True
    return m, [0] + ends


def test_block_mask_type_values():
    assert (int(BlockMaskType.MASKED), int(BlockMaskType.CAUSAL), int(BlockMaskType.FULL),
            int(BlockMaskType.PARTIAL)) == (0, 1, 2, 3)


@pytest.mark.parametrize("pat", load_printed_masks()["segment_patterns"], ids=lambda p: p["kind"])
def test_classifier_reproduces_printed_patterns(pat):
    """Known segment lengths -> the block pattern and dense sparsity the reference printed."""
    S, QB, KB = pat["seq_len"], pat["Q_BLOCK_SIZE"], pat["KV_BLOCK_SIZE"]
    dense, bounds = _segment_dense(pat["kind"], S, pat["segments"])
    assert abs((1 - dense.float().mean().item()) - pat["sparsity"]) < 5e-5
    rule = pat["kind"] if pat["kind"] in ("interleaved", "document") else "none"
    mask = create_omni_block_mask_from_dense(dense.view(1, 1, S, S), QB, KB, boundaries=bounds,
                                             boundary_rule=rule)
    assert _rows_compact(mask) == pat["rows"]
    # whatever the labels, the metadata must represent the dense mask it came from
    assert torch.equal(mask.to_dense_mask()[0, 0], dense)
    assert torch.equal(dense_mask_from_blocks(mask.kv_num_blocks, mask.kv_indices, mask.block_mask_types,
                                              QB, KB, S, S, mask.partial_block_mask_indices,
                                              mask.partial_block_masks)[0, 0], dense)


def test_causal_builder_matches_printed_pattern_and_closed_form():
    pat = [p for p in load_printed_masks()["segment_patterns"] if p["kind"] == "causal"][0]
    mask = create_causal_omni_block_mask(2, 3, 512, 512, 64, 64, device="cpu")
    assert _rows_compact(mask) == pat["rows"]
    assert mask.kv_num_blocks.shape == (2, 3, 8) and mask.kv_indices.shape == (2, 3, 8, 8)
    assert mask.kv_num_blocks.dtype == torch.int32 and mask.block_mask_types.dtype == torch.int32
    assert torch.equal(mask.to_dense_mask()[1, 2], torch.tril(torch.ones(512, 512, dtype=torch.bool)))
    assert abs(mask.sparsity() - 100 * (1 - 36 / 64)) < 1e-9
    # first BASELINE configuration: 10 of 16 blocks per head
    c1 = create_causal_omni_block_mask(1, 8, 512, 512, 128, 128, device="cpu")
    assert c1.kv_num_blocks[0, 0].tolist() == [1, 2, 3, 4] and int(c1.kv_num_blocks.sum()) == 80


@pytest.mark.parametrize("QB,KB,S", [(128, 64, 512), (64, 128, 512), (128, 128, 500), (128, 64, 300)])
def test_causal_builder_unequal_blocks_and_padding(QB, KB, S):
    mask = create_causal_omni_block_mask(1, 1, S, S, QB, KB, device="cpu")
    q_pad = -(-S // QB) * QB
    kv_pad = -(-S // KB) * KB
    assert (mask.q_len, mask.kv_len) == (q_pad, kv_pad)
    dense = mask.to_dense_mask()[0, 0]
    assert torch.equal(dense, torch.tril(torch.ones(q_pad, kv_pad, dtype=torch.bool)))
    # kv indices ascending inside the live slots, zero filled behind them
    for qb in range(mask.num_q_blocks):
        n = int(mask.kv_num_blocks[0, 0, qb])
        assert mask.kv_indices[0, 0, qb, :n].tolist() == list(range(n))
        assert (mask.kv_indices[0, 0, qb, n:] == 0).all() and (mask.block_mask_types[0, 0, qb, n:] == 0).all()


@pytest.mark.parametrize("QB,KB", [(128, 128), (128, 64), (64, 64)])
def test_dense_round_trip_random_masks(QB, KB):
    gen = torch.Generator().manual_seed(QB + KB)
    S = 512
    dense = torch.rand(2, 2, S, S, generator=gen) < 0.5
    dense[:, :, :, 128:256] = False          # empty block column
    dense[0, 0, 256:384, :] = False          # empty block row
    dense[1, 1, 0:128, 0:128] = True         # a FULL tile
    dense[1, 0, 384:512, 384:512] = torch.tril(torch.ones(128, 128, dtype=torch.bool))
    mask = create_omni_block_mask_from_dense(dense, QB, KB)
    assert torch.equal(mask.to_dense_mask(), dense)
    assert torch.equal(dense_mask_from_blocks(mask.kv_num_blocks, mask.kv_indices, mask.block_mask_types,
                                              QB, KB, S, S, mask.partial_block_mask_indices,
                                              mask.partial_block_masks), dense)
    assert int(mask.kv_num_blocks[0, 0, 256 // QB]) == 0


def test_build_partial_block_data_matches_loops():
    gen = torch.Generator().manual_seed(7)
    QB, KB, S = 64, 128, 512
    nb, idx, tys, _, _ = random_block_metadata(gen, 2, 2, S // QB, S // KB, QB, KB, with_bitless_partial=False)
    dense = torch.rand(2, 2, S - 20, S - 20, generator=gen) < 0.5   # ragged: gets zero padded
    mask = OmniBlockMask(nb, idx, tys, S, S, QB, KB)
    pidx, tiles = build_partial_block_data(mask, dense)
    padded = torch.zeros(2, 2, S, S, dtype=torch.bool)
    padded[:, :, : S - 20, : S - 20] = dense
    count = 0
    for b in range(2):
        for h in range(2):
            for qb in range(S // QB):
                for s in range(idx.shape[-1]):
                    if s < int(nb[b, h, qb]) and int(tys[b, h, qb, s]) == 3:
                        kb = int(idx[b, h, qb, s])
                        assert int(pidx[b, h, qb, s]) == count
                        assert torch.equal(tiles[count], padded[b, h, qb * QB:(qb + 1) * QB, kb * KB:(kb + 1) * KB])
                        count += 1
                    else:
                        assert int(pidx[b, h, qb, s]) == -1
    assert tiles.shape == (count, QB, KB) and tiles.dtype == torch.bool and pidx.dtype == torch.int32


def test_deduplicate_partial_tiles_shares_tiles_between_heads():
    """A dense mask that is the same for every head: the reference's tile store holds one copy
    per head (omni_attn_torch.py:173-196); after de-duplication one copy per distinct tile is
    left, in order of first appearance, and the mask represents the same dense mask."""
    gen = torch.Generator().manual_seed(11)
    B, H, S, QB, KB = 2, 4, 512, 128, 64
    per_batch = torch.rand(B, 1, S, S, generator=gen) < 0.5
    per_batch[0, 0, :128, :64] = per_batch[0, 0, 128:256, 64:128]  # two equal tiles inside one head as well
    dense = per_batch.expand(B, H, S, S).contiguous()
    mask = create_omni_block_mask_from_dense(dense, QB, KB)
    P = mask.partial_block_masks.shape[0]
    assert P == B * H * (S // QB) * (S // KB)          # every tile is PARTIAL and stored per head
    before = mask.to_dense_mask()
    old_idx, old_tiles = mask.partial_block_mask_indices.clone(), mask.partial_block_masks.clone()
    mask.deduplicate_partial_tiles()
    U = mask.partial_block_masks.shape[0]
    assert U == B * (S // QB) * (S // KB) - 1
    assert torch.equal(mask.to_dense_mask(), before) and torch.equal(before, dense)
    new_idx = mask.partial_block_mask_indices
    assert new_idx.dtype == torch.int32 and torch.equal(new_idx < 0, old_idx < 0)
    sel = old_idx >= 0
    assert torch.equal(mask.partial_block_masks[new_idx[sel].long()], old_tiles[old_idx[sel].long()])
    # order of first appearance: the tile numbers, in visiting order, never jump ahead
    seq = new_idx[sel].tolist()
    seen = -1
    for t in seq:
        assert t <= seen + 1
        seen = max(seen, t)
    # nothing to do the second time; masks without tiles pass through
    assert mask.deduplicate_partial_tiles().partial_block_masks.shape[0] == U
    assert create_causal_omni_block_mask(1, 2, 256, 256, device="cpu").deduplicate_partial_tiles().partial_block_masks is None


def test_to_dense_mask_partial_fallbacks():
    """PARTIAL without stored bits: causal in the reference's to_dense_mask, skipped by the kernels."""
    nb = torch.tensor([[[1, 2]]], dtype=torch.int32)
    idx = torch.tensor([[[[0, 0], [0, 1]]]], dtype=torch.int32)
    tys = torch.tensor([[[[3, 0], [2, 3]]]], dtype=torch.int32)
    mask = OmniBlockMask(nb, idx, tys, 128, 128, 64, 64)
    tril = torch.tril(torch.ones(128, 128, dtype=torch.bool))
    ref_like = mask.to_dense_mask()
    assert torch.equal(ref_like[0, 0], tril)
    kernel_like = mask.to_dense_mask(partial_fallback="skip")
    expect = torch.zeros(128, 128, dtype=torch.bool)
    expect[64:, :64] = True
    assert torch.equal(kernel_like[0, 0], expect)


@pytest.mark.parametrize("QB,KB", [(128, 128), (128, 64)])
def test_modality_builder_represents_token_rule(QB, KB):
    S = 700  # ragged: padded to 768
    spans = [(100, 150), (300, 128), (520, 90)]
    mp = torch.tensor([[[1, o, l] for o, l in spans] + [[0, 0, 0]]])
    mask = create_omni_block_mask_from_modality_positions(mp, 1, 3, S, S, QB, KB, device="cpu")
    brute = transfusion_mask_bruteforce(S, spans)
    pad, kpad = -(-S // QB) * QB, -(-S // KB) * KB
    expect = torch.zeros(pad, kpad, dtype=torch.bool)
    expect[:S, :S] = brute
    for h in range(3):
        assert torch.equal(mask.to_dense_mask(partial_fallback="skip")[0, h], expect)
    assert mask.partial_block_masks is not None and mask.partial_block_masks.shape[1:] == (QB, KB)
    # same answer through the dense classifier
    via_dense = create_omni_block_mask_from_dense(expect.view(1, 1, pad, kpad), QB, KB)
    assert torch.equal(via_dense.kv_num_blocks[0, 0], mask.kv_num_blocks[0, 0])
    assert torch.equal(via_dense.block_mask_types[0, 0], mask.block_mask_types[0, 0])
    assert torch.equal(via_dense.partial_block_masks, mask.partial_block_masks)


def test_aligned_images_need_no_partial_blocks():
    S = 2048
    mp = torch.tensor([[[1, 256, 1024], [1, 1536, 256]]])
    mask = create_omni_block_mask_from_modality_positions(mp, 1, 1, S, S, 128, 128, device="cpu")
    assert mask.partial_block_masks is None
    assert not (mask.block_mask_types == 3).any()
    assert torch.equal(mask.to_dense_mask()[0, 0], naive_attn_mask(S, mp)[0])
    # image query blocks list every block up to the image end, all FULL
    assert int(mask.kv_num_blocks[0, 0, 2]) == 10 and (mask.block_mask_types[0, 0, 2, :10] == 2).all()


def test_pad_to_block_size():
    x = torch.arange(2 * 3 * 5 * 4, dtype=torch.float32).view(2, 3, 5, 4)
    y, n = _pad_to_block_size(x, 4)
    assert n == 5 and y.shape == (2, 3, 8, 4) and torch.equal(y[:, :, :5], x) and (y[:, :, 5:] == 0).all()
    z, n = _pad_to_block_size(y, 4)
    assert z is y and n == 8
