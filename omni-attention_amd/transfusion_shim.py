"""Drop-in pieces for the attention path of the Transfusion model the reference vendors.

The reference's ``transfusion_pytorch`` builds a flex-attention ``BlockMask`` from the
modality positions in ``Transformer.forward`` (transfusion_pytorch/transfusion.py:1107-1125:
``create_block_mask(causal, ...)`` at :1109, ``create_block_mask(transfusion_attn_mask(
modality_positions), ...)`` at :1117-1119) and calls ``flex_attention(q, k, v, block_mask=...,
score_mod=softcap_score_mod(softcap))`` in ``Attention.forward`` (:953-961).  The functions here
have the same roles and argument meaning with the gfx950 operator underneath:

    transfusion.py                                   this module
    ------------------------------------------------ --------------------------------------------
    create_block_mask(causal, Q_LEN=n, KV_LEN=n)     create_causal_block_mask(batch, heads, n)
    create_block_mask(transfusion_attn_mask(mp),...) create_transfusion_block_mask(mp, heads, n)
    softcap_score_mod(softcap)           (:358-364)  softcap_score_mod(softcap)
    flex_attention(q, k, v, block_mask=, score_mod=) omni_flex_attention(q, k, v, block_mask=, score_mod=)

``omni_flex_attention`` is differentiable (forward and backward kernels), takes q, k, v as
[batch, heads, seq, head_dim] fp16 / bf16, pads sequences that are not a multiple of the block
and applies the model's own scale 1/sqrt(head_dim) (transfusion.py:872, the flex default).
A flex mask has no batch or head dimension (B = None, H = None); the operator's metadata is per
(batch, head), so the builders take the head count and, for the causal mask, the batch size.
"""
from typing import Optional, Union

import torch
from torch import Tensor

from omni_attn_torch import (OmniBlockMask, create_causal_omni_block_mask,
                             create_omni_block_mask_from_modality_positions, omni_attention)


class SoftcapScoreMod:
    """What ``softcap_score_mod(softcap)`` returns: callable like the reference's score_mod
    (score, b, h, q_idx, kv_idx) -> softcap * tanh(score / softcap) (transfusion.py:358-364), and
    recognisable by ``omni_flex_attention``, which hands ``softcap`` to the kernel instead of
    calling it per score."""

    def __init__(self, softcap: float):
        if not softcap > 0:
            raise ValueError("softcap must be positive")
        self.softcap = float(softcap)

    def __call__(self, score, b=None, h=None, q_idx=None, kv_idx=None):
        return torch.tanh(score / self.softcap) * self.softcap


def softcap_score_mod(softcap: float) -> SoftcapScoreMod:
    return SoftcapScoreMod(softcap)


def _round_up(n: int, m: int) -> int:
    return (n + m - 1) // m * m


def create_causal_block_mask(batch: int, heads: int, seq_len: int, Q_BLOCK_SIZE: int = 128,
                             KV_BLOCK_SIZE: int = 128, device: Union[str, torch.device] = "cuda") -> OmniBlockMask:
    """Plain causal mask (the ``causal_mask = True`` branch, transfusion.py:1107-1112)."""
    block = max(Q_BLOCK_SIZE, KV_BLOCK_SIZE)
    n = _round_up(seq_len, block)
    return create_causal_omni_block_mask(batch, heads, n, n, Q_BLOCK_SIZE, KV_BLOCK_SIZE, device=device)


def create_transfusion_block_mask(modality_positions: Tensor, heads: int, seq_len: int,
                                  Q_BLOCK_SIZE: int = 128, KV_BLOCK_SIZE: int = 128,
                                  device: Optional[Union[str, torch.device]] = None,
                                  pack: bool = True) -> OmniBlockMask:
    """Block mask of the Transfusion rule -- text causal, a modality span bidirectional within
    itself and visible to everything after it (transfusion_attn_mask, transfusion.py:343-356) --
    for ``modality_positions`` [batch, M, 3] rows of (type, offset, length).  Built with tensor
    algebra on ``device`` (default: where modality_positions live); with ``pack`` the PARTIAL tiles
    are packed to bits once, for the many launches (layers, steps) that reuse the mask."""
    device = modality_positions.device if device is None else torch.device(device)
    block = max(Q_BLOCK_SIZE, KV_BLOCK_SIZE)
    n = _round_up(seq_len, block)
    mask = create_omni_block_mask_from_modality_positions(
        modality_positions.long(), modality_positions.shape[0], heads, n, n, Q_BLOCK_SIZE, KV_BLOCK_SIZE,
        device=device)
    if pack and torch.device(device).type == "cuda":
        mask.pack_partial_masks()
    return mask


def omni_flex_attention(query: Tensor, key: Tensor, value: Tensor, block_mask: Optional[OmniBlockMask] = None,
                        score_mod: Optional[SoftcapScoreMod] = None) -> Tensor:
    """In place of ``flex_attention(q, k, v, **flex_attn_kwargs)`` (transfusion.py:961)."""
    if score_mod is not None and not isinstance(score_mod, SoftcapScoreMod):
        raise TypeError("the only score_mod the kernel implements is softcap_score_mod(softcap)")
    if block_mask is None:
        raise ValueError("block_mask is required: create_causal_block_mask / create_transfusion_block_mask")
    return omni_attention(query, key, value, block_mask, softcap=0.0 if score_mod is None else score_mod.softcap)
