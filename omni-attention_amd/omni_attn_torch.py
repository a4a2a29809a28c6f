"""Host side of the gfx950 block-sparse attention forward.

Counterpart of the reference's ``omni-attn-mma/omni_attn_torch.py`` for the forward
path only: the block-mask data structure and its builders, the five operator wrappers
with the reference's names and ``(query, key, value, block_mask)`` signature, and the
small utilities those wrappers use.  The wrappers call the ``omni_attn`` extension
module (built by ``build.py`` next to this file); there is no fallback path -- if the
module is missing, the call raises ``ImportError``.

Differences from the reference that are deliberate:
  * bf16 inputs stay bf16 (the reference forces ``.half()``, omni_attn_torch.py:609-611);
  * no global ``torch.cuda.synchronize()`` after the launch (omni_attn_torch.py:666);
  * builders are vectorised (the reference loops in the interpreter per block and per
    element, omni_attn_torch.py:101-143, :173-196, :1991-2005);
  * ``omni_attention_forward`` additionally returns the row logsumexp.
"""
import importlib
import math
import os
import sys
from dataclasses import dataclass, field
from enum import IntEnum
from typing import List, Optional, Sequence, Tuple, Union

import torch
import torch.nn.functional as F
from torch import Tensor


# ----------------------------------------------------------------------------
# Block mask types (values fixed by omni_attn_torch.py:38-41 / attn_naive.cu:4-7)
# ----------------------------------------------------------------------------

class BlockMaskType(IntEnum):
    MASKED = 0   # block skipped entirely
    CAUSAL = 1   # keep k_global <= q_global
    FULL = 2     # keep everything
    PARTIAL = 3  # keep the stored per-element mask


# ----------------------------------------------------------------------------
# Block mask data structure (omni_attn_torch.py:48-145)
# ----------------------------------------------------------------------------

@dataclass
class OmniBlockMask:
    """Block-sparse attention mask.

    kv_num_blocks    [B, H, num_q_blocks] int32, active KV blocks per query block
    kv_indices       [B, H, num_q_blocks, max_blocks] int32, KV block index per slot
    block_mask_types [B, H, num_q_blocks, max_blocks] int32, BlockMaskType per slot
    q_len, kv_len    padded lengths (multiples of the block sizes)
    partial_block_mask_indices  [B, H, num_q_blocks, max_blocks] int32, -1 = none
    partial_block_masks         [P, Q_BLOCK_SIZE, KV_BLOCK_SIZE] bool
    partial_block_bits          [P, Q_BLOCK_SIZE, KV_BLOCK_SIZE // 32] int32: the same tiles, one
                                bit per element, filled by pack_partial_masks() (not in the
                                reference; the wrappers use it when it is there)
    """
    kv_num_blocks: Tensor
    kv_indices: Tensor
    block_mask_types: Tensor
    q_len: int
    kv_len: int
    Q_BLOCK_SIZE: int = 128
    KV_BLOCK_SIZE: int = 128
    partial_block_mask_indices: Optional[Tensor] = None
    partial_block_masks: Optional[Tensor] = None
    partial_block_bits: Optional[Tensor] = None
    # cache of has_partial_slots(); travels with to()
    _any_partial_slot: Optional[bool] = field(default=None, repr=False, compare=False)

    def has_partial_slots(self) -> bool:
        """Does any slot carry the type PARTIAL?  Answered once per mask (one reduction, and on a GPU
        one read-back) and remembered: the wrappers that need the answer on every call
        (omni_attn_torch.py:763-765, :1067-1069) then cost no device synchronisation."""
        if self._any_partial_slot is None:
            self._any_partial_slot = bool((self.block_mask_types == int(BlockMaskType.PARTIAL)).any())
        return self._any_partial_slot

    def pack_partial_masks(self) -> "OmniBlockMask":
        """Pack the PARTIAL tiles once (on the GPU, by the extension's pre-pass kernel) for a mask
        that is used for many launches; the wrappers then pass the packed words."""
        if self.partial_block_masks is not None and self.partial_block_masks.numel() > 0:
            if not self.partial_block_masks.is_cuda:
                raise ValueError("pack_partial_masks needs the mask on the GPU: mask.to(device) first")
            self.partial_block_bits = _load_extension().omni_attn_pack_partial_masks(
                self.partial_block_masks.to(torch.bool).contiguous())
        return self

    def deduplicate_partial_tiles(self) -> "OmniBlockMask":
        """Keep one copy of every distinct PARTIAL tile and point the slots at it.

        The reference stores a tile per (batch, head, q_block, slot) in visiting order
        (omni_attn_torch.py:173-196), so a mask that is the same for every head holds H copies of
        each tile.  The kernels only follow ``partial_block_mask_indices``; sharing tiles changes
        no result.  Kept tiles stay in order of first appearance.  Runs where the mask lives."""
        pm = self.partial_block_masks
        if pm is None or self.partial_block_mask_indices is None or pm.shape[0] < 2:
            return self
        P = pm.shape[0]
        dev = pm.device
        if self.partial_block_bits is not None:
            rows = self.partial_block_bits.reshape(P, -1)
        else:  # 8 mask bytes -> one byte of bits, so the sort behind unique() moves 8x less
            flat = (pm.reshape(P, -1) != 0).to(torch.uint8)
            pad = (-flat.shape[1]) % 8
            if pad:
                flat = torch.nn.functional.pad(flat, (0, pad))
            weights = (2 ** torch.arange(8, device=dev, dtype=torch.int32)).view(1, 1, 8)
            rows = (flat.view(P, -1, 8).to(torch.int32) * weights).sum(-1).to(torch.uint8)
        uniq, inverse = torch.unique(rows, dim=0, return_inverse=True)
        U = uniq.shape[0]
        if U == P:
            return self
        first = torch.full((U,), P, dtype=torch.long, device=dev)
        first.scatter_reduce_(0, inverse, torch.arange(P, device=dev), reduce="amin")
        order = torch.argsort(first)                      # unique tiles by first appearance
        rank = torch.empty_like(order)
        rank[order] = torch.arange(U, device=dev)
        new_id = rank[inverse].to(torch.int32)            # old tile number -> new tile number
        keep = first[order]
        old = self.partial_block_mask_indices
        safe = old.clamp(min=0, max=P - 1).long()
        valid = (old >= 0) & (old < P)
        self.partial_block_mask_indices = torch.where(valid, new_id.to(old.device)[safe], old)
        self.partial_block_masks = pm[keep].contiguous()
        if self.partial_block_bits is not None:
            self.partial_block_bits = self.partial_block_bits[keep].contiguous()
        return self

    @property
    def num_q_blocks(self) -> int:
        return (self.q_len + self.Q_BLOCK_SIZE - 1) // self.Q_BLOCK_SIZE

    @property
    def num_kv_blocks(self) -> int:
        return (self.kv_len + self.KV_BLOCK_SIZE - 1) // self.KV_BLOCK_SIZE

    @property
    def device(self) -> torch.device:
        return self.kv_num_blocks.device

    @property
    def shape(self) -> Tuple[int, int, int, int]:
        B, H, _ = self.kv_num_blocks.shape
        return (B, H, self.q_len, self.kv_len)

    def to(self, device) -> "OmniBlockMask":
        mv = lambda t: None if t is None else t.to(device)
        return OmniBlockMask(
            mv(self.kv_num_blocks), mv(self.kv_indices), mv(self.block_mask_types),
            self.q_len, self.kv_len, self.Q_BLOCK_SIZE, self.KV_BLOCK_SIZE,
            mv(self.partial_block_mask_indices), mv(self.partial_block_masks), mv(self.partial_block_bits),
            self._any_partial_slot)

    def to_dense_mask(self, partial_fallback: str = "causal") -> Tensor:
        """Dense bool mask [B, H, q_len, kv_len], True = attend.

        Same result as the reference's per-element loops (omni_attn_torch.py:89-145),
        computed one block slot at a time over all (b, h, q_block) at once.

        ``partial_fallback`` decides what a PARTIAL slot without stored bits means:
        "causal" is what the reference's to_dense_mask does (omni_attn_torch.py:140-143);
        "skip" is what the kernels do (attn_naive.cu:119-131).
        """
        if partial_fallback not in ("causal", "skip"):
            raise ValueError("partial_fallback must be 'causal' or 'skip'")
        B, H, Tq, max_blocks = self.kv_indices.shape
        QB, KB = self.Q_BLOCK_SIZE, self.KV_BLOCK_SIZE
        Tk = self.num_kv_blocks
        dev = self.device
        q_pad, kv_pad = Tq * QB, Tk * KB
        # blocks[b, h, qb, kb, r, c]
        blocks = torch.zeros(B, H, Tq, Tk, QB, KB, dtype=torch.bool, device=dev)
        nb = self.kv_num_blocks.long()
        r = torch.arange(QB, device=dev).view(1, QB, 1)
        c = torch.arange(KB, device=dev).view(1, 1, KB)
        have_bits = (self.partial_block_mask_indices is not None
                     and self.partial_block_masks is not None)
        P = self.partial_block_masks.shape[0] if have_bits else 0
        for slot in range(max_blocks):
            active = nb > slot                                   # [B,H,Tq]
            if not bool(active.any()):
                break
            kvb = self.kv_indices[..., slot].long()
            ty = self.block_mask_types[..., slot].long()
            b_i, h_i, q_i = torch.nonzero(active, as_tuple=True)
            kvb_a, ty_a = kvb[b_i, h_i, q_i], ty[b_i, h_i, q_i]
            inside = (kvb_a >= 0) & (kvb_a < Tk)
            b_i, h_i, q_i, kvb_a, ty_a = b_i[inside], h_i[inside], q_i[inside], kvb_a[inside], ty_a[inside]
            qg = (q_i * QB).view(-1, 1, 1) + r
            kg = (kvb_a * KB).view(-1, 1, 1) + c
            causal_tile = kg <= qg                               # [n,QB,KB]
            tile = torch.zeros(len(b_i), QB, KB, dtype=torch.bool, device=dev)
            tile |= (ty_a == BlockMaskType.FULL).view(-1, 1, 1)
            tile |= (ty_a == BlockMaskType.CAUSAL).view(-1, 1, 1) & causal_tile
            is_p = ty_a == BlockMaskType.PARTIAL
            if bool(is_p.any()):
                if have_bits:
                    pid = self.partial_block_mask_indices[..., slot].long()[b_i, h_i, q_i]
                    ok = is_p & (pid >= 0) & (pid < P)
                    if bool(ok.any()):
                        tile[ok] = self.partial_block_masks[pid[ok]].to(torch.bool)
                    missing = is_p & ~ok
                else:
                    missing = is_p
                if partial_fallback == "causal":
                    tile |= missing.view(-1, 1, 1) & causal_tile
            blocks[b_i, h_i, q_i, kvb_a] = tile
        dense = blocks.permute(0, 1, 2, 4, 3, 5).reshape(B, H, q_pad, kv_pad)
        return dense[:, :, : self.q_len, : self.kv_len].contiguous()

    def to_score_mask(self) -> Tensor:
        """0 where attended, -inf where masked (omni_attn_torch.py:207-215)."""
        dense = self.to_dense_mask()
        zero = torch.zeros((), dtype=torch.float32, device=dense.device)
        return torch.where(dense, zero, torch.full_like(zero, float("-inf")))

    def sparsity(self) -> float:
        """Percentage of (q_block, kv_block) pairs that are skipped (omni_attn_torch.py:217-223)."""
        total_blocks = self.num_q_blocks * self.num_kv_blocks
        B, H = self.kv_num_blocks.shape[:2]
        avg_active = float(self.kv_num_blocks.float().sum().item()) / (B * H)
        return 100.0 * (1.0 - avg_active / total_blocks)


def _pad_dense(dense_mask: Tensor, q_len: int, kv_len: int) -> Tensor:
    if dense_mask.shape[2] == q_len and dense_mask.shape[3] == kv_len:
        return dense_mask
    B, H = dense_mask.shape[:2]
    padded = torch.zeros(B, H, q_len, kv_len, dtype=dense_mask.dtype, device=dense_mask.device)
    ql, kl = min(dense_mask.shape[2], q_len), min(dense_mask.shape[3], kv_len)
    padded[:, :, :ql, :kl] = dense_mask[:, :, :ql, :kl]
    return padded


def build_partial_block_data(block_mask: OmniBlockMask, dense_mask: Tensor) -> Tuple[Tensor, Tensor]:
    """Per-block bool tiles for the PARTIAL slots of ``block_mask``.

    Same output as omni_attn_torch.py:148-205: tiles are numbered in (b, h, q_block,
    slot) visiting order, ``partial_indices`` is -1 elsewhere, ragged tiles are zero
    padded.  Tiles are gathered in one indexing operation instead of a Python loop.
    """
    B, H, Tq, max_blocks = block_mask.block_mask_types.shape
    QB, KB = block_mask.Q_BLOCK_SIZE, block_mask.KV_BLOCK_SIZE
    dev = dense_mask.device
    Tk = block_mask.num_kv_blocks
    dense = _pad_dense(dense_mask.to(torch.bool), Tq * QB, Tk * KB)
    if dense.shape[2] != Tq * QB or dense.shape[3] != Tk * KB:
        dense = _pad_dense(dense, Tq * QB, Tk * KB)
    slot = torch.arange(max_blocks, device=dev).view(1, 1, 1, max_blocks)
    is_p = (block_mask.block_mask_types.to(dev) == BlockMaskType.PARTIAL) & \
           (slot < block_mask.kv_num_blocks.to(dev).long().unsqueeze(-1))
    partial_indices = torch.full((B, H, Tq, max_blocks), -1, dtype=torch.int32, device=dev)
    b_i, h_i, q_i, s_i = torch.nonzero(is_p, as_tuple=True)  # row-major = visiting order
    n = b_i.numel()
    if n == 0:
        return partial_indices, torch.empty(0, QB, KB, dtype=torch.bool, device=dev)
    partial_indices[b_i, h_i, q_i, s_i] = torch.arange(n, dtype=torch.int32, device=dev)
    kvb = block_mask.kv_indices.to(dev).long()[b_i, h_i, q_i, s_i]
    blocks = dense.view(B, H, Tq, QB, Tk, KB)
    tiles = blocks[b_i, h_i, q_i, :, kvb, :]                 # [n, QB, KB]
    return partial_indices, tiles.contiguous()


# ----------------------------------------------------------------------------
# Builders
# ----------------------------------------------------------------------------

def _round_up(x: int, m: int) -> int:
    return ((x + m - 1) // m) * m


def _pack_slots(active: Tensor, types: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
    """[..., Tk] active flags / types per KV block -> (kv_num_blocks, kv_indices, types)
    with the active blocks first, in ascending block order, zero filled behind them."""
    Tk = active.shape[-1]
    order = torch.argsort((~active).to(torch.int8), dim=-1, stable=True)
    nb = active.sum(-1).to(torch.int32)
    slot = torch.arange(Tk, device=active.device).expand_as(order)
    live = slot < nb.unsqueeze(-1)
    kv_indices = torch.where(live, order, torch.zeros_like(order)).to(torch.int32)
    tys = torch.where(live, torch.gather(types, -1, order), torch.zeros_like(types)).to(torch.int32)
    return nb.contiguous(), kv_indices.contiguous(), tys.contiguous()


def create_causal_omni_block_mask(
    batch: int, nheads: int, q_len: int, kv_len: int,
    Q_BLOCK_SIZE: int = 128, KV_BLOCK_SIZE: int = 128,
    device: Union[str, torch.device] = "cuda",
) -> OmniBlockMask:
    """Causal mask: FULL below the diagonal, CAUSAL on it, nothing above
    (omni_attn_torch.py:1950-2015).  The reference decides by ``kv_block <= q_block``,
    which assumes equal block sizes; here a KV block is listed when its first key is
    not after the query block's last row, and is FULL when its last key is not after
    the query block's first row -- identical for Q_BLOCK_SIZE == KV_BLOCK_SIZE."""
    QB, KB = Q_BLOCK_SIZE, KV_BLOCK_SIZE
    q_pad, kv_pad = _round_up(q_len, QB), _round_up(kv_len, KB)
    Tq, Tk = q_pad // QB, kv_pad // KB
    q0 = torch.arange(Tq, device=device).view(Tq, 1) * QB
    k0 = torch.arange(Tk, device=device).view(1, Tk) * KB
    active = k0 <= q0 + QB - 1
    full = (k0 + KB - 1) <= q0
    types = torch.where(full, int(BlockMaskType.FULL), int(BlockMaskType.CAUSAL))
    types = torch.where(active, types, torch.zeros_like(types))
    nb, idx, tys = _pack_slots(active, types)
    ex = lambda t: t.unsqueeze(0).unsqueeze(0).expand(batch, nheads, *t.shape).contiguous()
    return OmniBlockMask(ex(nb), ex(idx), ex(tys), q_pad, kv_pad, QB, KB)


def create_omni_block_mask_from_dense(
    dense_mask: Tensor,
    Q_BLOCK_SIZE: int = 128,
    KV_BLOCK_SIZE: int = 128,
    boundaries: Optional[Sequence[int]] = None,
    boundary_rule: str = "none",
) -> OmniBlockMask:
    """Classify every (q_block, kv_block) tile of a dense bool mask [B, H, S_q, S_kv].

    Rule of the reference's data generators (generate_attn_data.py:200-236): no True ->
    not listed; all True -> FULL; equal to the global causal pattern -> CAUSAL; anything
    else -> PARTIAL, with the tile stored.  ``boundaries`` reproduces the generators'
    extra rule for tiles whose query or key range strictly contains a segment boundary:
      boundary_rule="interleaved": such a tile, if not all True, is PARTIAL even when it
                                   equals the causal pattern (generate_attn_data.py:221-224);
      boundary_rule="document":    such a tile is PARTIAL even when all True
                                   (generate_attn_data.py:335-338).
    Lengths are padded to block multiples with False.
    """
    if boundary_rule not in ("none", "interleaved", "document"):
        raise ValueError("unknown boundary_rule")
    dense_mask = dense_mask.to(torch.bool)
    B, H, Sq, Sk = dense_mask.shape
    QB, KB = Q_BLOCK_SIZE, KV_BLOCK_SIZE
    q_pad, kv_pad = _round_up(Sq, QB), _round_up(Sk, KB)
    Tq, Tk = q_pad // QB, kv_pad // KB
    dense = _pad_dense(dense_mask, q_pad, kv_pad)
    dev = dense.device
    any_b = torch.empty(B, H, Tq, Tk, dtype=torch.bool, device=dev)
    all_b = torch.empty_like(any_b)
    caus_b = torch.empty_like(any_b)
    kk = torch.arange(kv_pad, device=dev).view(1, Tk, KB)
    for qb in range(Tq):  # one row of blocks at a time keeps the temporaries small
        slab = dense[:, :, qb * QB:(qb + 1) * QB, :].view(B, H, QB, Tk, KB)
        any_b[:, :, qb] = slab.any(-1).any(2)
        all_b[:, :, qb] = slab.all(-1).all(2)
        qq = torch.arange(qb * QB, (qb + 1) * QB, device=dev).view(QB, 1, 1)
        caus_b[:, :, qb] = (slab == (kk <= qq)).all(-1).all(2)
    types = torch.full((B, H, Tq, Tk), int(BlockMaskType.PARTIAL), dtype=torch.int64, device=dev)
    types = torch.where(caus_b, int(BlockMaskType.CAUSAL), types)
    types = torch.where(all_b, int(BlockMaskType.FULL), types)
    if boundaries is not None and boundary_rule != "none":
        bnd = torch.as_tensor(list(boundaries), device=dev).view(1, -1)
        q0 = torch.arange(Tq, device=dev).view(-1, 1) * QB
        k0 = torch.arange(Tk, device=dev).view(-1, 1) * KB
        # the generators clip block ends to the unpadded length
        q_cross = ((bnd > q0) & (bnd < torch.clamp(q0 + QB, max=Sq))).any(-1)
        k_cross = ((bnd > k0) & (bnd < torch.clamp(k0 + KB, max=Sk))).any(-1)
        cross = (q_cross.view(Tq, 1) | k_cross.view(1, Tk)).view(1, 1, Tq, Tk)
        if boundary_rule == "interleaved":
            types = torch.where(cross & ~all_b, int(BlockMaskType.PARTIAL), types)
        else:
            types = torch.where(cross, int(BlockMaskType.PARTIAL), types)
    types = torch.where(any_b, types, torch.zeros_like(types))
    nb, idx, tys = _pack_slots(any_b, types)
    mask = OmniBlockMask(nb, idx, tys, q_pad, kv_pad, QB, KB)
    if bool((tys == BlockMaskType.PARTIAL).any()):
        pidx, pm = build_partial_block_data(mask, dense)
        mask.partial_block_mask_indices = pidx
        mask.partial_block_masks = pm
    return mask


def modality_prefix_lengths(modality_positions: Tensor, seq_len: int) -> Tensor:
    """Row-wise allowed-prefix length of the Transfusion token rule.

    The rule (transfusion_pytorch/transfusion.py:496-515, same as :343-356) is
        allow[b, i, j] = (i >= j) or any_m (i >= off_m and j < off_m + len_m).
    Every term allows a prefix of the keys, so row i allows exactly the keys
    j < R[b, i] with R = max(i + 1, max over spans with off_m <= i of off_m + len_m).
    Returns R as int64 [B, seq_len].  Zero-length spans are inert.
    """
    mp = modality_positions.long()
    offs, lens = mp[..., 1], mp[..., 2]                       # [B, M]
    dev = mp.device
    i = torch.arange(seq_len, device=dev).view(1, seq_len, 1)
    ends = torch.where(lens > 0, offs + lens, torch.zeros_like(offs)).unsqueeze(1)  # [B,1,M]
    started = i >= offs.unsqueeze(1)                           # [B,S,M]
    reach = torch.where(started, ends, torch.zeros_like(ends)).amax(-1) if mp.shape[1] > 0 \
        else torch.zeros(mp.shape[0], seq_len, dtype=torch.long, device=dev)
    return torch.maximum(reach, i.squeeze(-1) + 1)


def naive_attn_mask(seq_len: int, modalities: Tensor, device=None) -> Tensor:
    """Dense Transfusion mask [B, seq_len, seq_len] (transfusion_pytorch/transfusion.py:496-515)."""
    modalities = modalities.to(device) if device is not None else modalities
    R = modality_prefix_lengths(modalities, seq_len)
    j = torch.arange(seq_len, device=R.device).view(1, 1, seq_len)
    return j < R.unsqueeze(-1)


def create_omni_block_mask_from_prefix_lengths(
    prefix_len: Tensor, nheads: int, q_len: int, kv_len: int,
    Q_BLOCK_SIZE: int = 128, KV_BLOCK_SIZE: int = 128,
) -> OmniBlockMask:
    """Block mask for a mask of the form ``allow[b, i, j] = j < prefix_len[b, i]`` with
    ``prefix_len >= i + 1`` nondecreasing in i, without materialising [S, S].

    Rows >= q_len and keys >= kv_len are padding (never attended / nothing allowed).
    Classification is the dense classifier's: nothing -> not listed, everything -> FULL,
    the global causal pattern -> CAUSAL, else PARTIAL with its tile stored once per
    batch element (heads share the tiles; their index tensors are equal).
    """
    QB, KB = Q_BLOCK_SIZE, KV_BLOCK_SIZE
    B = prefix_len.shape[0]
    dev = prefix_len.device
    q_pad, kv_pad = _round_up(q_len, QB), _round_up(kv_len, KB)
    Tq, Tk = q_pad // QB, kv_pad // KB
    R = torch.zeros(B, q_pad, dtype=torch.long, device=dev)
    R[:, :q_len] = torch.clamp(prefix_len[:, :q_len].long(), max=kv_len)
    rows = torch.arange(q_pad, device=dev)
    k0 = (torch.arange(Tk, device=dev) * KB).view(1, 1, Tk)
    # allowed keys of row i inside KV block kb form a prefix of length cnt[b, i, kb]
    cnt = torch.clamp(R.unsqueeze(-1) - k0, min=0, max=KB)            # [B, q_pad, Tk]
    cc = torch.clamp((rows + 1).view(1, -1, 1) - k0, min=0, max=KB)   # causal pattern
    cnt_b = cnt.view(B, Tq, QB, Tk)
    any_b = cnt_b.amax(2) > 0
    all_b = cnt_b.amin(2) == KB
    caus_b = (cnt_b == cc.view(1, Tq, QB, Tk)).all(2)
    types = torch.full((B, Tq, Tk), int(BlockMaskType.PARTIAL), dtype=torch.int64, device=dev)
    types = torch.where(caus_b, int(BlockMaskType.CAUSAL), types)
    types = torch.where(all_b, int(BlockMaskType.FULL), types)
    types = torch.where(any_b, types, torch.zeros_like(types))
    nb, idx, tys = _pack_slots(any_b, types)                          # [B,Tq], [B,Tq,Tk]
    pidx = None
    pm = None
    is_p = tys == BlockMaskType.PARTIAL
    if bool(is_p.any()):
        b_i, q_i, s_i = torch.nonzero(is_p, as_tuple=True)
        n = b_i.numel()
        pidx = torch.full((B, Tq, Tk), -1, dtype=torch.int32, device=dev)
        pidx[b_i, q_i, s_i] = torch.arange(n, dtype=torch.int32, device=dev)
        kvb = idx[b_i, q_i, s_i].long()
        c = cnt_b[b_i, q_i, :, kvb]                                   # [n, QB]
        pm = (torch.arange(KB, device=dev).view(1, 1, KB) < c.unsqueeze(-1)).contiguous()
        pidx = pidx.unsqueeze(1).expand(B, nheads, Tq, Tk).contiguous()
    ex = lambda t: t.unsqueeze(1).expand(B, nheads, *t.shape[1:]).contiguous()
    return OmniBlockMask(ex(nb), ex(idx), ex(tys), q_pad, kv_pad, QB, KB, pidx, pm)


def create_omni_block_mask_from_modality_positions(
    modality_positions: Tensor, batch: int, nheads: int, q_len: int, kv_len: int,
    Q_BLOCK_SIZE: int = 128, KV_BLOCK_SIZE: int = 128,
    device: Union[str, torch.device] = "cuda",
) -> OmniBlockMask:
    """Block mask of the Transfusion rule for ``modality_positions`` [B, M, 3] rows of
    (type, offset, length): text is causal, a span attends itself fully and everything
    before it (omni_attn_torch.py:1518-1736).

    The reference labels blocks with a dominant-type heuristic (:1596-1703) and takes the
    PARTIAL tiles from the token rule (:1723-1732).  Here every block is classified from
    the token rule itself, so the dense mask represented is always the token rule's;
    individual labels can differ from the heuristic's where that one is conservative
    (e.g. PARTIAL for a tile that is in fact all True).
    """
    assert modality_positions.shape[0] == batch, "modality_positions must be [batch, M, 3]"
    assert q_len == kv_len, "Q and KV sequence lengths must match"
    mp = modality_positions.to(device)
    R = modality_prefix_lengths(mp, q_len)
    return create_omni_block_mask_from_prefix_lengths(R, nheads, q_len, kv_len,
                                                      Q_BLOCK_SIZE, KV_BLOCK_SIZE)


# ----------------------------------------------------------------------------
# PyTorch attention (omni_attn_torch.py:302-387)
# ----------------------------------------------------------------------------

def naive_attention_with_dense_mask(query: Tensor, key: Tensor, value: Tensor,
                                    mask: Optional[Tensor] = None,
                                    scale: Optional[float] = None) -> Tensor:
    """softmax(Q K^T * scale + mask) V with ``mask`` 0 / -inf, [B, H, S_q, S_kv]."""
    D = query.shape[-1]
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    scores = torch.matmul(query, key.transpose(-2, -1)) * scale
    if mask is not None:
        scores = scores + mask.to(scores.dtype)
    weights = F.softmax(scores, dim=-1, dtype=torch.float32).to(query.dtype)
    return torch.matmul(weights, value)


def naive_attention(query: Tensor, key: Tensor, value: Tensor,
                    block_mask: Optional[OmniBlockMask] = None,
                    scale: Optional[float] = None) -> Tensor:
    mask = None if block_mask is None else block_mask.to_score_mask().to(query.device)
    return naive_attention_with_dense_mask(query, key, value, mask, scale)


# ----------------------------------------------------------------------------
# Operator wrappers (omni_attn_torch.py:517-1253)
# ----------------------------------------------------------------------------

def _load_extension():
    """``from omni_attn import ...`` with the directory of this file on the path, the
    place build.py puts the module (the reference looks there too, :548-552)."""
    try:
        return importlib.import_module("omni_attn")
    except ImportError:
        here = os.path.dirname(os.path.abspath(__file__))
        if here not in sys.path:
            sys.path.insert(0, here)
            try:
                return importlib.import_module("omni_attn")
            except ImportError:
                pass
        raise ImportError(
            "gfx950 extension module 'omni_attn' not found. Build it first:\n"
            "  python %s\n" % os.path.join(here, "build.py"))


def _pad_to_block_size(x: Tensor, BLOCK_SIZE: int) -> Tuple[Tensor, int]:
    """Zero-pad the sequence dimension (second to last) to a multiple of BLOCK_SIZE
    (omni_attn_torch.py:1261-1284)."""
    seq_len = x.shape[-2]
    padded_len = _round_up(seq_len, BLOCK_SIZE)
    if padded_len == seq_len:
        return x, seq_len
    return F.pad(x, (0, 0, 0, padded_len - seq_len)), seq_len


_SUPPORTED_HEAD_DIMS = (32, 64, 128)
_SUPPORTED_BLOCKS = (64, 128)


def _omni_attention(op_name: str, query: Tensor, key: Tensor, value: Tensor,
                    block_mask: OmniBlockMask, partial_needs_partial_types: bool,
                    return_lse: bool = False, keep_padded: bool = False, softcap: float = 0.0):
    ext = _load_extension()
    B, H, Q, D = query.shape
    KV = key.shape[2]
    assert key.shape == (B, H, KV, D), f"Key shape mismatch: {key.shape} vs expected {(B, H, KV, D)}"
    assert value.shape == (B, H, KV, D), f"Value shape mismatch: {value.shape} vs expected {(B, H, KV, D)}"
    assert Q == KV, f"Q and KV sequence lengths must match: Q={Q}, KV={KV}"
    if query.dtype not in (torch.float16, torch.bfloat16):
        raise ValueError(f"Unsupported dtype {query.dtype}. Supported: torch.float16, torch.bfloat16.")

    QB, KB = block_mask.Q_BLOCK_SIZE, block_mask.KV_BLOCK_SIZE
    query_padded, q_orig_len = _pad_to_block_size(query, QB)
    key_padded, _ = _pad_to_block_size(key, KB)
    value_padded, _ = _pad_to_block_size(value, KB)
    # Q, K and V share one padded length in the kernel; with QB != KB pad to the larger.
    S_pad = max(query_padded.shape[2], key_padded.shape[2])
    assert query_padded.shape[2] == block_mask.q_len, \
        f"Padded Q length ({query_padded.shape[2]}) doesn't match mask q_len ({block_mask.q_len})"
    assert key_padded.shape[2] == block_mask.kv_len, \
        f"Padded KV length ({key_padded.shape[2]}) doesn't match mask kv_len ({block_mask.kv_len})"
    if query_padded.shape[2] != S_pad:
        query_padded = F.pad(query_padded, (0, 0, 0, S_pad - query_padded.shape[2]))
    if key_padded.shape[2] != S_pad:
        key_padded = F.pad(key_padded, (0, 0, 0, S_pad - key_padded.shape[2]))
        value_padded = F.pad(value_padded, (0, 0, 0, S_pad - value_padded.shape[2]))

    num_q_blocks = block_mask.q_len // QB
    assert block_mask.kv_num_blocks.shape == (B, H, num_q_blocks), \
        f"kv_num_blocks shape mismatch: {block_mask.kv_num_blocks.shape} vs expected {(B, H, num_q_blocks)}"
    max_blocks = block_mask.kv_indices.shape[3]
    assert block_mask.kv_indices.shape == (B, H, num_q_blocks, max_blocks), \
        f"kv_indices shape mismatch: {block_mask.kv_indices.shape} vs expected {(B, H, num_q_blocks, max_blocks)}"
    assert block_mask.block_mask_types.shape == (B, H, num_q_blocks, max_blocks), \
        f"block_mask_types shape mismatch: {block_mask.block_mask_types.shape} vs expected {(B, H, num_q_blocks, max_blocks)}"
    if S_pad != block_mask.q_len:
        raise ValueError(
            f"q_len ({block_mask.q_len}) must be a multiple of KV_BLOCK_SIZE ({KB}) so that Q, K and V "
            f"share one padded length")

    # the scalar entry point takes any block size and head_dim <= 256, like the reference's
    # (attn_naive.cu:189-190, :305-408); the others only the shapes with an MFMA instance
    if op_name == "omni_attn_simple_kernel":
        if not 0 < D <= 256:
            raise ValueError(f"Unsupported head_dim={D}. Supported values: 1..256.")
    else:
        if D not in _SUPPORTED_HEAD_DIMS:
            raise ValueError(f"Unsupported head_dim={D}. Supported values: 32, 64, 128.")
        if QB not in _SUPPORTED_BLOCKS:
            raise ValueError(f"Unsupported Q_BLOCK_SIZE={QB}. Supported values: 64, 128.")
        if KB not in _SUPPORTED_BLOCKS:
            raise ValueError(f"Unsupported KV_BLOCK_SIZE={KB}. Supported values: 64, 128.")

    dev = query.device
    query_padded = query_padded.contiguous()
    key_padded = key_padded.contiguous()
    value_padded = value_padded.contiguous()
    output_padded = torch.empty_like(query_padded)
    kv_num_blocks = block_mask.kv_num_blocks.to(device=dev, dtype=torch.int32).contiguous()
    kv_indices = block_mask.kv_indices.to(device=dev, dtype=torch.int32).contiguous()
    block_mask_types = block_mask.block_mask_types.to(device=dev, dtype=torch.int32).contiguous()

    has_partial = (block_mask.partial_block_mask_indices is not None
                   and block_mask.partial_block_masks is not None)
    if partial_needs_partial_types:
        # the simple / cp_async / prefetch wrappers also require a PARTIAL slot to exist
        has_partial = has_partial and block_mask.has_partial_slots()
    if has_partial:
        partial_idx = block_mask.partial_block_mask_indices.to(device=dev, dtype=torch.int32).contiguous()
        partial_masks = block_mask.partial_block_masks.to(device=dev, dtype=torch.bool).contiguous()
    else:
        partial_idx = torch.empty(0, dtype=torch.int32, device=dev)
        partial_masks = torch.empty(0, dtype=torch.bool, device=dev)

    if has_partial and block_mask.partial_block_bits is not None and block_mask.partial_block_bits.device == dev:
        # tiles packed once by OmniBlockMask.pack_partial_masks(): same kernel, packed input
        lse_padded = (torch.empty(B, H, S_pad, dtype=torch.float32, device=dev) if (return_lse or keep_padded)
                      else torch.empty(0, dtype=torch.float32, device=dev))
        ext.omni_attn_forward_packed(query_padded, key_padded, value_padded, output_padded, lse_padded,
                                     kv_num_blocks, kv_indices, block_mask_types, QB, KB, q_orig_len,
                                     partial_idx, block_mask.partial_block_bits.contiguous(), float(softcap))
        if keep_padded:
            return output_padded, lse_padded, query_padded, key_padded, value_padded, q_orig_len
        if return_lse:
            return output_padded[:, :, :q_orig_len, :], lse_padded[:, :, :q_orig_len]
        return output_padded[:, :, :q_orig_len, :]
    if return_lse or softcap:
        lse_padded = torch.empty(B, H, S_pad, dtype=torch.float32, device=dev)
        ext.omni_attn_forward(query_padded, key_padded, value_padded, output_padded, lse_padded,
                              kv_num_blocks, kv_indices, block_mask_types, QB, KB, q_orig_len,
                              partial_idx, partial_masks, has_partial, float(softcap))
        if keep_padded:
            return output_padded, lse_padded, query_padded, key_padded, value_padded, q_orig_len
        if not return_lse:
            return output_padded[:, :, :q_orig_len, :]
        return output_padded[:, :, :q_orig_len, :], lse_padded[:, :, :q_orig_len]
    getattr(ext, op_name)(query_padded, key_padded, value_padded, output_padded,
                          kv_num_blocks, kv_indices, block_mask_types, QB, KB, q_orig_len,
                          partial_idx, partial_masks, has_partial)
    return output_padded[:, :, :q_orig_len, :]


def omni_attention_shared_kv(query: Tensor, key: Tensor, value: Tensor, block_mask: OmniBlockMask,
                             scale: Optional[float] = None) -> Tensor:
    """omni_attn_torch.py:517-671.  ``scale`` is accepted and ignored as in the reference:
    the kernel always uses 1/sqrt(head_dim)."""
    return _omni_attention("omni_attn_mma_stages_split_q_shared_kv", query, key, value, block_mask, False)


def omni_attention_simple(query: Tensor, key: Tensor, value: Tensor, block_mask: OmniBlockMask) -> Tensor:
    """omni_attn_torch.py:673-809."""
    return _omni_attention("omni_attn_simple_kernel", query, key, value, block_mask, True)


def omni_attention_cp_async(query: Tensor, key: Tensor, value: Tensor, block_mask: OmniBlockMask) -> Tensor:
    """omni_attn_torch.py:812-964."""
    return _omni_attention("omni_attn_cp_async", query, key, value, block_mask, True)


def omni_attention_preftech(query: Tensor, key: Tensor, value: Tensor, block_mask: OmniBlockMask,
                            scale: Optional[float] = None) -> Tensor:
    """omni_attn_torch.py:967-1110."""
    return _omni_attention("omni_attn_preftech_kernel", query, key, value, block_mask, True)


def omni_attention_shared_kv_swizzle(query: Tensor, key: Tensor, value: Tensor,
                                     block_mask: OmniBlockMask,
                                     scale: Optional[float] = None) -> Tensor:
    """omni_attn_torch.py:1113-1253."""
    return _omni_attention("omni_attn_mma_stages_split_q_shared_kv_swizzle", query, key, value,
                           block_mask, False)


def omni_attention_forward(query: Tensor, key: Tensor, value: Tensor,
                           block_mask: OmniBlockMask, softcap: float = 0.0) -> Tuple[Tensor, Tensor]:
    """Output and fp32 row logsumexp [B, H, S] (-inf for rows with no allowed key).
    Not in the reference, which has no logsumexp output."""
    return _omni_attention("omni_attn_forward", query, key, value, block_mask, False, return_lse=True,
                           softcap=softcap)


class _OmniAttentionFunction(torch.autograd.Function):
    """Forward and backward kernels as one differentiable operator.  The reference's operator
    cannot be differentiated (it has no backward and no logsumexp output); this is the form a
    training loop needs, e.g. in place of the flex_attention call of
    transfusion_pytorch/transfusion.py:953-983."""

    @staticmethod
    def forward(ctx, query, key, value, block_mask, softcap):
        out_padded, lse_padded, q_pad, k_pad, v_pad, seq_len = _omni_attention(
            "omni_attn_forward", query, key, value, block_mask, False, return_lse=True, keep_padded=True,
            softcap=softcap)
        ctx.save_for_backward(q_pad, k_pad, v_pad, out_padded, lse_padded)
        ctx.block_mask = block_mask
        ctx.seq_len = seq_len
        ctx.softcap = float(softcap)
        return out_padded[:, :, :seq_len, :]

    @staticmethod
    def backward(ctx, grad_out):
        ext = _load_extension()
        q_pad, k_pad, v_pad, out_padded, lse_padded = ctx.saved_tensors
        m, seq_len = ctx.block_mask, ctx.seq_len
        dev = q_pad.device
        S_pad = q_pad.shape[2]
        d_out = grad_out.to(q_pad.dtype)
        if S_pad != seq_len:
            d_out = F.pad(d_out, (0, 0, 0, S_pad - seq_len))
        d_out = d_out.contiguous()
        dq, dk, dv = torch.empty_like(q_pad), torch.empty_like(q_pad), torch.empty_like(q_pad)
        to_i32 = lambda t: t.to(device=dev, dtype=torch.int32).contiguous()
        has_partial = m.partial_block_mask_indices is not None and m.partial_block_masks is not None
        packed = has_partial and m.partial_block_bits is not None and m.partial_block_bits.device == dev
        if has_partial:
            pidx = to_i32(m.partial_block_mask_indices)
            tiles = (m.partial_block_bits.contiguous() if packed
                     else m.partial_block_masks.to(device=dev, dtype=torch.bool).contiguous())
        else:
            pidx = torch.empty(0, dtype=torch.int32, device=dev)
            tiles = torch.empty(0, dtype=torch.bool, device=dev)
        ext.omni_attn_backward(q_pad, k_pad, v_pad, out_padded, d_out, lse_padded, dq, dk, dv,
                               to_i32(m.kv_num_blocks), to_i32(m.kv_indices), to_i32(m.block_mask_types),
                               m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE, seq_len, pidx, tiles, has_partial, packed,
                               ctx.softcap)
        return dq[:, :, :seq_len, :], dk[:, :, :seq_len, :], dv[:, :, :seq_len, :], None, None


def omni_attention(query: Tensor, key: Tensor, value: Tensor, block_mask: OmniBlockMask,
                   softcap: float = 0.0) -> Tensor:
    """Differentiable block-sparse attention: the forward kernel, with the backward kernels
    behind ``.backward()`` (gradients with respect to query, key and value).  ``softcap`` > 0
    replaces the scaled score x by softcap * tanh(x / softcap) before mask and softmax
    (transfusion_pytorch/transfusion.py:358-364)."""
    return _OmniAttentionFunction.apply(query, key, value, block_mask, float(softcap))


# ----------------------------------------------------------------------------
# Utilities (omni_attn_torch.py:1287-1364, generate_attn_data.py:87-107)
# ----------------------------------------------------------------------------

def check_correctness(ref_output: Tensor, test_output: Tensor, rtol: float = 1e-2,
                      atol: float = 1e-3, name: str = "test") -> bool:
    """Shape / NaN / Inf diagnostics and ``allclose``; prints PASSED or FAILED."""
    if test_output is None:
        print(f"[{name}] test_output is None")
        return False
    if ref_output.shape != test_output.shape:
        print(f"[{name}] Shape mismatch: {ref_output.shape} vs {test_output.shape}")
        return False
    ref = ref_output.float()
    out = test_output.float().to(ref.device)
    total = out.numel()
    nan_out = int(torch.isnan(out).sum())
    if int((out == 0).sum()) == total:
        print(f"[{name}] WARNING: test_output is all zeros (possibly uninitialized)")
    elif nan_out == total:
        print(f"[{name}] WARNING: test_output is all NaN (kernel may have failed)")
    for label, t in (("ref_output", ref), ("test_output", out)):
        n_nan, n_inf = int(torch.isnan(t).sum()), int(torch.isinf(t).sum())
        if n_nan:
            print(f"[{name}] WARNING: {label} contains {n_nan} NaN values")
        if n_inf:
            print(f"[{name}] WARNING: {label} contains {n_inf} Inf values")
    diff = (ref - out).abs()
    passed = bool(torch.allclose(ref, out, rtol=rtol, atol=atol))
    print(f"[{name}] {'PASSED' if passed else 'FAILED'} (max_diff={diff.max().item():.6f}, "
          f"mean_diff={diff.mean().item():.6f}), min_diff={diff.min().item():.6f}")
    return passed


def block_pattern_rows(block_mask: OmniBlockMask, b: int = 0, h: int = 0) -> List[str]:
    """One string per query block, one letter per KV block: F, C, P, or a space, joined
    by single spaces -- the layout the reference's generators print
    (generate_attn_data.py:87-107)."""
    letters = {int(BlockMaskType.FULL): "F", int(BlockMaskType.CAUSAL): "C",
               int(BlockMaskType.PARTIAL): "P"}
    Tk = block_mask.num_kv_blocks
    rows = []
    nb = block_mask.kv_num_blocks[b, h].tolist()
    idx = block_mask.kv_indices[b, h].tolist()
    tys = block_mask.block_mask_types[b, h].tolist()
    for qb in range(len(nb)):
        cells = [" "] * Tk
        for s in range(nb[qb]):
            cells[idx[qb][s]] = letters.get(tys[qb][s], " ")
        rows.append(" ".join(cells))
    return rows
