"""Seeded synthetic workloads: the five benchmark configurations of this build.

Counterpart of the reference's data generators (omni-attn-mma/generate_attn_data.py,
generate_debug_data.py): seeded q/k/v drawn in fp32 and cast once, a span layout drawn
from the same generator, and the block mask built from it.  Everything is produced on
the CPU from ``torch.Generator().manual_seed(seed)`` so the same inputs can be rebuilt
anywhere.  Masks are described by the per-row allowed-prefix length ``prefix_len``
(allow[b, i, j] = j < prefix_len[b, i]), which is what the Transfusion token rule and
plain causal / full masks all reduce to (see omni_attn_torch.modality_prefix_lengths).
"""
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch

from omni_attn_torch import (OmniBlockMask, create_omni_block_mask_from_prefix_lengths,
                             modality_prefix_lengths)


@dataclass
class Workload:
    name: str
    q: torch.Tensor                 # [B, H, S, D] in `dtype`, CPU
    k: torch.Tensor
    v: torch.Tensor
    block_mask: OmniBlockMask       # CPU tensors
    prefix_len: torch.Tensor        # [B, S] int64: allow[b, i, j] = j < prefix_len[b, i]
    spans: List[List[Tuple[int, int]]]  # per batch element: (offset, length) of image spans
    dtype: torch.dtype
    info: Dict = field(default_factory=dict)

    @property
    def nonempty_blocks(self) -> int:
        return int(self.block_mask.kv_num_blocks.sum().item())

    @property
    def effective_flops(self) -> float:
        """4 * QB * KB * D per listed block: two GEMMs, 2 flop per multiply-add; CAUSAL and
        PARTIAL blocks count as full tiles, softmax flops are not counted."""
        D = self.info["D"]
        return 4.0 * self.block_mask.Q_BLOCK_SIZE * self.block_mask.KV_BLOCK_SIZE * D * self.nonempty_blocks


SPECS = {
    # name: (B, H, S, D, dtype, QB, KB)
    "c1_causal": (1, 8, 512, 64, torch.float16, 128, 128),
    "c2_interleaved": (2, 32, 4096, 128, torch.bfloat16, 128, 128),
    "c2_interleaved_8k": (1, 32, 8192, 128, torch.bfloat16, 128, 128),
    "c3_partial": (1, 16, 8192, 128, torch.bfloat16, 128, 64),
    "c4_long": (1, 32, 16384, 128, torch.bfloat16, 128, 128),
    "c5_batched": (8, 16, 8192, 64, torch.float16, 128, 128),
    "c5_full_control": (8, 16, 8192, 64, torch.float16, 128, 128),
}


def _randint(gen, lo: int, hi: int) -> int:
    """Uniform integer in [lo, hi]."""
    return int(torch.randint(lo, hi + 1, (1,), generator=gen).item())


def _interleaved_spans(gen, S: int, text_lo: int, text_hi: int, image_len: int, align: int,
                       max_images: Optional[int] = None) -> List[Tuple[int, int]]:
    """text, image, text, image, ... until S: text length U{text_lo..text_hi}; each image
    starts at the next multiple of ``align`` (the preceding text is extended up to it) and
    has ``image_len`` tokens; an image that would not fit is dropped and text fills the rest."""
    spans = []
    pos = 0
    while True:
        pos += _randint(gen, text_lo, text_hi)
        start = ((pos + align - 1) // align) * align
        if start + image_len > S or (max_images is not None and len(spans) >= max_images):
            break
        spans.append((start, image_len))
        pos = start + image_len
    return spans


def _random_spans(gen, S: int, count: int, len_lo: int, len_hi: int, aligned_to: int = 1) -> List[Tuple[int, int]]:
    """``count`` non-overlapping spans with lengths U{len_lo..len_hi} at random offsets:
    the free text (S minus the span lengths) is cut at ``count`` sorted random points."""
    lens = [_randint(gen, len_lo, len_hi) for _ in range(count)]
    while sum(lens) > S - count - 1 and lens:
        lens.pop()
    free = S - sum(lens)
    cuts = sorted(_randint(gen, 1, free - 1) for _ in lens)
    spans = []
    shift = 0
    for cut, ln in zip(cuts, lens):
        start = cut + shift
        if aligned_to > 1:
            start = (start // aligned_to) * aligned_to
            if spans and start < spans[-1][0] + spans[-1][1]:
                start = ((spans[-1][0] + spans[-1][1] + aligned_to - 1) // aligned_to) * aligned_to
        if start + ln > S:
            break
        spans.append((start, ln))
        shift += ln
    return spans


def _prefix_from_spans(spans_per_batch, S: int) -> torch.Tensor:
    B = len(spans_per_batch)
    M = max([len(s) for s in spans_per_batch] + [1])
    mp = torch.zeros(B, M, 3, dtype=torch.long)
    for b, spans in enumerate(spans_per_batch):
        for m, (off, ln) in enumerate(spans):
            mp[b, m, 0], mp[b, m, 1], mp[b, m, 2] = 1, off, ln
    return modality_prefix_lengths(mp, S)


def make_workload(name: str, seed: int = 0, B: Optional[int] = None, H: Optional[int] = None,
                  S: Optional[int] = None, with_qkv: bool = True) -> Workload:
    """Build one configuration.  B / H / S override the shape (used by tests to shrink a
    configuration; the layout rules stay the same)."""
    if name not in SPECS:
        raise KeyError("unknown workload %r (known: %s)" % (name, ", ".join(SPECS)))
    B0, H0, S0, D, dtype, QB, KB = SPECS[name]
    B, H, S = B or B0, H or H0, S or S0
    gen = torch.Generator(device="cpu").manual_seed(seed)
    info: Dict = {"seed": seed}

    spans: List[List[Tuple[int, int]]] = []
    prefix = None
    if name == "c1_causal":
        spans = [[] for _ in range(B)]
    elif name in ("c2_interleaved", "c2_interleaved_8k"):
        spans = [_interleaved_spans(gen, S, 128, 512, 1024, 128) for _ in range(B)]
    elif name == "c3_partial":
        # one image of 200..1100 tokens per 1024 tokens, at arbitrary (unaligned) offsets
        spans = [_random_spans(gen, S, max(1, S // 1024), 200, 1100) for _ in range(B)]
    elif name == "c4_long":
        spans = [_random_spans(gen, S, max(1, S // 2048), 1024, 1024) for _ in range(B)]
    elif name == "c5_batched":
        kinds = []
        for b in range(B):
            kind = ("causal", "full", "interleaved")[b % 3]
            kinds.append(kind)
            if kind == "interleaved":
                spans.append(_interleaved_spans(gen, S, 128, 1024, 1024, 128, max_images=_randint(gen, 0, 6)))
            else:
                spans.append([])
        info["layouts"] = kinds
        prefix = _prefix_from_spans(spans, S)
        for b, kind in enumerate(kinds):
            if kind == "full":
                prefix[b, :] = S
    elif name == "c5_full_control":
        spans = [[] for _ in range(B)]
        prefix = torch.full((B, S), S, dtype=torch.long)
    if prefix is None:
        prefix = _prefix_from_spans(spans, S)

    mask = create_omni_block_mask_from_prefix_lengths(prefix, H, S, S, QB, KB)

    q = k = v = torch.empty(0)
    if with_qkv:
        scale = D ** -0.5 if name == "c3_partial" else 1.0
        q, k, v = ((torch.randn(B, H, S, D, generator=gen, dtype=torch.float32) * scale).to(dtype)
                   for _ in range(3))
    info.update({"B": B, "H": H, "S": S, "D": D, "Q_BLOCK_SIZE": QB, "KV_BLOCK_SIZE": KB,
                 "dtype": str(dtype).replace("torch.", "")})
    return Workload(name, q, k, v, mask, prefix, spans, dtype, info)
