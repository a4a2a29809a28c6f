"""fp32 dense-mask attention oracle (test infrastructure, see oracle/__init__.py).

Follows naive_attention_with_dense_mask (omni-attn-mma/omni_attn_torch.py:348-387):
scores = Q K^T / sqrt(D), masked positions -> -inf, softmax in fp32, times V.  Run in
fp32 the reference's cast of the weights to the query dtype (:384) is the identity.
Adds the row logsumexp and the kernels' convention for rows with no allowed key:
output 0 (omni-attn-mma/mma/attn_naive.cu:177-183), logsumexp -inf.
"""
import math
from typing import Optional, Tuple

import torch


def attention_dense_fp32(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                         mask: torch.Tensor, row_chunk: int = 2048,
                         softcap: float = 0.0) -> Tuple[torch.Tensor, torch.Tensor]:
    """q, k, v: [..., S, D] (any float dtype, converted to fp32 as they are);
    mask: bool, broadcastable to [..., S, S], True = attend.
    softcap > 0: scaled scores x become softcap * tanh(x / softcap) before the mask, the way
    Transfusion's attention layer does it (transfusion_pytorch/transfusion.py:298-299 softclamp,
    :358-364 the flex score_mod, :966-968 the dense path).
    Returns (O fp32 [..., S, D], LSE fp32 [..., S])."""
    qf, kf, vf = q.float(), k.float(), v.float()
    S, D = qf.shape[-2], qf.shape[-1]
    scale = 1.0 / math.sqrt(D)
    out = torch.empty(qf.shape[:-1] + (vf.shape[-1],), dtype=torch.float32, device=qf.device)
    lse = torch.empty(qf.shape[:-1], dtype=torch.float32, device=qf.device)
    for r0 in range(0, S, row_chunk):
        r1 = min(S, r0 + row_chunk)
        s = torch.matmul(qf[..., r0:r1, :], kf.transpose(-1, -2)) * scale
        if softcap > 0:
            s = torch.tanh(s / softcap) * softcap
        m = mask[..., r0:r1, :]
        s = s.masked_fill(~m, float("-inf"))
        any_row = m.any(-1)
        l = torch.logsumexp(s, dim=-1)
        # softmax of an all -inf row is NaN in torch; those rows are defined as 0
        p = torch.softmax(s, dim=-1)
        p = torch.where(any_row.unsqueeze(-1), p, torch.zeros_like(p))
        out[..., r0:r1, :] = torch.matmul(p, vf)
        lse[..., r0:r1] = torch.where(any_row, l, torch.full_like(l, float("-inf")))
    return out, lse


def attention_dense_differentiable(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                                   mask: torch.Tensor, softcap: float = 0.0) -> torch.Tensor:
    """The same function as attention_dense_fp32 (output only) written so that autograd can
    go through it, in the dtype of its inputs (fp32, or fp64 for gradcheck): rows with no
    allowed key give 0 and pass no gradient."""
    D = q.shape[-1]
    s = torch.matmul(q, k.transpose(-1, -2)) / math.sqrt(D)
    if softcap > 0:
        s = torch.tanh(s / softcap) * softcap
    any_row = mask.any(-1, keepdim=True)
    s = s.masked_fill(~mask, float("-inf"))
    s = torch.where(any_row, s, torch.zeros_like(s))  # keeps softmax finite on empty rows
    p = torch.softmax(s, dim=-1)
    p = torch.where(any_row, p, torch.zeros_like(p))
    return torch.matmul(p, v)


def attention_dense_grads(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: torch.Tensor,
                          dout: torch.Tensor, softcap: float = 0.0) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dQ, dK, dV) of sum(O * dout) by autograd through attention_dense_differentiable in fp32
    (inputs of any float dtype are converted as they are)."""
    qf, kf, vf = (t.detach().float().clone().requires_grad_(True) for t in (q, k, v))
    out = attention_dense_differentiable(qf, kf, vf, mask, softcap)
    out.backward(dout.float())
    return qf.grad, kf.grad, vf.grad


def attention_dense_grads_closed_form(q, k, v, mask, dout):
    """The textbook closed form, written out with no autograd: P = softmax(mask(QK^T/sqrt(D))),
    delta_i = sum_d dO_id O_id, dV = P^T dO, dS = P * (dO V^T - delta), dQ = dS K / sqrt(D),
    dK = dS^T Q / sqrt(D).  Pins attention_dense_grads (and is pinned by gradcheck with it)."""
    qf, kf, vf, do = q.float(), k.float(), v.float(), dout.float()
    scale = 1.0 / math.sqrt(qf.shape[-1])
    s = torch.matmul(qf, kf.transpose(-1, -2)) * scale
    any_row = mask.any(-1, keepdim=True)
    s = torch.where(any_row, s.masked_fill(~mask, float("-inf")), torch.zeros_like(s))
    p = torch.where(any_row, torch.softmax(s, dim=-1), torch.zeros_like(s))
    o = torch.matmul(p, vf)
    delta = (do * o).sum(-1, keepdim=True)
    dv = torch.matmul(p.transpose(-1, -2), do)
    ds = p * (torch.matmul(do, vf.transpose(-1, -2)) - delta)
    return torch.matmul(ds, kf) * scale, torch.matmul(ds.transpose(-1, -2), qf) * scale, dv


def attention_dense_grads_chunked(q, k, v, mask, dout, row_chunk: int = 2048, softcap: float = 0.0):
    """The closed form of attention_dense_grads_closed_form worked over blocks of query rows, so
    that one [S, S] slab at S = 16384 needs a few hundred MB instead of several GB (q, k, v, dout:
    [S, D]; mask: [S, S] bool).  With softcap > 0 the score gradient carries the derivative of
    softcap * tanh(x / softcap), 1 - tanh^2.  Pinned against autograd in tests/test_oracle_pinning.py."""
    qf, kf, vf, do = q.float(), k.float(), v.float(), dout.float()
    S, D = qf.shape
    scale = 1.0 / math.sqrt(D)
    dq = torch.zeros_like(qf)
    dk = torch.zeros_like(kf)
    dv = torch.zeros_like(vf)
    for r0 in range(0, S, row_chunk):
        r1 = min(S, r0 + row_chunk)
        m = mask[r0:r1]
        x = torch.matmul(qf[r0:r1], kf.t()) * scale
        dfac = None
        if softcap > 0:
            t = torch.tanh(x / softcap)
            x = t * softcap
            dfac = 1.0 - t * t
        any_row = m.any(-1, keepdim=True)
        x = torch.where(any_row, x.masked_fill(~m, float("-inf")), torch.zeros_like(x))
        p = torch.where(any_row, torch.softmax(x, dim=-1), torch.zeros_like(x))
        o = torch.matmul(p, vf)
        delta = (do[r0:r1] * o).sum(-1, keepdim=True)
        dv += torch.matmul(p.t(), do[r0:r1])
        ds = p * (torch.matmul(do[r0:r1], vf.t()) - delta)
        if dfac is not None:
            ds = ds * dfac
        dq[r0:r1] = torch.matmul(ds, kf) * scale
        dk += torch.matmul(ds.t(), qf[r0:r1]) * scale
    return dq, dk, dv


def prefix_mask(prefix_len: torch.Tensor, kv_len: int) -> torch.Tensor:
    """allow[..., i, j] = j < prefix_len[..., i]."""
    j = torch.arange(kv_len, device=prefix_len.device)
    return j < prefix_len.unsqueeze(-1)


def transfusion_mask_bruteforce(seq_len: int, spans) -> torch.Tensor:
    """Token rule of transfusion_pytorch/transfusion.py:496-515 written as loops:
    allow[i, j] = (i >= j) or any span (off, length): i >= off and j < off + length."""
    allow = torch.zeros(seq_len, seq_len, dtype=torch.bool)
    for i in range(seq_len):
        for j in range(seq_len):
            ok = i >= j
            for off, length in spans:
                if i >= off and j < off + length:
                    ok = True
            allow[i, j] = ok
    return allow


def dense_mask_from_blocks(kv_num_blocks, kv_indices, block_mask_types, QB: int, KB: int,
                           q_len: int, kv_len: int, partial_idx=None, partial_masks=None,
                           seqlen_orig: Optional[int] = None) -> torch.Tensor:
    """Dense mask the kernels realise for given block metadata, as plain loops over the
    slots (scalar-kernel semantics, omni-attn-mma/mma/attn_naive.cu:95-175): MASKED and
    PARTIAL-without-bits slots are skipped, CAUSAL is k_global <= q_global, keys and
    rows at or beyond seqlen_orig are dropped."""
    B, H, Tq, _ = kv_indices.shape
    seqlen = q_len if seqlen_orig is None else min(seqlen_orig, q_len)
    dense = torch.zeros(B, H, q_len, kv_len, dtype=torch.bool)
    nb = kv_num_blocks.tolist()
    idx = kv_indices.tolist()
    tys = block_mask_types.tolist()
    pid = partial_idx.tolist() if partial_idx is not None else None
    for b in range(B):
        for h in range(H):
            for qb in range(Tq):
                q0, q1 = qb * QB, min(qb * QB + QB, q_len)
                for s in range(nb[b][h][qb]):
                    kb, ty = idx[b][h][qb][s], tys[b][h][qb][s]
                    k0, k1 = kb * KB, min(kb * KB + KB, kv_len)
                    if ty == 2:
                        dense[b, h, q0:q1, k0:k1] = True
                    elif ty == 1:
                        qq = torch.arange(q0, q1).view(-1, 1)
                        kk = torch.arange(k0, k1).view(1, -1)
                        dense[b, h, q0:q1, k0:k1] = kk <= qq
                    elif ty == 3:
                        if pid is None or partial_masks is None or pid[b][h][qb][s] < 0:
                            continue
                        dense[b, h, q0:q1, k0:k1] = partial_masks[pid[b][h][qb][s]][: q1 - q0, : k1 - k0]
    dense[:, :, seqlen:, :] = False
    dense[:, :, :, seqlen:] = False
    return dense
