"""Shared helpers for the tests (not collected)."""
import json
import os

import torch

HERE = os.path.dirname(os.path.abspath(__file__))

# Tolerances against the fp32 oracle on identical, already rounded inputs.
TOL_O = {torch.float16: 2e-3, torch.bfloat16: 1e-2}
TOL_LSE = 1e-3


def load_printed_masks():
    with open(os.path.join(HERE, "golden", "printed_masks.json")) as f:
        return json.load(f)


def typed_pattern_to_metadata(rows, with_bits=True, QB=128, KB=128):
    """Rows of F/C/P letters (slot order = KV block order) -> metadata tensors with the
    PARTIAL tiles the reference's debug-data generator uses: upper half of the query rows
    all True, lower half k_global <= q_global."""
    Tq = len(rows)
    Tk = max(len(r) for r in rows)
    code = {"C": 1, "F": 2, "P": 3}
    nb = torch.zeros(1, 1, Tq, dtype=torch.int32)
    idx = torch.zeros(1, 1, Tq, Tk, dtype=torch.int32)
    tys = torch.zeros(1, 1, Tq, Tk, dtype=torch.int32)
    pidx = torch.full((1, 1, Tq, Tk), -1, dtype=torch.int32)
    tiles = []
    for qb, row in enumerate(rows):
        nb[0, 0, qb] = len(row)
        for s, ch in enumerate(row):
            idx[0, 0, qb, s] = s
            tys[0, 0, qb, s] = code[ch]
            if ch == "P" and with_bits:
                qq = torch.arange(qb * QB, qb * QB + QB).view(-1, 1)
                kk = torch.arange(s * KB, s * KB + KB).view(1, -1)
                pidx[0, 0, qb, s] = len(tiles)
                tiles.append((kk <= qq) | (qq < qb * QB + QB // 2))
    pm = torch.stack(tiles) if tiles else None
    return nb, idx, tys, (pidx if tiles else None), pm


def random_block_metadata(gen, B, H, Tq, Tk, QB, KB, p_empty=0.3, with_partial=True,
                          with_masked_slots=True, with_bitless_partial=True, shuffle=False):
    """Random typed metadata exercising every slot kind the kernels distinguish."""
    nb = torch.zeros(B, H, Tq, dtype=torch.int32)
    idx = torch.zeros(B, H, Tq, Tk, dtype=torch.int32)
    tys = torch.zeros(B, H, Tq, Tk, dtype=torch.int32)
    pidx = torch.full((B, H, Tq, Tk), -1, dtype=torch.int32)
    tiles = []
    for b in range(B):
        for h in range(H):
            for qb in range(Tq):
                cols = [kb for kb in range(Tk) if torch.rand((), generator=gen).item() > p_empty]
                if (b, h, qb) == (0, 0, Tq - 1):
                    cols = []  # a query block with nothing listed: rows of zeros
                if shuffle:
                    perm = torch.randperm(len(cols), generator=gen).tolist()
                    cols = [cols[i] for i in perm]
                nb[b, h, qb] = len(cols)
                for s, kb in enumerate(cols):
                    r = torch.rand((), generator=gen).item()
                    if r < 0.35:
                        ty = 2
                    elif r < 0.6:
                        ty = 1
                    elif r < 0.9 and with_partial:
                        ty = 3
                    elif with_masked_slots:
                        ty = 0
                    else:
                        ty = 2
                    idx[b, h, qb, s] = kb
                    tys[b, h, qb, s] = ty
                    if ty == 3:
                        if with_bitless_partial and torch.rand((), generator=gen).item() < 0.15:
                            continue  # PARTIAL slot without bits: must be skipped
                        dens = torch.rand((), generator=gen).item()
                        tile = torch.rand(QB, KB, generator=gen) < dens
                        if torch.rand((), generator=gen).item() < 0.3:
                            tile[: QB // 2] = False  # fully masked rows inside a listed block
                        pidx[b, h, qb, s] = len(tiles)
                        tiles.append(tile)
    pm = torch.stack(tiles) if tiles else None
    return nb, idx, tys, (pidx if tiles else None), pm


def max_abs(a, b):
    return (a.float() - b.float()).abs().max().item()


def compare_with_oracle(o, lse, ref_o, ref_lse, dtype, what=""):
    """Assert the north-star bars: max-abs on O, 1e-3 on LSE, empty rows exact."""
    o = o.float().cpu()
    lse = lse.float().cpu()
    assert not torch.isnan(o).any(), f"{what}: NaN in output"
    empty = torch.isinf(ref_lse) & (ref_lse < 0)
    assert torch.equal(torch.isinf(lse) & (lse < 0), empty), f"{what}: empty-row set differs"
    assert not torch.isnan(lse).any(), f"{what}: NaN in logsumexp"
    if empty.any():
        assert (o[empty] == 0).all(), f"{what}: empty rows must be exactly 0"
    err_o = max_abs(o, ref_o)
    live = ~empty
    err_l = (lse[live] - ref_lse[live]).abs().max().item() if live.any() else 0.0
    assert err_o <= TOL_O[dtype], f"{what}: max|dO|={err_o:.3e} > {TOL_O[dtype]}"
    assert err_l <= TOL_LSE, f"{what}: max|dLSE|={err_l:.3e} > {TOL_LSE}"
    return err_o, err_l
