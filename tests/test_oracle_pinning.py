"""Pins the CPU oracle (oracle/) before anything is compared against it.

Each check is chosen so that a plausible mistake -- a dropped scale, softmax over the
wrong axis, a transposed operand, block-local instead of global causal indices, a wrong
empty-row convention -- fails at least one of them.  None of them retypes the oracle's
own formula: they use a library routine, brute-force loops, closed forms, and the
known answers the reference's generators printed (tests/golden/printed_masks.json).
"""
import math

import pytest
import torch
import torch.nn.functional as F

from helpers import load_printed_masks, random_block_metadata, typed_pattern_to_metadata
from oracle.block_walk import attention_block_walk
from oracle.dense_oracle import (attention_dense_fp32, dense_mask_from_blocks, prefix_mask,
                                 transfusion_mask_bruteforce)


def _rand(gen, *shape):
    return torch.randn(*shape, generator=gen)


def test_dense_oracle_matches_library_sdpa():
    gen = torch.Generator().manual_seed(1)
    q, k, v = (_rand(gen, 2, 3, 96, 32) for _ in range(3))
    mask = torch.rand(2, 3, 96, 96, generator=gen) < 0.5
    mask[..., 0] = True  # the library returns NaN for empty rows; keep every row alive here
    o, lse = attention_dense_fp32(q, k, v, mask)
    ref = F.scaled_dot_product_attention(q, k, v, attn_mask=mask)
    assert torch.allclose(o, ref, atol=2e-6, rtol=1e-5)
    s = (q @ k.transpose(-1, -2)) / math.sqrt(32)
    ref_lse = torch.logsumexp(s.masked_fill(~mask, float("-inf")), -1)
    assert torch.allclose(lse, ref_lse, atol=1e-6)


def test_dense_oracle_matches_bruteforce_loops():
    gen = torch.Generator().manual_seed(2)
    S, D = 7, 5
    q, k, v = (_rand(gen, S, D).double() for _ in range(3))
    mask = torch.rand(S, S, generator=gen) < 0.6
    mask[3] = False  # an empty row
    exp_o = torch.zeros(S, D, dtype=torch.float64)
    exp_l = torch.full((S,), float("-inf"), dtype=torch.float64)
    for i in range(S):
        ws = []
        for j in range(S):
            if mask[i, j]:
                dot = sum(q[i, d].item() * k[j, d].item() for d in range(D)) / math.sqrt(D)
                ws.append((j, dot))
        if not ws:
            continue
        z = sum(math.exp(w) for _, w in ws)
        exp_l[i] = math.log(z)
        for j, w in ws:
            exp_o[i] += math.exp(w) / z * v[j]
    o, lse = attention_dense_fp32(q, k, v, mask)
    assert torch.allclose(o.double(), exp_o, atol=1e-6)
    assert torch.equal(torch.isinf(lse), torch.isinf(exp_l))
    live = ~torch.isinf(exp_l)
    assert torch.allclose(lse.double()[live], exp_l[live], atol=1e-6)
    assert (o[3] == 0).all() and lse[3] == float("-inf")


def test_dense_oracle_closed_forms():
    gen = torch.Generator().manual_seed(3)
    S, D = 16, 8
    v = _rand(gen, S, D)
    # zero queries: uniform weights over the allowed keys -> mean of their V rows, lse = log n
    q = torch.zeros(S, D)
    k = _rand(gen, S, D)
    causal = torch.tril(torch.ones(S, S, dtype=torch.bool))
    o, lse = attention_dense_fp32(q, k, v, causal)
    for i in range(S):
        assert torch.allclose(o[i], v[: i + 1].mean(0), atol=1e-6)
        assert abs(lse[i].item() - math.log(i + 1)) < 1e-6
    # one allowed key: output is that V row exactly, lse = q.k / sqrt(D)
    q = _rand(gen, S, D)
    one = torch.zeros(S, S, dtype=torch.bool)
    one[torch.arange(S), (torch.arange(S) * 5) % S] = True
    o, lse = attention_dense_fp32(q, k, v, one)
    cols = (torch.arange(S) * 5) % S
    assert torch.allclose(o, v[cols], atol=1e-6)
    assert torch.allclose(lse, (q * k[cols]).sum(-1) / math.sqrt(D), atol=1e-5)
    # scale is 1/sqrt(D), not 1/D or 1: doubling D by zero-padding changes the result
    # exactly as if the scores were divided by sqrt(2)
    qp, kp = torch.cat([q, torch.zeros_like(q)], -1), torch.cat([k, torch.zeros_like(k)], -1)
    o2, _ = attention_dense_fp32(qp, kp, v, causal)
    o3, _ = attention_dense_fp32(q / math.sqrt(2.0), k, v, causal)
    assert torch.allclose(o2, o3, atol=1e-6)


def test_row_chunking_is_invisible():
    gen = torch.Generator().manual_seed(4)
    q, k, v = (_rand(gen, 2, 50, 16) for _ in range(3))
    mask = torch.rand(2, 50, 50, generator=gen) < 0.4
    a = attention_dense_fp32(q, k, v, mask, row_chunk=7)
    b = attention_dense_fp32(q, k, v, mask, row_chunk=4096)
    assert torch.allclose(a[0], b[0], atol=1e-6) and torch.equal(torch.isinf(a[1]), torch.isinf(b[1]))


def test_transfusion_rule_prefix_form_matches_bruteforce():
    from omni_attn_torch import modality_prefix_lengths, naive_attn_mask
    S = 40
    cases = [[], [(5, 10)], [(0, 7), (20, 6)], [(3, 4), (10, 25), (38, 2)], [(12, 0)]]
    for spans in cases:
        brute = transfusion_mask_bruteforce(S, spans)
        mp = torch.zeros(1, max(1, len(spans)), 3, dtype=torch.long)
        for m, (off, ln) in enumerate(spans):
            mp[0, m] = torch.tensor([1, off, ln])
        assert torch.equal(naive_attn_mask(S, mp)[0], brute), spans
        assert torch.equal(prefix_mask(modality_prefix_lengths(mp, S), S)[0], brute), spans


def test_transfusion_rule_known_answer_8x8():
    """One image span (offset 2, length 3) in 8 tokens, written out by hand from the rule
    allow[i, j] = (i >= j) or (i >= offset and j < offset + length)
    (transfusion_pytorch/transfusion.py:496-515): tokens before the image are causal, tokens
    of the image see the whole image, later tokens see the image through causality anyway.
    Pins the brute-force restatement and the product's two forms by something that is neither."""
    from omni_attn_torch import modality_prefix_lengths, naive_attn_mask
    expected = torch.tensor([
        [1, 0, 0, 0, 0, 0, 0, 0],
        [1, 1, 0, 0, 0, 0, 0, 0],
        [1, 1, 1, 1, 1, 0, 0, 0],
        [1, 1, 1, 1, 1, 0, 0, 0],
        [1, 1, 1, 1, 1, 0, 0, 0],
        [1, 1, 1, 1, 1, 1, 0, 0],
        [1, 1, 1, 1, 1, 1, 1, 0],
        [1, 1, 1, 1, 1, 1, 1, 1]], dtype=torch.bool)
    assert torch.equal(transfusion_mask_bruteforce(8, [(2, 3)]), expected)
    mp = torch.tensor([[[1, 2, 3]]], dtype=torch.long)
    assert torch.equal(naive_attn_mask(8, mp)[0], expected)
    assert torch.equal(prefix_mask(modality_prefix_lengths(mp, 8), 8)[0], expected)
    # a transposed or sign-flipped rule would give one of these instead
    assert not torch.equal(expected, expected.t())
    assert modality_prefix_lengths(mp, 8)[0].tolist() == [1, 2, 5, 5, 5, 6, 7, 8]


@pytest.mark.parametrize("pat", load_printed_masks()["typed_block_patterns"], ids=lambda p: p["source"])
def test_block_semantics_against_printed_sparsity(pat):
    """Typed block patterns + the sparsity the reference printed for their dense mask.
    Patterns contain CAUSAL blocks off the diagonal, so block-local causal indices, or a
    PARTIAL tile read transposed, change the number."""
    S, QB, KB = pat["seq_len"], pat["Q_BLOCK_SIZE"], pat["KV_BLOCK_SIZE"]
    nb, idx, tys, pidx, pm = typed_pattern_to_metadata(pat["rows"], True, QB, KB)
    dense = dense_mask_from_blocks(nb, idx, tys, QB, KB, S, S, pidx, pm)
    assert abs((1.0 - dense.float().mean().item()) - pat["sparsity"]) < 5e-5
    # the C walk must realise the same mask: with q = 0 every allowed key has weight
    # 1/n, so with V = one-hot(key) the output row is the mask row divided by n
    q = torch.zeros(1, 1, S, 64)
    k = torch.zeros(1, 1, S, 64)
    for d0 in range(0, S, 64):
        v = torch.zeros(1, 1, S, 64)
        v[0, 0, d0:d0 + 64] = torch.eye(64)
        o, lse = attention_block_walk(q, k, v, nb, idx, tys, QB, KB, S, pidx, pm)
        n = dense[0, 0].sum(-1, keepdim=True).clamp(min=1).float()
        assert torch.allclose(o[0, 0], dense[0, 0, :, d0:d0 + 64].float() / n, atol=1e-6)
    assert torch.allclose(lse[0, 0], torch.log(dense[0, 0].sum(-1).float()), atol=1e-5)


@pytest.mark.parametrize("QB,KB", [(128, 128), (128, 64), (64, 128), (64, 64)])
def test_block_walk_matches_dense_oracle(QB, KB):
    gen = torch.Generator().manual_seed(10 * QB + KB)
    B, H, S, D = 2, 2, 512, 32
    q, k, v = (_rand(gen, B, H, S, D) for _ in range(3))
    nb, idx, tys, pidx, pm = random_block_metadata(gen, B, H, S // QB, S // KB, QB, KB, shuffle=True)
    for seqlen in (S, S - 37):
        dense = dense_mask_from_blocks(nb, idx, tys, QB, KB, S, S, pidx, pm, seqlen_orig=seqlen)
        ro, rl = attention_dense_fp32(q, k, v, dense)
        o, lse = attention_block_walk(q, k, v, nb, idx, tys, QB, KB, seqlen, pidx, pm)
        assert torch.allclose(o, ro, atol=2e-5), (o - ro).abs().max()
        assert torch.equal(torch.isinf(lse), torch.isinf(rl))
        live = ~torch.isinf(rl)
        assert torch.allclose(lse[live], rl[live], atol=2e-5)
        assert (o[~live] == 0).all()
        assert (~live).any(), "the case must contain empty rows"


def test_partial_index_beyond_the_stored_tiles_is_skipped_by_the_walk():
    """An index >= the number of stored tiles means "no bits stored" (the product's contract;
    the reference reads such an index unchecked, attn_naive.cu:124-131)."""
    gen = torch.Generator().manual_seed(6)
    q, k, v = (_rand(gen, 1, 1, 256, 32) for _ in range(3))
    nb = torch.tensor([[[2, 2]]], dtype=torch.int32)
    idx = torch.tensor([[[[0, 1], [0, 1]]]], dtype=torch.int32)
    tys = torch.tensor([[[[2, 3], [3, 2]]]], dtype=torch.int32)
    tiles = torch.rand(2, 128, 128, generator=gen) < 0.5
    pidx_bad = torch.tensor([[[[-1, 2], [1 << 20, -1]]]], dtype=torch.int32)
    pidx_none = torch.full((1, 1, 2, 2), -1, dtype=torch.int32)
    a = attention_block_walk(q, k, v, nb, idx, tys, 128, 128, 256, pidx_bad, tiles)
    b = attention_block_walk(q, k, v, nb, idx, tys, 128, 128, 256, pidx_none, tiles)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    pidx_ok = torch.tensor([[[[-1, 1], [0, -1]]]], dtype=torch.int32)
    c = attention_block_walk(q, k, v, nb, idx, tys, 128, 128, 256, pidx_ok, tiles)
    assert not torch.equal(a[0], c[0])


def test_walk_treats_any_non_zero_mask_byte_as_attend():
    gen = torch.Generator().manual_seed(7)
    q, k, v = (_rand(gen, 1, 1, 128, 32) for _ in range(3))
    nb = torch.tensor([[[1]]], dtype=torch.int32)
    idx = torch.zeros(1, 1, 1, 1, dtype=torch.int32)
    tys = torch.full((1, 1, 1, 1), 3, dtype=torch.int32)
    pidx = torch.zeros(1, 1, 1, 1, dtype=torch.int32)
    bits = torch.rand(1, 128, 128, generator=gen) < 0.5
    a = attention_block_walk(q, k, v, nb, idx, tys, 128, 128, 128, pidx, bits)
    b = attention_block_walk(q, k, v, nb, idx, tys, 128, 128, 128, pidx, bits.to(torch.uint8) * 0xfe)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def test_bitless_partial_slot_is_skipped_by_the_walk():
    """PARTIAL without stored bits contributes nothing (attn_naive.cu:119-131)."""
    gen = torch.Generator().manual_seed(5)
    q, k, v = (_rand(gen, 1, 1, 256, 32) for _ in range(3))
    nb = torch.tensor([[[1, 2]]], dtype=torch.int32)
    idx = torch.tensor([[[[0, 0], [0, 1]]]], dtype=torch.int32)
    tys = torch.tensor([[[[1, 0], [3, 1]]]], dtype=torch.int32)
    o, lse = attention_block_walk(q, k, v, nb, idx, tys, 128, 128, 256)
    tys_skip = torch.tensor([[[[1, 0], [0, 1]]]], dtype=torch.int32)
    o2, lse2 = attention_block_walk(q, k, v, nb, idx, tys_skip, 128, 128, 256)
    assert torch.equal(o, o2) and torch.equal(lse, lse2)


# ---- gradients (oracle of the backward kernels) ------------------------------------------------

def test_gradient_oracle_gradcheck_and_closed_form():
    from oracle.dense_oracle import (attention_dense_differentiable, attention_dense_grads,
                                     attention_dense_grads_closed_form)
    gen = torch.Generator().manual_seed(31)
    S, D = 7, 4
    mask = torch.rand(2, S, S, generator=gen) < 0.6
    mask[0, 3] = False  # a row with no allowed key: zero output, no gradient
    q, k, v = (torch.randn(2, S, D, generator=gen, dtype=torch.float64, requires_grad=True) for _ in range(3))
    assert torch.autograd.gradcheck(lambda a, b, c: attention_dense_differentiable(a, b, c, mask), (q, k, v),
                                    eps=1e-6, atol=1e-6)
    dout = torch.randn(2, S, D, generator=gen)
    g_auto = attention_dense_grads(q, k, v, mask, dout)
    g_form = attention_dense_grads_closed_form(q, k, v, mask, dout)
    for a, b in zip(g_auto, g_form):
        assert torch.allclose(a, b, atol=2e-6), (a - b).abs().max()
    assert (g_auto[0][0, 3] == 0).all()  # the empty row passes nothing to its query
    # the forward of the differentiable form is the oracle's forward
    o_ref, _ = attention_dense_fp32(q.detach(), k.detach(), v.detach(), mask)
    assert torch.allclose(attention_dense_differentiable(q.detach().float(), k.detach().float(),
                                                         v.detach().float(), mask), o_ref, atol=1e-6)


def test_gradient_oracle_one_allowed_key_per_row():
    """With one allowed key per row the output is that V row whatever Q and K are:
    dQ = dK = 0 and dV[j] = sum of dO over the rows that attend key j."""
    from oracle.dense_oracle import attention_dense_grads
    gen = torch.Generator().manual_seed(32)
    S, D = 9, 8
    target = torch.randint(0, S, (S,), generator=gen)
    mask = torch.zeros(S, S, dtype=torch.bool)
    mask[torch.arange(S), target] = True
    q, k, v, dout = (torch.randn(S, D, generator=gen) for _ in range(4))
    dq, dk, dv = attention_dense_grads(q, k, v, mask, dout)
    assert dq.abs().max() < 1e-6 and dk.abs().max() < 1e-6
    expect = torch.zeros(S, D).index_add_(0, target, dout)
    assert torch.allclose(dv, expect, atol=1e-6)


# ---- the soft-capped branch of the oracle -------------------------------------------------------
# (transfusion_pytorch/transfusion.py:298-299 softclamp; :966-968: applied to the SCALED score,
# before the mask).  None of the checks below evaluates softcap * tanh(x / softcap) with torch.

def test_softcap_limits():
    gen = torch.Generator().manual_seed(41)
    S, D = 12, 8
    q, k, v = (_rand(gen, S, D) for _ in range(3))
    mask = torch.rand(S, S, generator=gen) < 0.5
    mask[5] = False
    # cap -> infinity: the plain oracle (tanh(x) = x - x^3/3 + ...: relative deviation (x / cap)^2 / 3)
    o0, l0 = attention_dense_fp32(q, k, v, mask)
    o1, l1 = attention_dense_fp32(q, k, v, mask, softcap=1e6)
    live = ~torch.isinf(l0)
    assert torch.allclose(o0, o1, atol=1e-6) and torch.allclose(l0[live], l1[live], atol=1e-6)
    assert torch.equal(torch.isinf(l0), torch.isinf(l1)) and (o1[5] == 0).all()
    # cap -> 0: every allowed score lies in [-cap, cap], so the weights are uniform up to
    # exp(2 cap): mean of the allowed V rows, lse = log n +- cap
    cap = 1e-3
    o2, l2 = attention_dense_fp32(q, k, v, mask, softcap=cap)
    for i in range(S):
        n = int(mask[i].sum())
        if n == 0:
            assert (o2[i] == 0).all() and l2[i] == float("-inf")
            continue
        assert torch.allclose(o2[i], v[mask[i]].mean(0), atol=4 * cap * v.abs().max().item())
        assert abs(l2[i].item() - math.log(n)) <= cap + 1e-6


def test_softcap_two_key_row_by_hand():
    """One query, two keys, worked with math.tanh / math.exp: the cap acts on q.k / sqrt(D)."""
    q = torch.tensor([[1.5, -2.0, 0.5, 3.0]])
    k = torch.tensor([[2.0, 1.0, -1.0, 4.0], [-3.0, 0.5, 2.0, -1.0]])
    v = torch.tensor([[1.0, 10.0], [-2.0, 4.0]])
    cap = 2.0
    x = [sum(float(a) * float(b) for a, b in zip(q[0], k[j])) / 2.0 for j in range(2)]  # sqrt(4) = 2
    assert x == [6.25, -3.75]
    y = [cap * math.tanh(xi / cap) for xi in x]
    z = [math.exp(yi) for yi in y]
    expect_o = [(z[0] * float(v[0, d]) + z[1] * float(v[1, d])) / (z[0] + z[1]) for d in range(2)]
    expect_l = math.log(z[0] + z[1])
    qq = torch.cat([q, torch.zeros(1, 4)])          # two rows (the second attends nothing)
    mask = torch.tensor([[True, True], [False, False]])
    o, lse = attention_dense_fp32(qq, k, v, mask, softcap=cap)
    assert abs(o[0, 0].item() - expect_o[0]) < 1e-6 and abs(o[0, 1].item() - expect_o[1]) < 1e-6
    assert abs(lse[0].item() - expect_l) < 1e-6
    # a cap applied to the raw product (12.5 and -7.5, saturated at +-2 as well, but
    # by different amounts) or after the mask would give other numbers:
    y_raw = [cap * math.tanh(2.0 * xi / cap) / 2.0 for xi in x]
    assert abs(y_raw[0] - y[0]) > 0.5


def test_softcap_acts_on_the_scaled_score():
    """Zero-padding the head dimension to 4 D halves every scaled score and leaves q.k alone: with
    the cap on the scaled score the result equals that of scores halved before the cap."""
    gen = torch.Generator().manual_seed(42)
    S, D = 10, 8
    q, k, v = (_rand(gen, S, D) * 3 for _ in range(3))
    causal = torch.tril(torch.ones(S, S, dtype=torch.bool))
    pad = torch.zeros(S, 3 * D)
    a, la = attention_dense_fp32(torch.cat([q, pad], -1), torch.cat([k, pad], -1), v, causal, softcap=1.5)
    b, lb = attention_dense_fp32(q / 2.0, k, v, causal, softcap=1.5)
    assert torch.allclose(a, b, atol=1e-6) and torch.allclose(la, lb, atol=1e-6)
    c, _ = attention_dense_fp32(q, k, v, causal, softcap=1.5)
    assert (a - c).abs().max() > 1e-2  # and the cap is not scale-invariant


def test_softcap_per_element_loop_and_gradcheck():
    from oracle.dense_oracle import (attention_dense_differentiable, attention_dense_grads,
                                     attention_dense_grads_chunked)
    gen = torch.Generator().manual_seed(43)
    S, D, cap = 6, 4, 0.8
    q, k, v = (_rand(gen, S, D) * 2 for _ in range(3))
    mask = torch.rand(S, S, generator=gen) < 0.6
    mask[2] = False
    o, lse = attention_dense_fp32(q, k, v, mask, softcap=cap)
    for i in range(S):
        ws = {}
        for j in range(S):
            if mask[i, j]:
                x = sum(float(q[i, d]) * float(k[j, d]) for d in range(D)) / math.sqrt(D)
                ws[j] = math.exp(cap * math.tanh(x / cap))
        if not ws:
            assert (o[i] == 0).all() and lse[i] == float("-inf")
            continue
        tot = sum(ws.values())
        for d in range(D):
            assert abs(o[i, d].item() - sum(w * float(v[j, d]) for j, w in ws.items()) / tot) < 1e-5
        assert abs(lse[i].item() - math.log(tot)) < 1e-5
    q64, k64, v64 = (t.double().requires_grad_(True) for t in (q, k, v))
    assert torch.autograd.gradcheck(lambda a, b, c: attention_dense_differentiable(a, b, c, mask, cap),
                                    (q64, k64, v64), eps=1e-6, atol=1e-6)
    # the row-blocked closed form (with the cap's derivative 1 - tanh^2) against autograd
    dout = _rand(gen, S, D)
    for sc in (0.0, cap):
        auto = attention_dense_grads(q, k, v, mask, dout, softcap=sc)
        for chunk in (4, 64):
            form = attention_dense_grads_chunked(q, k, v, mask, dout, row_chunk=chunk, softcap=sc)
            for a, b in zip(auto, form):
                assert torch.allclose(a, b, atol=2e-6), (a - b).abs().max()


# ---- what rounding P and O to bf16 costs (the limit of the absolute bar on sparse rows) ----------

def test_bf16_two_rounding_model_on_a_two_key_row():
    """The row the GPU test test_bf16_error_on_rows_with_few_keys_is_the_two_roundings quotes, by
    hand: weights 1 : 12.416 (the walk meets the small one first, so the reference point of the
    exponentials stays at it), V = 0.515625 and -2.78125.  fp32: -2.5355.  With the large weight
    rounded to bf16 (12.4375) over the unrounded row sum: -2.53999, which bf16 rounds away from the
    fp32 value to -2.546875: 0.0114 from the oracle, beyond the absolute bar of 1e-2, inside
    2^-8 (sum p |v| / l + |O|)."""
    p_small, p_large = 1.0, 1.0 / 0.08054216206073761
    v_small, v_large = 0.515625, -2.78125
    exact = (p_small * v_small + p_large * v_large) / (p_small + p_large)
    assert abs(exact - (-2.535505)) < 1e-5
    rounded_p = torch.tensor(p_large).to(torch.bfloat16).item()
    assert rounded_p == 12.4375
    kernel_fp32 = (p_small * v_small + rounded_p * v_large) / (p_small + p_large)
    assert abs(kernel_fp32 - (-2.53999)) < 1e-5
    out = torch.tensor(kernel_fp32).to(torch.bfloat16).item()
    assert out == -2.546875
    err = abs(out - exact)
    assert 1e-2 < err < 1.2e-2
    mean_abs = (p_small * abs(v_small) + p_large * abs(v_large)) / (p_small + p_large)
    assert err <= 2.0 ** -8 * (mean_abs + abs(exact))
