"""PARTIAL tiles packed to bits by the pre-pass kernel, and the forward on packed tiles.

Bars: byte and bit work is exact -- the packed words equal numpy's packbits of the same
tiles bit for bit, and the forward on packed tiles equals the forward on byte tiles bit for
bit (same kernel, same arithmetic); against the CPU oracle the usual bars apply (max-abs
2e-3 fp16 / 1e-2 bf16 on the output, 1e-3 on the logsumexp).
"""
import numpy as np
import pytest
import torch

import omni_attn_capi
from baseline_configs import make_workload
from helpers import compare_with_oracle, random_block_metadata
from oracle.block_walk import attention_block_walk
from oracle.dense_oracle import attention_dense_fp32, prefix_mask
from test_gpu_parity import run_kernel

pytestmark = pytest.mark.gpu


def packbits_reference(tiles: torch.Tensor) -> torch.Tensor:
    """[P, QB, KB] bytes -> [P, QB, KB // 32] int32, bit j of word c = (byte 32 c + j != 0)."""
    bits = (tiles.cpu().numpy().astype(np.uint8) != 0)
    packed = np.packbits(bits, axis=-1, bitorder="little")            # [P, QB, KB // 8] bytes
    words = packed.reshape(packed.shape[0], packed.shape[1], -1, 4).copy().view("<u4")[..., 0]
    return torch.from_numpy(words.astype(np.uint32).view(np.int32))


@pytest.mark.parametrize("QB,KB", [(128, 128), (128, 64), (64, 128), (64, 64)])
@pytest.mark.parametrize("P", [1, 7, 3000])
def test_pack_kernel_matches_packbits(QB, KB, P, gpu_device):
    gen = torch.Generator().manual_seed(P * 7 + QB + KB)
    dens = torch.rand(P, 1, 1, generator=gen)
    bits = torch.rand(P, QB, KB, generator=gen) < dens
    if P > 2:
        bits[1] = True
        bits[2] = False
    expected = packbits_reference(bits)
    got = omni_attn_capi.pack_partial_masks(bits.to(gpu_device))
    torch.cuda.synchronize()
    assert got.dtype == torch.int32 and got.shape == (P, QB, KB // 32)
    assert torch.equal(got.cpu(), expected)
    # bytes other than 0 / 1: any non-zero byte is a set bit
    values = torch.tensor([1, 2, 0x40, 0x80, 0xff], dtype=torch.uint8)
    as_bytes = torch.where(bits, values[torch.randint(0, 5, bits.shape, generator=gen)],
                           torch.zeros((), dtype=torch.uint8))
    got2 = omni_attn_capi.pack_partial_masks(as_bytes.to(gpu_device))
    torch.cuda.synchronize()
    assert torch.equal(got2.cpu(), expected)


def test_pack_of_zero_tiles_and_bad_arguments(gpu_device):
    lib = omni_attn_capi.load_library()
    assert lib.omni_attn_pack_partial_masks_gfx950(0, 0, 0, 128, 128, 0) == 0        # nothing to do
    assert lib.omni_attn_pack_partial_masks_gfx950(0, 0, 3, 128, 128, 0) == 1        # null pointers
    assert lib.omni_attn_pack_partial_masks_gfx950(4096, 4096, 3, 96, 128, 0) == 4   # block size
    assert lib.omni_attn_pack_partial_masks_gfx950(4096, 4096, -1, 128, 128, 0) == 2


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("QB,KB", [(128, 128), (128, 64), (64, 128), (64, 64)])
def test_packed_forward_equals_byte_forward_and_oracle(dtype, D, QB, KB, gpu_device):
    gen = torch.Generator().manual_seed(31 * D + 3 * QB + KB)
    B, H, S = 2, 2, 512
    q, k, v = (torch.randn(B, H, S, D, generator=gen).to(dtype) for _ in range(3))
    nb, idx, tys, pidx, pm = random_block_metadata(gen, B, H, S // QB, S // KB, QB, KB, shuffle=True)
    for seqlen in (S, S - 45):
        o_b, l_b = run_kernel(q, k, v, nb, idx, tys, QB, KB, seqlen, pidx, pm, device=gpu_device)
        dev = lambda t: t.to(gpu_device).contiguous()
        bits = omni_attn_capi.pack_partial_masks(dev(pm))
        o_p = torch.full_like(o_b, float("nan"))
        l_p = torch.full_like(l_b, float("nan"))
        omni_attn_capi.fwd(dev(q), dev(k), dev(v), o_p, l_p, dev(nb), dev(idx), dev(tys), QB, KB, seqlen,
                           dev(pidx), None, partial_bits=bits)
        torch.cuda.synchronize()
        assert torch.equal(o_p, o_b) and torch.equal(l_p, l_b), "packed and byte tiles must agree bit for bit"
        wo, wl = attention_block_walk(q, k, v, nb, idx, tys, QB, KB, seqlen, pidx, pm)
        compare_with_oracle(o_p, l_p, wo, wl, dtype, f"packed tiles vs block walk, seqlen={seqlen}")


def test_packed_forward_on_c3_partial_full_size(gpu_device):
    w = make_workload("c3_partial", seed=0)
    m = w.block_mask
    B, H, S, D = w.q.shape
    dev = lambda t: t.to(gpu_device).contiguous()
    q, k, v = dev(w.q), dev(w.k), dev(w.v)
    nb, idx, tys, pidx, pm = (dev(t) for t in (m.kv_num_blocks, m.kv_indices, m.block_mask_types,
                                               m.partial_block_mask_indices, m.partial_block_masks))
    bits = omni_attn_capi.pack_partial_masks(pm)
    assert torch.equal(bits.cpu(), packbits_reference(m.partial_block_masks))
    o_b, l_b = torch.empty_like(q), torch.empty(B, H, S, dtype=torch.float32, device=gpu_device)
    o_p, l_p = torch.full_like(q, float("nan")), torch.full_like(l_b, float("nan"))
    omni_attn_capi.fwd(q, k, v, o_b, l_b, nb, idx, tys, m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE, S, pidx, pm)
    omni_attn_capi.fwd(q, k, v, o_p, l_p, nb, idx, tys, m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE, S, pidx, None,
                       partial_bits=bits)
    torch.cuda.synchronize()
    assert torch.equal(o_p, o_b) and torch.equal(l_p, l_b)
    o_cpu, l_cpu = o_p.cpu(), l_p.cpu()
    mask = prefix_mask(w.prefix_len[0], S)
    for h in range(0, H, 3):
        ro, rl = attention_dense_fp32(w.q[0, h], w.k[0, h], w.v[0, h], mask)
        compare_with_oracle(o_cpu[0, h], l_cpu[0, h], ro, rl, w.dtype, f"c3 packed, head {h}")


def test_wrappers_use_packed_tiles_when_the_mask_has_them(gpu_device):
    import omni_attn_torch as oat
    w = make_workload("c3_partial", seed=4, H=2, S=1024)
    q, k, v = (t.to(gpu_device) for t in (w.q, w.k, w.v))
    m = w.block_mask.to(gpu_device)
    o_bytes, lse_bytes = oat.omni_attention_forward(q, k, v, m)
    mp = w.block_mask.to(gpu_device).pack_partial_masks()
    assert mp.partial_block_bits is not None and mp.partial_block_bits.shape[-1] == m.KV_BLOCK_SIZE // 32
    o_bits, lse_bits = oat.omni_attention_forward(q, k, v, mp)
    o_sw = oat.omni_attention_shared_kv_swizzle(q, k, v, mp)
    torch.cuda.synchronize()
    assert torch.equal(o_bits, o_bytes) and torch.equal(lse_bits, lse_bytes) and torch.equal(o_sw, o_bytes)
    ro, rl = attention_dense_fp32(w.q, w.k, w.v, prefix_mask(w.prefix_len, 1024).unsqueeze(1))
    compare_with_oracle(o_bits, lse_bits, ro, rl, w.dtype, "wrapper on packed tiles")


def test_deduplicated_tiles_give_the_same_output(gpu_device):
    """Sharing equal PARTIAL tiles between heads (on the GPU, on bytes and on packed words) leaves
    the forward bit for bit the same."""
    import omni_attn_torch as oat
    gen = torch.Generator().manual_seed(12)
    B, H, S, D = 1, 4, 512, 64
    dense = (torch.rand(B, 1, S, S, generator=gen) < 0.6).expand(B, H, S, S).contiguous()
    dense[..., torch.arange(S), torch.arange(S)] = True
    q, k, v = (torch.randn(B, H, S, D, generator=gen).half().to(gpu_device) for _ in range(3))
    m = oat.create_omni_block_mask_from_dense(dense, 128, 128).to(gpu_device)
    P = m.partial_block_masks.shape[0]
    o_ref, lse_ref = oat.omni_attention_forward(q, k, v, m)
    m_bytes = oat.create_omni_block_mask_from_dense(dense, 128, 128).to(gpu_device).deduplicate_partial_tiles()
    m_bits = oat.create_omni_block_mask_from_dense(dense, 128, 128).to(gpu_device).pack_partial_masks()
    m_bits.deduplicate_partial_tiles()
    for mm in (m_bytes, m_bits):
        assert mm.partial_block_masks.shape[0] == P // H and mm.partial_block_masks.is_cuda
        o, lse = oat.omni_attention_forward(q, k, v, mm)
        assert torch.equal(o, o_ref) and torch.equal(lse, lse_ref)
    assert m_bits.partial_block_bits.shape[0] == P // H
    ro, rl = attention_dense_fp32(q.cpu(), k.cpu(), v.cpu(), dense)
    compare_with_oracle(o_ref, lse_ref, ro, rl, torch.float16, "de-duplicated tiles")
