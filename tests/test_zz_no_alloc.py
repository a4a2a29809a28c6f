"""The backward entry point that allocates nothing (its workspace is a device array built into
the library) against the backward entry point that takes a workspace: same kernels, so the
gradients must agree bit for bit.  Two calls in a row, the second on a smaller input, so that
what the first call left in the built-in array cannot leak into the second."""
import pytest
import torch

import omni_attn_capi
from baseline_configs import make_workload

pytestmark = pytest.mark.gpu


def _run(w, dout, device, no_alloc):
    m = w.block_mask
    dev = lambda t: None if t is None else t.to(device).contiguous()
    q, k, v, do = dev(w.q), dev(w.k), dev(w.v), dev(dout)
    nb, idx, tys = dev(m.kv_num_blocks), dev(m.kv_indices), dev(m.block_mask_types)
    pidx, pm = dev(m.partial_block_mask_indices), dev(m.partial_block_masks)
    S = q.shape[2]
    o = torch.empty_like(q)
    lse = torch.empty(q.shape[:3], dtype=torch.float32, device=device)
    omni_attn_capi.fwd(q, k, v, o, lse, nb, idx, tys, m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE, S, pidx, pm)
    dq, dk, dv = (torch.full_like(q, float("nan")) for _ in range(3))
    omni_attn_capi.bwd(q, k, v, o, do, lse, dq, dk, dv, nb, idx, tys, m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE, S,
                       pidx, pm, no_alloc=no_alloc)
    torch.cuda.synchronize()
    return dq, dk, dv


def test_no_alloc_backward_equals_workspace_backward_twice(gpu_device):
    gen = torch.Generator().manual_seed(9)
    big = make_workload("c3_partial", seed=6, H=4, S=2048)
    small = make_workload("c3_partial", seed=7, H=1, S=512)
    for w in (big, small):  # second call: smaller input, same built-in array
        dout = torch.randn(w.q.shape, generator=gen).to(w.dtype)
        got = _run(w, dout, gpu_device, no_alloc=True)
        ref = _run(w, dout, gpu_device, no_alloc=False)
        for name, a, b in zip(("dQ", "dK", "dV"), got, ref):
            assert torch.isfinite(a.float()).all(), name
            assert torch.equal(a, b), f"{name} differs between the two entry points"


def test_no_alloc_backward_rejects_sizes_beyond_its_scratch(gpu_device):
    lib = omni_attn_capi.load_library()
    max_rows = lib.omni_attn_bwd_noalloc_max_rows()
    assert max_rows == 4 << 20
    one = 4096  # non-null: the size check comes before any pointer is used
    rc = lib.omni_attn_bwd_noalloc_gfx950(one, one, one, one, one, one, one, one, one, one, one, one, 0, 0, 0,
                                          64, 64, 2048, 128, 16, 16, 128, 128, 0, 2048, 1, 0.0, 0)
    assert rc == 10 and "scratch" in omni_attn_capi.status_string(rc)
