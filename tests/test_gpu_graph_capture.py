"""The forward and the backward entry point that allocates nothing, recorded in a HIP graph.

The entry points only enqueue kernels on the stream they are given, so a caller can capture them
(after one eager call, which sets the kernels' LDS limits and looks up the built-in workspace).
Every replay is checked bit for bit against an eager run on the same inputs, with new inputs and
the program's own eager work between the replays."""
import pytest
import torch

import omni_attn_capi
from baseline_configs import make_workload

pytestmark = pytest.mark.gpu


def test_forward_and_no_alloc_backward_replay_in_a_graph(gpu_device):
    w = make_workload("c3_partial", seed=8, H=2, S=1024)
    m = w.block_mask
    dev = lambda t: t.to(gpu_device).contiguous()
    q, k, v = dev(w.q), dev(w.k), dev(w.v)
    gen = torch.Generator().manual_seed(21)
    dout = dev(torch.randn(w.q.shape, generator=gen).to(w.dtype))
    nb, idx, tys = dev(m.kv_num_blocks), dev(m.kv_indices), dev(m.block_mask_types)
    pidx, pm = dev(m.partial_block_mask_indices), dev(m.partial_block_masks)
    S = q.shape[2]
    o = torch.empty_like(q)
    lse = torch.empty(q.shape[:3], dtype=torch.float32, device=gpu_device)
    dq, dk, dv = (torch.empty_like(q) for _ in range(3))
    outputs = (o, lse, dq, dk, dv)

    def launch(stream):
        omni_attn_capi.fwd(q, k, v, o, lse, nb, idx, tys, m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE, S, pidx, pm,
                           stream=stream.cuda_stream)
        omni_attn_capi.bwd(q, k, v, o, dout, lse, dq, dk, dv, nb, idx, tys, m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE, S,
                           pidx, pm, no_alloc=True, stream=stream.cuda_stream)

    side = torch.cuda.Stream(device=gpu_device)
    side.wait_stream(torch.cuda.current_stream(gpu_device))
    with torch.cuda.stream(side):
        launch(side)  # eager first call
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        launch(torch.cuda.current_stream(gpu_device))
    torch.cuda.synchronize()

    for rep in range(3):
        for t in (q, k, v, dout):  # new inputs in the captured buffers
            t.copy_(torch.randn(t.shape, generator=gen).to(t.dtype))
        torch.cuda.synchronize()
        launch(torch.cuda.current_stream(gpu_device))
        torch.cuda.synchronize()
        eager = [t.clone() for t in outputs]
        for t in outputs:
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("O", "LSE", "dQ", "dK", "dV"), outputs, eager):
            assert torch.equal(a, b), f"replay {rep}: {name} differs from the eager run"
