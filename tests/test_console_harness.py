"""The console harness: tensor-only fixture round trip (CPU) and a full run (GPU)."""
import io

import pytest
import torch

import console_harness
from baseline_configs import make_workload


def test_fixture_round_trip(tmp_path):
    w = make_workload("c3_partial", seed=3, H=2, S=1024)
    p = str(tmp_path / "fx.safetensors")
    console_harness.save_fixture(p, w.q, w.k, w.v, w.block_mask, w.q.shape[2])
    q, k, v, m, seq_len = console_harness.load_fixture(p)
    assert seq_len == 1024 and torch.equal(q, w.q) and torch.equal(k, w.k) and torch.equal(v, w.v)
    a = w.block_mask
    assert (m.q_len, m.kv_len, m.Q_BLOCK_SIZE, m.KV_BLOCK_SIZE) == (a.q_len, a.kv_len, a.Q_BLOCK_SIZE, a.KV_BLOCK_SIZE)
    for name in ("kv_num_blocks", "kv_indices", "block_mask_types", "partial_block_mask_indices"):
        assert torch.equal(getattr(m, name), getattr(a, name)), name
    assert m.partial_block_masks.dtype == torch.bool
    assert torch.equal(m.partial_block_masks, a.partial_block_masks.bool())
    assert torch.equal(m.to_dense_mask(), a.to_dense_mask())


@pytest.mark.gpu
@pytest.mark.parametrize("name,kw", [("c1_causal", {}), ("c3_partial", {"H": 2, "S": 1024})])
def test_all_entry_points_pass_on_the_console(name, kw, gpu_device):
    w = make_workload(name, seed=1, **kw)
    buf = io.StringIO()
    results = console_harness.run(w.q, w.k, w.v, w.block_mask, device=gpu_device, iters=3, out=buf)
    text = buf.getvalue()
    assert len(results) == 5 and all(p for p, _ in results.values()), text
    assert text.count("PASSED") == 5 and "effective" in text
