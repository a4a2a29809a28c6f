"""Host side of the operator wrappers, without a GPU: a stand-in for the extension module records
the calls, and every way of reading a value back out of a tensor (which on a GPU tensor is a device
synchronisation) is made to raise while a wrapper runs.  Contract: the reference's wrappers force a
global synchronize per call (omni-attn-mma/omni_attn_torch.py:641-671); these must not."""
import pytest
import torch

import omni_attn_torch as oat


class RecordingExtension:
    def __init__(self):
        self.calls = []

    def __getattr__(self, name):
        def call(*args):
            self.calls.append((name, args))
        return call


READ_BACKS = ("item", "tolist", "__bool__", "__int__", "__float__", "__index__", "cpu", "numpy", "nonzero")


def forbid_read_backs(monkeypatch):
    def boom(self, *a, **k):
        raise AssertionError("a wrapper read a value back from a tensor")
    for name in READ_BACKS:
        monkeypatch.setattr(torch.Tensor, name, boom, raising=False)


def partial_mask():
    spans = torch.tensor([[[1, 37, 90], [1, 200, 41]]], dtype=torch.long)
    prefix = oat.modality_prefix_lengths(spans, 256)
    return oat.create_omni_block_mask_from_prefix_lengths(prefix, 2, 256, 256, 128, 64)


@pytest.mark.parametrize("op", ["omni_attention_shared_kv", "omni_attention_shared_kv_swizzle",
                                "omni_attention_simple", "omni_attention_cp_async", "omni_attention_preftech",
                                "omni_attention_forward"])
def test_wrappers_read_nothing_back(op, monkeypatch):
    ext = RecordingExtension()
    monkeypatch.setattr(oat, "_load_extension", lambda: ext)
    mask = partial_mask()
    assert mask.has_partial_slots() is True          # answered here, once, and remembered
    q = torch.zeros(1, 2, 250, 64, dtype=torch.bfloat16)
    forbid_read_backs(monkeypatch)
    out = getattr(oat, op)(q, q, q, mask)
    out = out[0] if isinstance(out, tuple) else out
    assert out.shape == q.shape and len(ext.calls) == 1
    name, args = ext.calls[0]
    has_partial = args[12] if name != "omni_attn_forward" else args[13]
    assert has_partial is True


def test_partial_flag_of_the_three_wrappers_that_look_at_the_types(monkeypatch):
    """simple / cp_async / preftech pass has_partial only when a PARTIAL slot exists
    (omni_attn_torch.py:763-765); the answer is cached on the mask and survives to()."""
    ext = RecordingExtension()
    monkeypatch.setattr(oat, "_load_extension", lambda: ext)
    mask = partial_mask()
    mask.block_mask_types = torch.where(mask.block_mask_types == 3, torch.full_like(mask.block_mask_types, 2),
                                        mask.block_mask_types)
    mask._any_partial_slot = None
    moved = mask.to("cpu")
    assert moved.has_partial_slots() is False and moved.to("cpu")._any_partial_slot is False
    q = torch.zeros(1, 2, 256, 64, dtype=torch.float16)
    forbid_read_backs(monkeypatch)
    oat.omni_attention_simple(q, q, q, moved)
    oat.omni_attention_shared_kv(q, q, q, moved)
    assert ext.calls[0][1][12] is False      # tensors present, no PARTIAL slot
    assert ext.calls[1][1][12] is True       # shared_kv: both tensors present is enough (:641-642)
