"""The C-ABI library and the Python module load and export what include/*.h declares.
CPU only: no kernel is launched (argument validation returns before any device work)."""
import ctypes
import glob
import os
import re

import pytest
import torch

from conftest import PKG, ROOT

import omni_attn_capi


def _declared_functions():
    names = []
    for header in glob.glob(os.path.join(ROOT, "include", "*.h")):
        text = open(header).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names += re.findall(r"\b(omni_attn_\w+)\s*\(", text)
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    declared = _declared_functions()
    assert set(declared) == set(omni_attn_capi.EXPORTED_SYMBOLS)
    lib = ctypes.CDLL(omni_attn_capi.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert omni_attn_capi.load_library().omni_attn_abi_version() == 1


def test_argument_validation_codes():
    lib = omni_attn_capi.load_library()
    one = 4096  # any non-null value: validation fails before it would be dereferenced
    def call(q=one, D=128, QB=128, KB=128, Tq=4, S=512, dtype=1, B=1):
        return omni_attn_capi.fwd_raw(q, one, one, one, 0, one, one, one, 0, 0,
                                      B, 2, S, D, Tq, 4, QB, KB, S, dtype, 0)
    assert call(q=0) == 1
    assert call(B=0) == 2
    assert call(Tq=5) == 2            # Tq != ceil(S / QB)
    assert call(D=96) == 3
    assert call(D=256) == 3
    assert call(QB=32) == 4
    assert call(KB=256) == 4
    assert call(dtype=7) == 5
    assert call(q=one + 8) == 8     # 16-byte alignment of q, k, v, o
    for code in range(0, 9):
        assert omni_attn_capi.status_string(code)
    assert "head_dim" in omni_attn_capi.status_string(3)


def test_python_module_surface():
    import omni_attn
    for name in ("omni_attn_mma_stages_split_q_shared_kv", "omni_attn_simple_kernel", "omni_attn_cp_async",
                 "omni_attn_preftech_kernel", "omni_attn_preftech",
                 "omni_attn_mma_stages_split_q_shared_kv_swizzle", "omni_attn_forward"):
        assert callable(getattr(omni_attn, name)), name
    assert omni_attn.abi_version() == 1
    assert os.path.dirname(omni_attn.__file__) == PKG


def test_module_rejects_bad_tensors_with_runtime_error():
    """Errors surface as RuntimeError like the reference's std::runtime_error."""
    import omni_attn
    q = torch.zeros(1, 1, 128, 64, dtype=torch.float16)
    nb = torch.ones(1, 1, 1, dtype=torch.int32)
    idx = torch.zeros(1, 1, 1, 1, dtype=torch.int32)
    e_i = torch.empty(0, dtype=torch.int32)
    e_b = torch.empty(0, dtype=torch.bool)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        omni_attn.omni_attn_simple_kernel(q, q, q, q.clone(), nb, idx, idx, 128, 128, 128, e_i, e_b, False)
    with pytest.raises(RuntimeError, match="dtype"):
        omni_attn.omni_attn_simple_kernel(q.float(), q, q, q.clone(), nb, idx, idx, 128, 128, 128, e_i, e_b, False)
    with pytest.raises(TypeError):  # 13 positional arguments, no keywords, as in the reference
        omni_attn.omni_attn_simple_kernel(q, q, q, q.clone(), nb, idx, idx, Q_BLOCK_SIZE=128)


def test_wrappers_validate_before_launch():
    from omni_attn_torch import create_causal_omni_block_mask, omni_attention_shared_kv
    mask = create_causal_omni_block_mask(1, 2, 256, 256, 128, 128, device="cpu")
    q = torch.zeros(1, 2, 256, 64, dtype=torch.float16)
    with pytest.raises(AssertionError, match="Q and KV sequence lengths must match"):
        omni_attention_shared_kv(q, q[:, :, :128], q[:, :, :128], mask)
    with pytest.raises(AssertionError, match="doesn't match mask q_len"):
        omni_attention_shared_kv(q[:, :, :100], q[:, :, :100], q[:, :, :100], mask)
    with pytest.raises(ValueError, match="head_dim"):
        omni_attention_shared_kv(torch.zeros(1, 2, 256, 48, dtype=torch.float16),
                                 torch.zeros(1, 2, 256, 48, dtype=torch.float16),
                                 torch.zeros(1, 2, 256, 48, dtype=torch.float16), mask)
    with pytest.raises(ValueError, match="dtype"):
        omni_attention_shared_kv(q.float(), q.float(), q.float(), mask)
