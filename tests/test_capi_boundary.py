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
    assert omni_attn_capi.load_library().omni_attn_abi_version() == 4


def test_argument_validation_codes():
    lib = omni_attn_capi.load_library()
    one = 4096  # any non-null value: validation fails before it would be dereferenced
    def call(q=one, D=128, QB=128, KB=128, Tq=4, S=512, dtype=1, B=1, P=0, softcap=0.0):
        return omni_attn_capi.fwd_raw(q, one, one, one, 0, one, one, one, 0, 0,
                                      B, 2, S, D, Tq, 4, QB, KB, P, S, dtype, 0, softcap)
    assert call(q=0) == 1
    assert call(B=0) == 2
    assert call(Tq=5) == 2            # Tq != ceil(S / QB)
    assert call(P=-1) == 2            # negative number of stored partial tiles
    assert call(softcap=-1.0) == 2    # softcap must be 0 (off) or positive and finite
    assert call(softcap=float("nan")) == 2 and call(softcap=float("inf")) == 2
    assert call(D=96) == 3
    assert call(D=256) == 3
    assert call(QB=32) == 4
    assert call(KB=256) == 4
    assert call(dtype=7) == 5
    assert call(q=one + 8) == 8     # 16-byte alignment of q, k, v, o
    for code in range(0, 11):
        assert omni_attn_capi.status_string(code)
    assert "head_dim" in omni_attn_capi.status_string(3)


def test_python_module_surface():
    import omni_attn
    for name in ("omni_attn_mma_stages_split_q_shared_kv", "omni_attn_simple_kernel", "omni_attn_cp_async",
                 "omni_attn_preftech_kernel", "omni_attn_preftech",
                 "omni_attn_mma_stages_split_q_shared_kv_swizzle", "omni_attn_forward"):
        assert callable(getattr(omni_attn, name)), name
    assert omni_attn.abi_version() == 4
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


def test_kernel_resources_of_the_built_library():
    """The build records registers / scratch / occupancy of every kernel instance and refuses
    instances that spill or lose occupancy; the record of the library in the tree passes the
    same check (and the check itself rejects a spilling or low-occupancy record)."""
    import importlib.util
    import json
    spec = importlib.util.spec_from_file_location("_omni_build", os.path.join(PKG, "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    if not os.path.exists(build.RESOURCES_JSON):
        build.build_capi(jobs=4)
    with open(build.RESOURCES_JSON) as f:
        kernels = json.load(f)
    fwd = {k: v for k, v in kernels.items() if "fwd_kernel" in k}
    assert len(fwd) == 24
    build.check_resources(kernels)
    for name, r in fwd.items():
        assert r["scratch_bytes"] == 0 and r["vgprs"] <= 256 and r["waves_per_simd"] >= 2, (name, r)
    # both backward kernels, plain and soft-capped, 24 instances each way: two waves per SIMD or more
    for tag in ("bwd_dq_kernel", "bwd_dkdv_kernel"):
        inst = {k: v for k, v in kernels.items() if tag in k}
        assert len(inst) == 48
        for name, r in inst.items():
            assert r["scratch_bytes"] == 0 and r["waves_per_simd"] >= 2, (name, r)
    low_bwd = {"k_bwd_dkdv_kernel_x": {"scratch_bytes": 0, "vgpr_spills": 0, "sgpr_spills": 0, "waves_per_simd": 1}}
    with pytest.raises(RuntimeError, match="waves per SIMD"):
        build.check_resources(low_bwd)
    bad = {"k_fwd_kernel_x": {"scratch_bytes": 16, "vgpr_spills": 4, "sgpr_spills": 0, "waves_per_simd": 2}}
    with pytest.raises(RuntimeError, match="scratch"):
        build.check_resources(bad)
    low = {"k_fwd_kernel_x": {"scratch_bytes": 0, "vgpr_spills": 0, "sgpr_spills": 0, "waves_per_simd": 1}}
    with pytest.raises(RuntimeError, match="waves per SIMD"):
        build.check_resources(low)
    remarks = ("a.hpp:1:1: remark: Function Name: kern_a [-Rpass-analysis=kernel-resource-usage]\n"
               "a.hpp:1:1: remark:     VGPRs: 77 [-Rpass-analysis=kernel-resource-usage]\n"
               "a.hpp:1:1: remark:     ScratchSize [bytes/lane]: 8 [-Rpass-analysis=kernel-resource-usage]\n"
               "a.hpp:1:1: remark:     Occupancy [waves/SIMD]: 5 [-Rpass-analysis=kernel-resource-usage]\n")
    assert build.parse_resource_remarks(remarks) == {"kern_a": {"vgprs": 77, "scratch_bytes": 8, "waves_per_simd": 5}}
