"""ctypes binding of the C restatement (test infrastructure, see oracle/__init__.py)."""
import ctypes
import os
from typing import Optional, Tuple

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libomni_oracle.so")
_lib = None


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            from . import build as _build
            _build.build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.omni_oracle_block_walk.restype = ctypes.c_int
    return _lib


def _ptr(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def attention_block_walk(q, k, v, kv_num_blocks, kv_indices, block_mask_types, QB: int, KB: int,
                         seqlen_orig: Optional[int] = None, partial_idx=None,
                         partial_masks=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """q, k, v [B, H, S, D] (any float dtype; converted to fp32 as they are) -> (O, LSE) fp32."""
    lib = _load()
    qf, kf, vf = (t.detach().cpu().float().contiguous() for t in (q, k, v))
    B, H, S, D = qf.shape
    nb = kv_num_blocks.cpu().to(torch.int32).contiguous()
    idx = kv_indices.cpu().to(torch.int32).contiguous()
    tys = block_mask_types.cpu().to(torch.int32).contiguous()
    pidx = None if partial_idx is None else partial_idx.cpu().to(torch.int32).contiguous()
    pm = None if partial_masks is None else partial_masks.cpu().to(torch.uint8).contiguous()
    if pm is not None and pm.numel() == 0:
        pidx, pm = None, None
    o = torch.empty_like(qf)
    lse = torch.empty(B, H, S, dtype=torch.float32)
    rc = lib.omni_oracle_block_walk(_ptr(qf), _ptr(kf), _ptr(vf), _ptr(o), _ptr(lse), _ptr(nb),
                                    _ptr(idx), _ptr(tys), _ptr(pidx), _ptr(pm), B, H, S, D,
                                    nb.shape[2], idx.shape[3], QB, KB,
                                    0 if pm is None else int(pm.shape[0]),
                                    S if seqlen_orig is None else int(seqlen_orig))
    if rc != 0:
        raise RuntimeError("omni_oracle_block_walk failed with %d" % rc)
    return o, lse
