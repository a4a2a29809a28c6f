"""ctypes binding of the C ABI in include/omni_attn_gfx950.h.

This is the stub a Python caller that does not want the torch extension module would
write: it hands raw device pointers and sizes to ``libomni_attn_gfx950.so``.  Tensors
are only used here as owners of device memory.  There is no fallback: a missing
library raises ``OSError`` on first use.
"""
import ctypes
import os
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libomni_attn_gfx950.so")

DTYPE_F16 = 0
DTYPE_BF16 = 1

EXPORTED_SYMBOLS = (
    "omni_attn_fwd_gfx950",
    "omni_attn_fwd_packed_gfx950",
    "omni_attn_fwd_generic_gfx950",
    "omni_attn_pack_partial_masks_gfx950",
    "omni_attn_bwd_gfx950",
    "omni_attn_bwd_workspace_bytes",
    "omni_attn_bwd_noalloc_gfx950",
    "omni_attn_bwd_noalloc_max_rows",
    "omni_attn_mfma_peak_probe_gfx950",
    "omni_attn_status_string",
    "omni_attn_last_hip_error",
    "omni_attn_abi_version",
)

_lib = None


def load_library() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        lib = ctypes.CDLL(LIB_PATH)
        vp, i32 = ctypes.c_void_p, ctypes.c_int
        lib.omni_attn_fwd_gfx950.restype = i32
        lib.omni_attn_fwd_gfx950.argtypes = [vp] * 10 + [i32] * 11 + [ctypes.c_float, vp]
        lib.omni_attn_fwd_generic_gfx950.restype = i32
        lib.omni_attn_fwd_generic_gfx950.argtypes = [vp] * 10 + [i32] * 11 + [ctypes.c_float, vp]
        lib.omni_attn_fwd_packed_gfx950.restype = i32
        lib.omni_attn_fwd_packed_gfx950.argtypes = [vp] * 10 + [i32] * 11 + [ctypes.c_float, vp]
        lib.omni_attn_pack_partial_masks_gfx950.restype = i32
        lib.omni_attn_pack_partial_masks_gfx950.argtypes = [vp, vp, i32, i32, i32, vp]
        lib.omni_attn_bwd_workspace_bytes.restype = ctypes.c_size_t
        lib.omni_attn_bwd_workspace_bytes.argtypes = [i32, i32, i32]
        lib.omni_attn_bwd_gfx950.restype = i32
        lib.omni_attn_bwd_gfx950.argtypes = [vp] * 16 + [ctypes.c_size_t] + [i32] * 11 + [ctypes.c_float, vp]
        lib.omni_attn_bwd_noalloc_max_rows.restype = ctypes.c_size_t
        lib.omni_attn_bwd_noalloc_gfx950.restype = i32
        lib.omni_attn_bwd_noalloc_gfx950.argtypes = [vp] * 15 + [i32] * 11 + [ctypes.c_float, vp]
        lib.omni_attn_mfma_peak_probe_gfx950.restype = i32
        lib.omni_attn_mfma_peak_probe_gfx950.argtypes = [i32, i32, vp, ctypes.POINTER(ctypes.c_double), vp]
        lib.omni_attn_status_string.restype = ctypes.c_char_p
        lib.omni_attn_status_string.argtypes = [i32]
        lib.omni_attn_last_hip_error.restype = i32
        lib.omni_attn_abi_version.restype = i32
        _lib = lib
    return _lib


def status_string(code: int) -> str:
    return load_library().omni_attn_status_string(int(code)).decode()


def mfma_peak_probe(dtype: int, iters: int, sink: torch.Tensor, stream: Optional[int] = None) -> float:
    """Enqueue the pure matrix-instruction loop; returns the flop count of the launch."""
    flops = ctypes.c_double(0.0)
    if stream is None:
        stream = torch.cuda.current_stream(sink.device).cuda_stream
    with torch.cuda.device(sink.device):
        rc = load_library().omni_attn_mfma_peak_probe_gfx950(dtype, iters, sink.data_ptr(), ctypes.byref(flops), stream)
    if rc != 0:
        raise RuntimeError("omni_attn_mfma_peak_probe_gfx950: %s (status %d)" % (status_string(rc), rc))
    return flops.value


def _ptr(t: Optional[torch.Tensor]) -> int:
    return 0 if t is None else t.data_ptr()


def fwd_raw(q_ptr, k_ptr, v_ptr, o_ptr, lse_ptr, nb_ptr, idx_ptr, types_ptr, pidx_ptr, pmask_ptr,
            B, H, S_pad, D, Tq, max_blocks, QB, KB, num_partial, seqlen_orig, dtype, stream_ptr,
            softcap: float = 0.0) -> int:
    """The C call itself; returns the status code."""
    return load_library().omni_attn_fwd_gfx950(
        q_ptr, k_ptr, v_ptr, o_ptr, lse_ptr, nb_ptr, idx_ptr, types_ptr, pidx_ptr, pmask_ptr,
        B, H, S_pad, D, Tq, max_blocks, QB, KB, num_partial, seqlen_orig, dtype, softcap, stream_ptr)


def pack_partial_masks(partial_masks: torch.Tensor, stream: Optional[int] = None) -> torch.Tensor:
    """[P, QB, KB] bool / uint8 tiles on the GPU -> [P, QB, KB // 32] int32 words (the bit
    pattern of the library's uint32 words), packed by the library's pre-pass kernel."""
    if not (partial_masks.is_cuda and partial_masks.is_contiguous() and partial_masks.dim() == 3
            and partial_masks.dtype in (torch.bool, torch.uint8)):
        raise RuntimeError("partial_masks must be a contiguous [P, QB, KB] bool GPU tensor")
    P, QB, KB = partial_masks.shape
    out = torch.empty(P, QB, KB // 32, dtype=torch.int32, device=partial_masks.device)
    if stream is None:
        stream = torch.cuda.current_stream(partial_masks.device).cuda_stream
    with torch.cuda.device(partial_masks.device):
        rc = load_library().omni_attn_pack_partial_masks_gfx950(partial_masks.data_ptr(), out.data_ptr(), P, QB, KB, stream)
    if rc != 0:
        raise RuntimeError("omni_attn_pack_partial_masks_gfx950: %s (status %d)" % (status_string(rc), rc))
    return out


def fwd(q, k, v, o, lse, kv_num_blocks, kv_indices, block_mask_types, QB, KB, seqlen_orig,
        partial_idx=None, partial_masks=None, stream: Optional[int] = None, partial_bits=None,
        softcap: float = 0.0, generic: bool = False) -> None:
    """Enqueue the forward on ``stream`` (default: torch's current stream of q's device).
    q, k, v, o: contiguous [B, H, S_pad, D] fp16 or bf16 on the GPU; lse: fp32 [B, H, S_pad]
    or None.  PARTIAL tiles either as bytes (``partial_masks``) or packed by
    ``pack_partial_masks`` (``partial_bits``).  Raises RuntimeError with the library's message
    on a non-zero status."""
    B, H, S, D = q.shape
    for t in (q, k, v, o):
        if not (t.is_cuda and t.is_contiguous() and t.dtype == q.dtype and t.shape == q.shape):
            raise RuntimeError("q, k, v, o must be contiguous GPU tensors of one shape and dtype")
    if q.dtype == torch.bfloat16:
        dtype = DTYPE_BF16
    elif q.dtype == torch.float16:
        dtype = DTYPE_F16
    else:
        raise RuntimeError("q must be torch.float16 or torch.bfloat16")
    for t in (kv_num_blocks, kv_indices, block_mask_types) + ((partial_idx,) if partial_idx is not None else ()):
        if not (t.is_cuda and t.is_contiguous() and t.dtype == torch.int32):
            raise RuntimeError("block-mask tensors must be contiguous int32 GPU tensors")
    if partial_masks is not None:
        if not (partial_masks.is_cuda and partial_masks.is_contiguous()
                and partial_masks.dtype in (torch.bool, torch.uint8)):
            raise RuntimeError("partial_masks must be a contiguous bool GPU tensor")
        if partial_masks.numel() == 0:
            partial_idx, partial_masks = None, None
    if stream is None:
        stream = torch.cuda.current_stream(q.device).cuda_stream
    if partial_bits is not None:
        if partial_masks is not None:
            raise RuntimeError("pass partial_masks or partial_bits, not both")
        if not (partial_bits.is_cuda and partial_bits.is_contiguous() and partial_bits.dtype == torch.int32
                and partial_bits.dim() == 3 and partial_bits.shape[1:] == (QB, KB // 32)):
            raise RuntimeError("partial_bits must be a contiguous [P, QB, KB // 32] int32 GPU tensor")
        with torch.cuda.device(q.device):
            rc = load_library().omni_attn_fwd_packed_gfx950(
                _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), _ptr(kv_num_blocks), _ptr(kv_indices),
                _ptr(block_mask_types), _ptr(partial_idx if partial_bits.shape[0] else None),
                _ptr(partial_bits if partial_bits.shape[0] else None), B, H, S, D, kv_num_blocks.shape[2],
                kv_indices.shape[3], QB, KB, int(partial_bits.shape[0]), int(seqlen_orig), dtype, float(softcap),
                stream)
        if rc != 0:
            raise RuntimeError("omni_attn_fwd_packed_gfx950: %s (status %d)" % (status_string(rc), rc))
        return
    if generic:
        with torch.cuda.device(q.device):
            rc = load_library().omni_attn_fwd_generic_gfx950(
                _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), _ptr(kv_num_blocks), _ptr(kv_indices),
                _ptr(block_mask_types), _ptr(partial_idx), _ptr(partial_masks), B, H, S, D, kv_num_blocks.shape[2],
                kv_indices.shape[3], QB, KB, 0 if partial_masks is None else int(partial_masks.shape[0]),
                int(seqlen_orig), dtype, float(softcap), stream)
        if rc != 0:
            raise RuntimeError("omni_attn_fwd_generic_gfx950: %s (status %d)" % (status_string(rc), rc))
        return
    with torch.cuda.device(q.device):
        rc = fwd_raw(_ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), _ptr(kv_num_blocks),
                     _ptr(kv_indices), _ptr(block_mask_types), _ptr(partial_idx), _ptr(partial_masks),
                     B, H, S, D, kv_num_blocks.shape[2], kv_indices.shape[3], QB, KB,
                     0 if partial_masks is None else int(partial_masks.shape[0]),
                     int(seqlen_orig), dtype, stream, float(softcap))
    if rc != 0:
        raise RuntimeError("omni_attn_fwd_gfx950: %s (status %d)" % (status_string(rc), rc))


def bwd(q, k, v, o, dout, lse, dq, dk, dv, kv_num_blocks, kv_indices, block_mask_types, QB, KB, seqlen_orig,
        partial_idx=None, partial_masks=None, partial_bits=None, workspace: Optional[torch.Tensor] = None,
        stream: Optional[int] = None, no_alloc: bool = False, softcap: float = 0.0) -> None:
    """Enqueue the backward (two kernels) on ``stream``.  All of q, k, v, o, dout, dq, dk, dv are
    contiguous [B, H, S_pad, D] GPU tensors of one 16-bit dtype, lse is the forward's fp32
    [B, H, S_pad].  ``workspace``: a GPU tensor of at least omni_attn_bwd_workspace_bytes bytes
    (allocated here, by torch, when not given).  ``no_alloc=True`` calls omni_attn_bwd_noalloc_gfx950
    instead: no workspace, the library's built-in scratch."""
    B, H, S, D = q.shape
    for t in (q, k, v, o, dout, dq, dk, dv):
        if not (t.is_cuda and t.is_contiguous() and t.dtype == q.dtype and t.shape == q.shape):
            raise RuntimeError("q, k, v, o, dout, dq, dk, dv must be contiguous GPU tensors of one shape and dtype")
    if q.dtype == torch.bfloat16:
        dtype = DTYPE_BF16
    elif q.dtype == torch.float16:
        dtype = DTYPE_F16
    else:
        raise RuntimeError("q must be torch.float16 or torch.bfloat16")
    if not (lse.is_cuda and lse.is_contiguous() and lse.dtype == torch.float32 and lse.shape == q.shape[:3]):
        raise RuntimeError("lse must be the forward's contiguous fp32 [B, H, S_pad] tensor")
    lib = load_library()
    ws_bytes = 0
    if not no_alloc:
        need = lib.omni_attn_bwd_workspace_bytes(B, H, S)
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
        ws_bytes = workspace.numel() * workspace.element_size()
    num_partial = 0
    if partial_bits is not None:
        num_partial = int(partial_bits.shape[0])
    elif partial_masks is not None:
        num_partial = int(partial_masks.shape[0])
    if num_partial == 0:
        partial_idx = partial_masks = partial_bits = None
    if stream is None:
        stream = torch.cuda.current_stream(q.device).cuda_stream
    if no_alloc:
        with torch.cuda.device(q.device):
            rc = lib.omni_attn_bwd_noalloc_gfx950(
                _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(dout), _ptr(lse), _ptr(dq), _ptr(dk), _ptr(dv),
                _ptr(kv_num_blocks), _ptr(kv_indices), _ptr(block_mask_types), _ptr(partial_idx),
                _ptr(partial_masks if partial_bits is None else None), _ptr(partial_bits),
                B, H, S, D, kv_num_blocks.shape[2], kv_indices.shape[3], QB, KB, num_partial, int(seqlen_orig),
                dtype, float(softcap), stream)
        if rc != 0:
            raise RuntimeError("omni_attn_bwd_noalloc_gfx950: %s (status %d)" % (status_string(rc), rc))
        return
    with torch.cuda.device(q.device):
        rc = lib.omni_attn_bwd_gfx950(
            _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(dout), _ptr(lse), _ptr(dq), _ptr(dk), _ptr(dv),
            _ptr(kv_num_blocks), _ptr(kv_indices), _ptr(block_mask_types), _ptr(partial_idx),
            _ptr(partial_masks if partial_bits is None else None), _ptr(partial_bits), _ptr(workspace), ws_bytes,
            B, H, S, D, kv_num_blocks.shape[2], kv_indices.shape[3], QB, KB, num_partial, int(seqlen_orig),
            dtype, float(softcap), stream)
    if rc != 0:
        raise RuntimeError("omni_attn_bwd_gfx950: %s (status %d)" % (status_string(rc), rc))
