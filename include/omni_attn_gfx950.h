/*
 * C ABI of the gfx950 (MI355X / CDNA4) block-sparse FlashAttention-2 forward.
 *
 * This is the boundary a binding for the reference's operator would bind: plain
 * pointers and sizes, no torch types.  The reference exposes the same operation
 * through five pybind entry points that share one 13-argument signature
 * (omni-attn-mma/pybind/omni_attn.cc:10-68, exported at :70-77); each of them
 * unpacks its torch::Tensor arguments into exactly the pointer/size list below
 * before launching (e.g. omni-attn-mma/mma/attn_naive.cu:317-402).
 *
 * All pointers are device pointers valid on the device that is current when the
 * call is made.  Calls are asynchronous: work is enqueued on `stream` and the
 * function returns without waiting.  No device memory is allocated or freed by
 * any entry point and no state is kept between calls.
 */
#ifndef OMNI_ATTN_GFX950_H
#define OMNI_ATTN_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element type of Q, K, V and O (fp32 accumulation in both cases). */
enum omni_attn_dtype {
  OMNI_ATTN_DTYPE_F16 = 0,
  OMNI_ATTN_DTYPE_BF16 = 1
};

/* Block types, values fixed by omni-attn-mma/omni_attn_torch.py:38-41 and
 * omni-attn-mma/mma/attn_naive.cu:4-7. */
enum omni_attn_block_type {
  OMNI_ATTN_BLOCK_MASKED = 0,
  OMNI_ATTN_BLOCK_CAUSAL = 1,
  OMNI_ATTN_BLOCK_FULL = 2,
  OMNI_ATTN_BLOCK_PARTIAL = 3
};

/* Return codes.  0 is success; everything else leaves O untouched. */
enum omni_attn_status {
  OMNI_ATTN_OK = 0,
  OMNI_ATTN_ERR_NULL_POINTER = 1,      /* a required pointer is NULL */
  OMNI_ATTN_ERR_BAD_SHAPE = 2,         /* non-positive size, or Tq != ceil(S_pad / QB) */
  OMNI_ATTN_ERR_UNSUPPORTED_HEAD_DIM = 3,   /* D not in {32, 64, 128} */
  OMNI_ATTN_ERR_UNSUPPORTED_BLOCK = 4, /* QB or KB not in {64, 128} */
  OMNI_ATTN_ERR_UNSUPPORTED_DTYPE = 5,
  OMNI_ATTN_ERR_LAUNCH = 6,            /* hipLaunch failed; see omni_attn_last_hip_error() */
  OMNI_ATTN_ERR_TOO_LARGE = 7,         /* a tensor exceeds 2^31-1 elements per (b,h) slab */
  OMNI_ATTN_ERR_MISALIGNED = 8,        /* q, k, v, o or partial masks not 16-byte aligned, or a
                                          32-bit array not 4-byte aligned */
  OMNI_ATTN_ERR_WORKSPACE = 9,         /* workspace smaller than omni_attn_bwd_workspace_bytes() */
  OMNI_ATTN_ERR_SCRATCH_LIMIT = 10     /* omni_attn_bwd_noalloc_gfx950: B * H * S_pad beyond its
                                          built-in scratch (omni_attn_bwd_noalloc_max_rows()) */
};

/*
 * Block-sparse attention forward:  for every (b, h) and every query block qb,
 *   O[b,h,q,:] = softmax_k( mask(Q[b,h,q,:] . K[b,h,k,:] / sqrt(D)) ) V[b,h,k,:]
 * over the KV blocks listed in kv_indices[b,h,qb,0:kv_num_blocks[b,h,qb]] only.
 *
 * Replaces the body of the reference's five launchers
 *   omni_attn_simple_kernel                         (omni-attn-mma/mma/attn_naive.cu:305-408)
 *   omni_attn_cp_async                              (omni-attn-mma/mma/omni_attn_cp_async.cu)
 *   omni_attn_preftech_kernel                       (omni-attn-mma/mma/omni_attn_preftech.cu)
 *   omni_attn_mma_stages_split_q_shared_kv          (omni-attn-mma/mma/omni_attn_shared_kv.cu:693-1009)
 *   omni_attn_mma_stages_split_q_shared_kv_swizzle  (omni-attn-mma/mma/omni_attn_swizzle.cu:721-1036)
 * with the mask semantics of the scalar kernel (omni-attn-mma/mma/attn_naive.cu:21-302):
 *
 *   q, k, v, o       [B, H, S_pad, D] row-major, 16-bit elements of type `dtype`.
 *   lse_or_null      [B, H, S_pad] fp32 natural-log logsumexp of the masked, scaled
 *                    scores of each row, or NULL to skip it (the reference has no such
 *                    output).  Rows with no allowed key get -inf.
 *   kv_num_blocks    [B, H, Tq] int32.
 *   kv_indices       [B, H, Tq, max_blocks] int32, KV block index per slot.
 *   block_mask_types [B, H, Tq, max_blocks] int32, omni_attn_block_type per slot.
 *   partial_idx_or_null   [B, H, Tq, max_blocks] int32 index into partial_masks for
 *                    PARTIAL slots (-1 = none), or NULL when has_partial is false.
 *   partial_masks_or_null [P, QB, KB] one byte per element, non-zero = attend, 0 = masked
 *                    (torch.bool storage; any non-zero byte counts as attend, as in
 *                    attn_naive.cu:151), row-major q_local*KB + k_local, or NULL.
 *   num_partial      P, the number of tiles stored in partial_masks (0 when NULL).  The
 *                    reference reads tile partial_idx[...] unchecked (attn_naive.cu:124-131);
 *                    here an index outside [0, P) means "no bits stored".
 *   Tq               number of query blocks, must equal ceil(S_pad / QB).
 *   seqlen_orig      rows >= seqlen_orig are written as zeros (lse -inf); keys
 *                    >= seqlen_orig are never attended (attn_naive.cu:64-72, :113).  Those rows
 *                    of q, k and v are never read: the padding may hold anything.
 *   softcap          0 = off (the reference's operator).  > 0: the scaled score x = q.k / sqrt(D)
 *                    is replaced by softcap * tanh(x / softcap) before the mask and the softmax,
 *                    the score_mod Transfusion's attention layer passes to flex_attention
 *                    (transfusion_pytorch/transfusion.py:358-364, :958-959).  Negative, NaN or
 *                    infinite values are refused (OMNI_ATTN_ERR_BAD_SHAPE).
 *
 * Semantics per slot: MASKED is skipped; FULL keeps everything; CAUSAL keeps
 * k_global <= q_global; PARTIAL keeps the stored bytes; a PARTIAL slot whose
 * partial pointers are NULL or whose index is negative (attn_naive.cu:119-131) or
 * >= num_partial is skipped.  A row with no allowed key yields O = 0.
 * The softmax scale is always 1/sqrt(D) (attn_naive.cu:88).
 * Out-of-range metadata cannot fault the device: kv_num_blocks is clamped to
 * [0, max_blocks], kv_indices to [0, ceil(S_pad / KB) - 1], and a partial index outside
 * [0, num_partial) skips its slot.
 *
 * `stream` is a hipStream_t passed as void* (NULL = the legacy default stream).
 */
int omni_attn_fwd_gfx950(const void* q, const void* k, const void* v, void* o,
                         float* lse_or_null,
                         const int32_t* kv_num_blocks,
                         const int32_t* kv_indices,
                         const int32_t* block_mask_types,
                         const int32_t* partial_idx_or_null,
                         const uint8_t* partial_masks_or_null,
                         int B, int H, int S_pad, int D,
                         int Tq, int max_blocks, int QB, int KB, int num_partial,
                         int seqlen_orig, int dtype, float softcap, void* stream);

/*
 * The same operation for shapes the MFMA kernel has no instance for: any QB > 0, KB > 0 and any
 * D in 1..256 -- the generality of the reference's scalar kernel omni_attn_simple_kernel
 * (omni-attn-mma/mma/attn_naive.cu:21-302; D <= 256 from its `float out[256]`, :189-190; its
 * launcher :305-408 has no block-size or head-dim whitelist).  Same arguments, semantics and
 * status codes as omni_attn_fwd_gfx950 (pointers need only their natural alignment); two-pass
 * fp32 softmax per query row like the reference's kernel.  A correctness path, not a fast one.
 */
int omni_attn_fwd_generic_gfx950(const void* q, const void* k, const void* v, void* o,
                                 float* lse_or_null,
                                 const int32_t* kv_num_blocks,
                                 const int32_t* kv_indices,
                                 const int32_t* block_mask_types,
                                 const int32_t* partial_idx_or_null,
                                 const uint8_t* partial_masks_or_null,
                                 int B, int H, int S_pad, int D,
                                 int Tq, int max_blocks, int QB, int KB, int num_partial,
                                 int seqlen_orig, int dtype, float softcap, void* stream);

/*
 * Pre-pass for masks that are reused over many launches: packs the bool tiles that the
 * reference's build_partial_block_data produces (omni-attn-mma/omni_attn_torch.py:148-205,
 * [P, QB, KB] bytes) into [P, QB, KB / 32] 32-bit words, bit j of word c of a row = key
 * 32 c + j of that row, any non-zero byte counting as set.  QB, KB in {64, 128};
 * partial_masks 16-byte aligned.  Asynchronous on `stream`; allocates nothing.
 */
int omni_attn_pack_partial_masks_gfx950(const uint8_t* partial_masks, uint32_t* partial_bits,
                                        int num_partial, int QB, int KB, void* stream);

/*
 * omni_attn_fwd_gfx950 with the PARTIAL tiles already packed by
 * omni_attn_pack_partial_masks_gfx950 (same semantics and results bit for bit; the byte
 * tiles of the reference's signature, omni-attn-mma/pybind/omni_attn.cc:10-68, are
 * replaced by their packed form).
 */
int omni_attn_fwd_packed_gfx950(const void* q, const void* k, const void* v, void* o,
                                float* lse_or_null,
                                const int32_t* kv_num_blocks,
                                const int32_t* kv_indices,
                                const int32_t* block_mask_types,
                                const int32_t* partial_idx_or_null,
                                const uint32_t* partial_bits_or_null,
                                int B, int H, int S_pad, int D,
                                int Tq, int max_blocks, int QB, int KB, int num_partial,
                                int seqlen_orig, int dtype, float softcap, void* stream);

/*
 * Backward of omni_attn_fwd_gfx950: gradients of a scalar loss with respect to q, k and v,
 * given dout = dLoss/dO and the o and lse the forward wrote for the same q, k, v and mask.
 * The reference's operator is forward-only (omni-attn-mma/pybind/omni_attn.cc:70-77 exports no
 * backward); this is what a caller needs to put the operator into the attention layer of
 * transfusion_pytorch/transfusion.py:953-983 for training.  What is differentiated is exactly
 * the forward's function: listed blocks only, FULL / CAUSAL / PARTIAL / MASKED semantics,
 * scale 1/sqrt(D), rows >= seqlen_orig and rows with no allowed key get zero gradients.
 *
 *   dout, dq, dk, dv  [B, H, S_pad, D], same 16-bit type as q.  dq, dk, dv are written
 *                     completely (rows of K/V that no query attends get zeros).
 *   lse               [B, H, S_pad] fp32 as written by the forward (required).
 *   partial tiles     as bytes (partial_masks_or_null) or packed (partial_bits_or_null);
 *                     pass one of them or neither.
 *   workspace         device memory of at least omni_attn_bwd_workspace_bytes(B, H, S_pad)
 *                     bytes (two floats per row), 4-byte aligned; holds -rowsum(dout . o) and
 *                     the rows' exponent offsets between the two kernels of the backward.
 *                     Contents before and after the call are meaningless.
 * No limits beyond the forward's (Tq * ceil(max_blocks / 64) must fit an int).  Metadata of more
 * than 4096 64-slot words per (batch, head) slab (2602 at head_dim 128 with 128-key blocks) is
 * scanned in windows of that many words by every dK/dV workgroup.
 * Rows at or beyond seqlen_orig of q, k, v, o and dout are never read (the padding may hold anything).
 * Two kernels are enqueued on `stream`; nothing is allocated; results are bitwise reproducible.
 */
size_t omni_attn_bwd_workspace_bytes(int B, int H, int S_pad);
int omni_attn_bwd_gfx950(const void* q, const void* k, const void* v, const void* o,
                         const void* dout, const float* lse,
                         void* dq, void* dk, void* dv,
                         const int32_t* kv_num_blocks,
                         const int32_t* kv_indices,
                         const int32_t* block_mask_types,
                         const int32_t* partial_idx_or_null,
                         const uint8_t* partial_masks_or_null,
                         const uint32_t* partial_bits_or_null,
                         void* workspace, size_t workspace_bytes,
                         int B, int H, int S_pad, int D,
                         int Tq, int max_blocks, int QB, int KB, int num_partial,
                         int seqlen_orig, int dtype, float softcap, void* stream);

/*
 * omni_attn_bwd_gfx950 for callers that cannot allocate device memory for the workspace: code
 * under HIP graph capture, tight serving or training loops, harnesses that forbid allocation.
 * No counterpart in the reference.  Same kernels and bit-identical results; the workspace is a
 * 32 MiB device array built into the library (each GPU the library runs on holds its copy until
 * the process ends), so B * H * S_pad must not exceed omni_attn_bwd_noalloc_max_rows()
 * (4 194 304), else OMNI_ATTN_ERR_SCRATCH_LIMIT.  Calls no hipMalloc / hipFree or any other
 * allocating routine.  All calls on one GPU share that GPU's array: calls that overlap in time
 * on one GPU (different streams, different threads) race and must be serialised by the caller.
 * Before recording a call into a HIP graph make one eager call with the same dtype, head_dim, block
 * sizes and soft-cap setting on that device: the first call per device looks up the array's address
 * and the device's topology, the first call per kernel instance raises that instance's dynamic-LDS
 * limit -- none of them a stream operation.
 */
size_t omni_attn_bwd_noalloc_max_rows(void);
int omni_attn_bwd_noalloc_gfx950(const void* q, const void* k, const void* v, const void* o,
                                 const void* dout, const float* lse,
                                 void* dq, void* dk, void* dv,
                                 const int32_t* kv_num_blocks,
                                 const int32_t* kv_indices,
                                 const int32_t* block_mask_types,
                                 const int32_t* partial_idx_or_null,
                                 const uint8_t* partial_masks_or_null,
                                 const uint32_t* partial_bits_or_null,
                                 int B, int H, int S_pad, int D,
                                 int Tq, int max_blocks, int QB, int KB, int num_partial,
                                 int seqlen_orig, int dtype, float softcap, void* stream);

/*
 * Measurement aid (no counterpart in the reference): enqueue a kernel that issues nothing but
 * 32x32x16 matrix instructions of `dtype` from registers -- two workgroups of four waves per
 * compute unit, `iters` x 8 instructions per wave -- so that a caller timing the launch can
 * report what the matrix cores of this device sustain at the clock they get under that
 * load.  *flops_out receives the flop count of the launch; `sink` is a device float the
 * kernel may write.  Allocates nothing.
 */
int omni_attn_mfma_peak_probe_gfx950(int dtype, int iters, float* sink, double* flops_out,
                                     void* stream);

/* Static description of a return code (never NULL). */
const char* omni_attn_status_string(int status);

/* hipError_t of the most recent failed launch on the calling thread (0 if none). */
int omni_attn_last_hip_error(void);

/* Version of this ABI; bumped when a signature changes (2: num_partial added; 3: softcap added;
 * 4: the two study probes omni_attn_mfma_mix_probe_gfx950 / omni_attn_issue_probe_gfx950 removed). */
int omni_attn_abi_version(void);

#ifdef __cplusplus
}
#endif

#endif /* OMNI_ATTN_GFX950_H */
