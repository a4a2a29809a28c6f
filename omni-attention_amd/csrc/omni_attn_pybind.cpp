// Python module `omni_attn`: the operator surface the reference exports from
// omni-attn-mma/pybind/omni_attn.cc:70-77 (five functions, one 13-argument positional
// signature, :10-68), rebuilt over the gfx950 C ABI.  All five names run the same
// kernel; `omni_attn_preftech` is the name the reference's own wrapper tries to import
// (omni-attn-mma/omni_attn_torch.py:978), and `omni_attn_forward` additionally returns
// the row logsumexp.
//
// Host-only C++: the device code lives behind include/omni_attn_gfx950.h.
#include <torch/extension.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include <stdexcept>
#include <string>

#include "omni_attn_gfx950.h"

namespace {

void check_qkvo(const torch::Tensor& t, const char* name, const torch::Tensor& q) {
  if (!t.is_cuda()) throw std::runtime_error(std::string(name) + " must be a GPU tensor");
  if (t.dim() != 4) throw std::runtime_error(std::string(name) + " must have shape [B, H, S, D]");
  if (t.scalar_type() != q.scalar_type())
    throw std::runtime_error(std::string("Tensor dtype mismatch: ") + name +
                             " must have the dtype of Q (torch.float16 or torch.bfloat16)");
  if (t.sizes() != q.sizes())
    throw std::runtime_error(std::string(name) + " must have the shape of Q");
  if (t.device() != q.device())
    throw std::runtime_error(std::string(name) + " must be on the device of Q");
}

void check_meta(const torch::Tensor& t, const char* name, const torch::Tensor& q) {
  if (t.scalar_type() != torch::kInt32)
    throw std::runtime_error(std::string("Tensor dtype mismatch: ") + name + " must be torch.int32");
  if (t.device() != q.device())
    throw std::runtime_error(std::string(name) + " must be on the device of Q");
}

void forward_impl(const torch::Tensor& Q, const torch::Tensor& K, const torch::Tensor& V,
                  torch::Tensor& O, float* lse, const torch::Tensor& kv_num_blocks,
                  const torch::Tensor& kv_indices, const torch::Tensor& block_mask_types,
                  int Q_BLOCK_SIZE, int KV_BLOCK_SIZE, int seqlen_orig,
                  const torch::Tensor& partial_block_mask_indices,
                  const torch::Tensor& partial_block_masks, bool has_partial, bool packed = false,
                  double softcap = 0.0, bool generic_fallback = false) {
  if (Q.scalar_type() != torch::kHalf && Q.scalar_type() != torch::kBFloat16)
    throw std::runtime_error("Tensor dtype mismatch: Q must be torch.float16 or torch.bfloat16");
  check_qkvo(Q, "Q", Q);
  check_qkvo(K, "K", Q);
  check_qkvo(V, "V", Q);
  check_qkvo(O, "O", Q);
  if (!Q.is_contiguous() || !K.is_contiguous() || !V.is_contiguous() || !O.is_contiguous())
    throw std::runtime_error(
        "Q, K, V, O tensors must be contiguous. Call .contiguous() before calling this function.");
  check_meta(kv_num_blocks, "kv_num_blocks", Q);
  check_meta(kv_indices, "kv_indices", Q);
  check_meta(block_mask_types, "block_mask_types", Q);
  if (!kv_num_blocks.is_contiguous() || !kv_indices.is_contiguous() ||
      !block_mask_types.is_contiguous())
    throw std::runtime_error(
        "Block mask tensors must be contiguous. Call .contiguous() before calling this function.");

  const int64_t B = Q.size(0), H = Q.size(1), S = Q.size(2), D = Q.size(3);
  if (kv_num_blocks.dim() != 3 || kv_indices.dim() != 4 || block_mask_types.dim() != 4)
    throw std::runtime_error(
        "kv_num_blocks must be [B, H, num_q_blocks]; kv_indices and block_mask_types "
        "[B, H, num_q_blocks, max_blocks]");
  const int64_t num_q_blocks = kv_num_blocks.size(2);
  const int64_t max_blocks = kv_indices.size(3);
  if (Q_BLOCK_SIZE <= 0 || KV_BLOCK_SIZE <= 0)
    throw std::runtime_error("Q_BLOCK_SIZE and KV_BLOCK_SIZE must be positive");
  const int64_t expected = (S + Q_BLOCK_SIZE - 1) / Q_BLOCK_SIZE;
  if (num_q_blocks != expected)
    throw std::runtime_error("Block mask num_q_blocks (" + std::to_string(num_q_blocks) +
                             ") does not match expected value (" + std::to_string(expected) +
                             ") based on seqlen=" + std::to_string(S) +
                             " and Q_BLOCK_SIZE=" + std::to_string(Q_BLOCK_SIZE));
  if (kv_num_blocks.size(0) != B || kv_num_blocks.size(1) != H || kv_indices.size(0) != B ||
      kv_indices.size(1) != H || kv_indices.size(2) != num_q_blocks ||
      block_mask_types.sizes() != kv_indices.sizes())
    throw std::runtime_error("Block mask tensor shapes do not match Q's batch / heads / blocks");

  const int32_t* pidx = nullptr;
  const uint8_t* pmask = nullptr;
  int num_partial = 0;
  if (has_partial) {
    if (partial_block_mask_indices.scalar_type() != torch::kInt32)
      throw std::runtime_error(
          "Tensor dtype mismatch: partial_block_mask_indices must be torch.int32");
    if (!packed && partial_block_masks.scalar_type() != torch::kBool)
      throw std::runtime_error("Tensor dtype mismatch: partial_block_masks must be torch.bool");
    if (packed && partial_block_masks.scalar_type() != torch::kInt32)
      throw std::runtime_error("Tensor dtype mismatch: packed partial tiles must be torch.int32");
    if (!partial_block_mask_indices.is_contiguous() || !partial_block_masks.is_contiguous())
      throw std::runtime_error("Partial block mask tensors must be contiguous.");
    if (partial_block_mask_indices.sizes() != kv_indices.sizes())
      throw std::runtime_error("partial_block_mask_indices must have the shape of kv_indices");
    if (partial_block_masks.dim() != 3 || partial_block_masks.size(1) != Q_BLOCK_SIZE ||
        partial_block_masks.size(2) != (packed ? KV_BLOCK_SIZE / 32 : KV_BLOCK_SIZE))
      throw std::runtime_error(
          packed ? "packed partial tiles must be [num_partial, Q_BLOCK_SIZE, KV_BLOCK_SIZE / 32]"
                 : "partial_block_masks must be [num_partial, Q_BLOCK_SIZE, KV_BLOCK_SIZE]");
    if (partial_block_mask_indices.device() != Q.device() ||
        partial_block_masks.device() != Q.device())
      throw std::runtime_error("Partial block mask tensors must be on the device of Q");
    if (partial_block_masks.size(0) > 0) {
      pidx = partial_block_mask_indices.data_ptr<int32_t>();
      pmask = static_cast<const uint8_t*>(partial_block_masks.data_ptr());
      num_partial = int(partial_block_masks.size(0));
    }
  }

  c10::DeviceGuard guard(Q.device());
  hipStream_t stream = c10::hip::getCurrentHIPStream(Q.device().index()).stream();
  const int dtype = Q.scalar_type() == torch::kBFloat16 ? OMNI_ATTN_DTYPE_BF16 : OMNI_ATTN_DTYPE_F16;
  // The scalar entry point of the reference takes any block size and any head_dim <= 256
  // (omni-attn-mma/mma/attn_naive.cu:189-190, :305-408): shapes without an MFMA instance go to
  // the generic kernel when the caller is that entry point.
  const bool has_instance = (D == 32 || D == 64 || D == 128) && (Q_BLOCK_SIZE == 64 || Q_BLOCK_SIZE == 128) &&
                            (KV_BLOCK_SIZE == 64 || KV_BLOCK_SIZE == 128);
  const int rc =
      (generic_fallback && !has_instance && !packed)
          ? omni_attn_fwd_generic_gfx950(
                Q.data_ptr(), K.data_ptr(), V.data_ptr(), O.data_ptr(), lse,
                kv_num_blocks.data_ptr<int32_t>(), kv_indices.data_ptr<int32_t>(),
                block_mask_types.data_ptr<int32_t>(), pidx, pmask, int(B), int(H), int(S), int(D),
                int(num_q_blocks), int(max_blocks), Q_BLOCK_SIZE, KV_BLOCK_SIZE, num_partial, seqlen_orig,
                dtype, float(softcap), static_cast<void*>(stream))
      : packed ? omni_attn_fwd_packed_gfx950(
                   Q.data_ptr(), K.data_ptr(), V.data_ptr(), O.data_ptr(), lse,
                   kv_num_blocks.data_ptr<int32_t>(), kv_indices.data_ptr<int32_t>(),
                   block_mask_types.data_ptr<int32_t>(), pidx, reinterpret_cast<const uint32_t*>(pmask),
                   int(B), int(H), int(S), int(D), int(num_q_blocks), int(max_blocks), Q_BLOCK_SIZE,
                   KV_BLOCK_SIZE, num_partial, seqlen_orig, dtype, float(softcap), static_cast<void*>(stream))
             : omni_attn_fwd_gfx950(
                   Q.data_ptr(), K.data_ptr(), V.data_ptr(), O.data_ptr(), lse,
                   kv_num_blocks.data_ptr<int32_t>(), kv_indices.data_ptr<int32_t>(),
                   block_mask_types.data_ptr<int32_t>(), pidx, pmask, int(B), int(H), int(S), int(D),
                   int(num_q_blocks), int(max_blocks), Q_BLOCK_SIZE, KV_BLOCK_SIZE, num_partial,
                   seqlen_orig, dtype, float(softcap), static_cast<void*>(stream));
  if (rc != OMNI_ATTN_OK) {
    std::string msg = std::string("omni_attn: ") + omni_attn_status_string(rc);
    if (rc == OMNI_ATTN_ERR_UNSUPPORTED_HEAD_DIM) msg += ", got head_dim=" + std::to_string(D);
    if (rc == OMNI_ATTN_ERR_UNSUPPORTED_BLOCK)
      msg += ", got Q_BLOCK_SIZE=" + std::to_string(Q_BLOCK_SIZE) +
             " KV_BLOCK_SIZE=" + std::to_string(KV_BLOCK_SIZE);
    if (rc == OMNI_ATTN_ERR_LAUNCH)
      msg += " (hipError " + std::to_string(omni_attn_last_hip_error()) + ")";
    throw std::runtime_error(msg);
  }
}

// The reference's signature: tensors by value, void return.
void omni_attn_op(torch::Tensor Q, torch::Tensor K, torch::Tensor V, torch::Tensor O,
                  torch::Tensor kv_num_blocks, torch::Tensor kv_indices,
                  torch::Tensor block_mask_types, int Q_BLOCK_SIZE, int KV_BLOCK_SIZE,
                  int seqlen_orig, torch::Tensor partial_block_mask_indices,
                  torch::Tensor partial_block_masks, bool has_partial) {
  forward_impl(Q, K, V, O, nullptr, kv_num_blocks, kv_indices, block_mask_types, Q_BLOCK_SIZE,
               KV_BLOCK_SIZE, seqlen_orig, partial_block_mask_indices, partial_block_masks,
               has_partial);
}

// omni_attn_simple_kernel: as above, and like the reference's scalar kernel for any Q_BLOCK_SIZE,
// KV_BLOCK_SIZE and head_dim <= 256.
void omni_attn_simple_op(torch::Tensor Q, torch::Tensor K, torch::Tensor V, torch::Tensor O,
                         torch::Tensor kv_num_blocks, torch::Tensor kv_indices,
                         torch::Tensor block_mask_types, int Q_BLOCK_SIZE, int KV_BLOCK_SIZE,
                         int seqlen_orig, torch::Tensor partial_block_mask_indices,
                         torch::Tensor partial_block_masks, bool has_partial) {
  forward_impl(Q, K, V, O, nullptr, kv_num_blocks, kv_indices, block_mask_types, Q_BLOCK_SIZE,
               KV_BLOCK_SIZE, seqlen_orig, partial_block_mask_indices, partial_block_masks,
               has_partial, false, 0.0, true);
}

// Same arguments plus LSE [B, H, S] fp32, written in place.
void omni_attn_forward(torch::Tensor Q, torch::Tensor K, torch::Tensor V, torch::Tensor O,
                       torch::Tensor LSE, torch::Tensor kv_num_blocks, torch::Tensor kv_indices,
                       torch::Tensor block_mask_types, int Q_BLOCK_SIZE, int KV_BLOCK_SIZE,
                       int seqlen_orig, torch::Tensor partial_block_mask_indices,
                       torch::Tensor partial_block_masks, bool has_partial, double softcap) {
  if (LSE.scalar_type() != torch::kFloat32)
    throw std::runtime_error("Tensor dtype mismatch: LSE must be torch.float32");
  if (!LSE.is_contiguous() || LSE.dim() != 3 || Q.dim() != 4 || LSE.size(0) != Q.size(0) ||
      LSE.size(1) != Q.size(1) || LSE.size(2) != Q.size(2) || LSE.device() != Q.device())
    throw std::runtime_error("LSE must be a contiguous [B, H, S] tensor on the device of Q");
  forward_impl(Q, K, V, O, LSE.data_ptr<float>(), kv_num_blocks, kv_indices, block_mask_types,
               Q_BLOCK_SIZE, KV_BLOCK_SIZE, seqlen_orig, partial_block_mask_indices,
               partial_block_masks, has_partial, false, softcap);
}

// PARTIAL tiles [P, QB, KB] bool -> [P, QB, KB / 32] int32 words, packed on the GPU.
torch::Tensor omni_attn_pack_partial_masks(torch::Tensor partial_block_masks) {
  if (!partial_block_masks.is_cuda() || partial_block_masks.scalar_type() != torch::kBool ||
      partial_block_masks.dim() != 3 || !partial_block_masks.is_contiguous())
    throw std::runtime_error("partial_block_masks must be a contiguous [P, Q_BLOCK_SIZE, KV_BLOCK_SIZE] bool GPU tensor");
  const int64_t P = partial_block_masks.size(0), QB = partial_block_masks.size(1), KB = partial_block_masks.size(2);
  if (KB % 32 != 0) throw std::runtime_error("KV_BLOCK_SIZE must be a multiple of 32");
  c10::DeviceGuard guard(partial_block_masks.device());
  torch::Tensor out = torch::empty({P, QB, KB / 32}, partial_block_masks.options().dtype(torch::kInt32));
  hipStream_t stream = c10::hip::getCurrentHIPStream(partial_block_masks.device().index()).stream();
  const int rc = omni_attn_pack_partial_masks_gfx950(
      static_cast<const uint8_t*>(partial_block_masks.data_ptr()),
      reinterpret_cast<uint32_t*>(out.data_ptr<int32_t>()), int(P), int(QB), int(KB), static_cast<void*>(stream));
  if (rc != OMNI_ATTN_OK) throw std::runtime_error(std::string("omni_attn: ") + omni_attn_status_string(rc));
  return out;
}

// omni_attn_forward with packed PARTIAL tiles; LSE may be an empty tensor (no logsumexp).
void omni_attn_forward_packed(torch::Tensor Q, torch::Tensor K, torch::Tensor V, torch::Tensor O,
                              torch::Tensor LSE, torch::Tensor kv_num_blocks, torch::Tensor kv_indices,
                              torch::Tensor block_mask_types, int Q_BLOCK_SIZE, int KV_BLOCK_SIZE,
                              int seqlen_orig, torch::Tensor partial_block_mask_indices,
                              torch::Tensor partial_block_bits, double softcap) {
  float* lse = nullptr;
  if (LSE.numel() > 0) {
    if (LSE.scalar_type() != torch::kFloat32)
      throw std::runtime_error("Tensor dtype mismatch: LSE must be torch.float32");
    if (!LSE.is_contiguous() || LSE.dim() != 3 || Q.dim() != 4 || LSE.size(0) != Q.size(0) ||
        LSE.size(1) != Q.size(1) || LSE.size(2) != Q.size(2) || LSE.device() != Q.device())
      throw std::runtime_error("LSE must be a contiguous [B, H, S] tensor on the device of Q");
    lse = LSE.data_ptr<float>();
  }
  forward_impl(Q, K, V, O, lse, kv_num_blocks, kv_indices, block_mask_types, Q_BLOCK_SIZE, KV_BLOCK_SIZE,
               seqlen_orig, partial_block_mask_indices, partial_block_bits, true, true, softcap);
}

// Backward of omni_attn_forward: dQ, dK, dV written in place (the reference exports no backward).
// PARTIAL tiles as bool bytes or, when `packed`, as the int32 words of omni_attn_pack_partial_masks.
void omni_attn_backward(torch::Tensor Q, torch::Tensor K, torch::Tensor V, torch::Tensor O,
                        torch::Tensor dO, torch::Tensor LSE, torch::Tensor dQ, torch::Tensor dK,
                        torch::Tensor dV, torch::Tensor kv_num_blocks, torch::Tensor kv_indices,
                        torch::Tensor block_mask_types, int Q_BLOCK_SIZE, int KV_BLOCK_SIZE,
                        int seqlen_orig, torch::Tensor partial_block_mask_indices,
                        torch::Tensor partial_tiles, bool has_partial, bool packed, double softcap) {
  if (Q.scalar_type() != torch::kHalf && Q.scalar_type() != torch::kBFloat16)
    throw std::runtime_error("Tensor dtype mismatch: Q must be torch.float16 or torch.bfloat16");
  check_qkvo(Q, "Q", Q);
  check_qkvo(K, "K", Q);
  check_qkvo(V, "V", Q);
  check_qkvo(O, "O", Q);
  check_qkvo(dO, "dO", Q);
  check_qkvo(dQ, "dQ", Q);
  check_qkvo(dK, "dK", Q);
  check_qkvo(dV, "dV", Q);
  for (const torch::Tensor* t : {&Q, &K, &V, &O, &dO, &dQ, &dK, &dV})
    if (!t->is_contiguous())
      throw std::runtime_error("Q, K, V, O, dO, dQ, dK, dV tensors must be contiguous.");
  check_meta(kv_num_blocks, "kv_num_blocks", Q);
  check_meta(kv_indices, "kv_indices", Q);
  check_meta(block_mask_types, "block_mask_types", Q);
  if (!kv_num_blocks.is_contiguous() || !kv_indices.is_contiguous() || !block_mask_types.is_contiguous())
    throw std::runtime_error("Block mask tensors must be contiguous.");
  const int64_t B = Q.size(0), H = Q.size(1), S = Q.size(2), D = Q.size(3);
  if (kv_num_blocks.dim() != 3 || kv_indices.dim() != 4 || block_mask_types.sizes() != kv_indices.sizes() ||
      kv_num_blocks.size(0) != B || kv_num_blocks.size(1) != H || kv_indices.size(0) != B ||
      kv_indices.size(1) != H || kv_indices.size(2) != kv_num_blocks.size(2))
    throw std::runtime_error("Block mask tensor shapes do not match Q's batch / heads / blocks");
  if (LSE.scalar_type() != torch::kFloat32 || !LSE.is_contiguous() || LSE.dim() != 3 || LSE.size(0) != B ||
      LSE.size(1) != H || LSE.size(2) != S || LSE.device() != Q.device())
    throw std::runtime_error("LSE must be the forward's contiguous fp32 [B, H, S] tensor on the device of Q");
  const int32_t* pidx = nullptr;
  const void* tiles = nullptr;
  int num_partial = 0;
  if (has_partial && partial_tiles.numel() > 0) {
    if (partial_block_mask_indices.scalar_type() != torch::kInt32 ||
        partial_block_mask_indices.sizes() != kv_indices.sizes() || !partial_block_mask_indices.is_contiguous() ||
        partial_block_mask_indices.device() != Q.device())
      throw std::runtime_error("partial_block_mask_indices must be a contiguous int32 tensor of the shape of kv_indices");
    if (partial_tiles.scalar_type() != (packed ? torch::kInt32 : torch::kBool) || partial_tiles.dim() != 3 ||
        partial_tiles.size(1) != Q_BLOCK_SIZE || partial_tiles.size(2) != (packed ? KV_BLOCK_SIZE / 32 : KV_BLOCK_SIZE) ||
        !partial_tiles.is_contiguous() || partial_tiles.device() != Q.device())
      throw std::runtime_error("partial tiles must be [num_partial, Q_BLOCK_SIZE, KV_BLOCK_SIZE] bool or packed int32 words");
    pidx = partial_block_mask_indices.data_ptr<int32_t>();
    tiles = partial_tiles.data_ptr();
    num_partial = int(partial_tiles.size(0));
  }
  c10::DeviceGuard guard(Q.device());
  hipStream_t stream = c10::hip::getCurrentHIPStream(Q.device().index()).stream();
  const size_t ws_bytes = omni_attn_bwd_workspace_bytes(int(B), int(H), int(S));
  torch::Tensor workspace = torch::empty({int64_t(ws_bytes)}, Q.options().dtype(torch::kUInt8));
  const int dtype = Q.scalar_type() == torch::kBFloat16 ? OMNI_ATTN_DTYPE_BF16 : OMNI_ATTN_DTYPE_F16;
  const int rc = omni_attn_bwd_gfx950(
      Q.data_ptr(), K.data_ptr(), V.data_ptr(), O.data_ptr(), dO.data_ptr(), LSE.data_ptr<float>(),
      dQ.data_ptr(), dK.data_ptr(), dV.data_ptr(), kv_num_blocks.data_ptr<int32_t>(),
      kv_indices.data_ptr<int32_t>(), block_mask_types.data_ptr<int32_t>(), pidx,
      packed ? nullptr : static_cast<const uint8_t*>(tiles), packed ? static_cast<const uint32_t*>(tiles) : nullptr,
      workspace.data_ptr(), ws_bytes, int(B), int(H), int(S), int(D), int(kv_num_blocks.size(2)),
      int(kv_indices.size(3)), Q_BLOCK_SIZE, KV_BLOCK_SIZE, num_partial, seqlen_orig, dtype, float(softcap),
      static_cast<void*>(stream));
  if (rc != OMNI_ATTN_OK) {
    std::string msg = std::string("omni_attn: ") + omni_attn_status_string(rc);
    if (rc == OMNI_ATTN_ERR_LAUNCH) msg += " (hipError " + std::to_string(omni_attn_last_hip_error()) + ")";
    throw std::runtime_error(msg);
  }
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "gfx950 block-sparse FlashAttention-2 forward (omni-attention operator surface)";
  m.def("omni_attn_mma_stages_split_q_shared_kv", &omni_attn_op,
        "omni_attn_mma_stages_split_q_shared_kv");
  m.def("omni_attn_simple_kernel", &omni_attn_simple_op, "omni_attn_simple_kernel");
  m.def("omni_attn_cp_async", &omni_attn_op, "omni_attn_cp_async");
  m.def("omni_attn_preftech_kernel", &omni_attn_op, "omni_attn_preftech_kernel");
  m.def("omni_attn_preftech", &omni_attn_op, "omni_attn_preftech");
  m.def("omni_attn_mma_stages_split_q_shared_kv_swizzle", &omni_attn_op,
        "omni_attn_mma_stages_split_q_shared_kv_swizzle");
  namespace py = pybind11;
  m.def("omni_attn_forward", &omni_attn_forward, "omni_attn_forward (also writes logsumexp)", py::arg("Q"),
        py::arg("K"), py::arg("V"), py::arg("O"), py::arg("LSE"), py::arg("kv_num_blocks"), py::arg("kv_indices"),
        py::arg("block_mask_types"), py::arg("Q_BLOCK_SIZE"), py::arg("KV_BLOCK_SIZE"), py::arg("seqlen_orig"),
        py::arg("partial_block_mask_indices"), py::arg("partial_block_masks"), py::arg("has_partial"),
        py::arg("softcap") = 0.0);
  m.def("omni_attn_pack_partial_masks", &omni_attn_pack_partial_masks,
        "omni_attn_pack_partial_masks (bool tiles -> 32-bit words)");
  m.def("omni_attn_forward_packed", &omni_attn_forward_packed,
        "omni_attn_forward_packed (PARTIAL tiles as packed words)", py::arg("Q"), py::arg("K"), py::arg("V"),
        py::arg("O"), py::arg("LSE"), py::arg("kv_num_blocks"), py::arg("kv_indices"), py::arg("block_mask_types"),
        py::arg("Q_BLOCK_SIZE"), py::arg("KV_BLOCK_SIZE"), py::arg("seqlen_orig"),
        py::arg("partial_block_mask_indices"), py::arg("partial_block_bits"), py::arg("softcap") = 0.0);
  m.def("omni_attn_backward", &omni_attn_backward, "omni_attn_backward (dQ, dK, dV of omni_attn_forward)",
        py::arg("Q"), py::arg("K"), py::arg("V"), py::arg("O"), py::arg("dO"), py::arg("LSE"), py::arg("dQ"),
        py::arg("dK"), py::arg("dV"), py::arg("kv_num_blocks"), py::arg("kv_indices"), py::arg("block_mask_types"),
        py::arg("Q_BLOCK_SIZE"), py::arg("KV_BLOCK_SIZE"), py::arg("seqlen_orig"),
        py::arg("partial_block_mask_indices"), py::arg("partial_tiles"), py::arg("has_partial"), py::arg("packed"),
        py::arg("softcap") = 0.0);
  m.def("abi_version", []() { return omni_attn_abi_version(); });
}
