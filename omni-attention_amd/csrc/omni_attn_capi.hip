// C ABI of the forward: argument validation, instance dispatch, error codes.
// Mirrors what the reference's launchers check before they launch
// (omni-attn-mma/mma/attn_naive.cu:312-356, omni-attn-mma/mma/omni_attn_shared_kv.cu:701-768)
// minus everything that is a property of torch tensors (dtype objects, contiguity),
// which the binding layer above this file checks.
#include "../../include/omni_attn_gfx950.h"
#include "omni_attn_bwd_kernel.hpp"

#include <atomic>
#include <cmath>
#include <cstdint>

namespace omni_attn {
template <bool BF16, int D>
int launch_fwd_blocks(const FwdParams& p, int QB, int KB, hipStream_t stream);
template <> int launch_fwd_blocks<false, 32>(const FwdParams&, int, int, hipStream_t);
template <> int launch_fwd_blocks<false, 64>(const FwdParams&, int, int, hipStream_t);
template <> int launch_fwd_blocks<false, 128>(const FwdParams&, int, int, hipStream_t);
template <> int launch_fwd_blocks<true, 32>(const FwdParams&, int, int, hipStream_t);
template <> int launch_fwd_blocks<true, 64>(const FwdParams&, int, int, hipStream_t);
template <> int launch_fwd_blocks<true, 128>(const FwdParams&, int, int, hipStream_t);
template <bool BF16, int D>
int launch_bwd_blocks(const BwdParams& p, int QB, int KB, hipStream_t stream);
template <> int launch_bwd_blocks<false, 32>(const BwdParams&, int, int, hipStream_t);
template <> int launch_bwd_blocks<false, 64>(const BwdParams&, int, int, hipStream_t);
template <> int launch_bwd_blocks<false, 128>(const BwdParams&, int, int, hipStream_t);
template <> int launch_bwd_blocks<true, 32>(const BwdParams&, int, int, hipStream_t);
template <> int launch_bwd_blocks<true, 64>(const BwdParams&, int, int, hipStream_t);
template <> int launch_bwd_blocks<true, 128>(const BwdParams&, int, int, hipStream_t);
}  // namespace omni_attn

namespace {
thread_local int g_last_hip_error = 0;
}  // namespace
void omni_attn::record_hip_error(int hip_error) { g_last_hip_error = hip_error; }
namespace {

// What the work order needs to know about the device, queried once per device: the number
// of XCDs (each has its own L2; workgroup ids are dealt round-robin over them), the compute
// units per XCD and the size of one L2.  A partitioned device (CPX: one XCD per device)
// reports 1 XCD and its own CU count.
struct DeviceTopology {
  int n_xcd;
  int cus_per_xcd;
  long long l2_bytes;
};
constexpr int kMaxDevices = 64;
DeviceTopology g_topology[kMaxDevices];
std::atomic<bool> g_topology_known[kMaxDevices];

int query_topology(DeviceTopology* out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return int(e);
  const bool cached = dev >= 0 && dev < kMaxDevices;
  if (cached && g_topology_known[dev].load(std::memory_order_acquire)) {
    *out = g_topology[dev];
    return 0;
  }
  int xcc = 0, cus = 0, l2 = 0;
  if (hipDeviceGetAttribute(&xcc, hipDeviceAttributeNumberOfXccs, dev) != hipSuccess || xcc <= 0) xcc = 1;
  e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess) return int(e);
  if (hipDeviceGetAttribute(&l2, hipDeviceAttributeL2CacheSize, dev) != hipSuccess || l2 <= 0) l2 = 4 << 20;
  DeviceTopology t;
  t.n_xcd = xcc;
  t.cus_per_xcd = cus / xcc > 0 ? cus / xcc : 1;
  t.l2_bytes = l2;
  if (cached) {
    g_topology[dev] = t;
    g_topology_known[dev].store(true, std::memory_order_release);
  }
  *out = t;
  return 0;
}
}  // namespace

namespace {
// Both forward entry points: PARTIAL tiles as bytes (partial_masks) or packed (partial_bits).
int forward(const void* q, const void* k, const void* v, void* o, float* lse_or_null,
            const int32_t* kv_num_blocks, const int32_t* kv_indices, const int32_t* block_mask_types,
            const int32_t* partial_idx_or_null, const uint8_t* partial_masks_or_null,
            const uint32_t* partial_bits_or_null, int B, int H, int S_pad, int D, int Tq,
            int max_blocks, int QB, int KB, int num_partial, int seqlen_orig, int dtype, float softcap,
            void* stream) {
  using namespace omni_attn;
  if (!q || !k || !v || !o || !kv_num_blocks || !kv_indices || !block_mask_types)
    return OMNI_ATTN_ERR_NULL_POINTER;
  // 16-byte loads and stores on q, k, v, o and the mask tiles; 4-byte ones on the rest
  const auto misaligned = [](const void* ptr, uintptr_t a) { return (reinterpret_cast<uintptr_t>(ptr) & (a - 1)) != 0; };
  if (misaligned(q, 16) || misaligned(k, 16) || misaligned(v, 16) || misaligned(o, 16) ||
      misaligned(partial_masks_or_null, 16) || misaligned(partial_bits_or_null, 4) ||
      misaligned(lse_or_null, 4) || misaligned(kv_num_blocks, 4) ||
      misaligned(kv_indices, 4) || misaligned(block_mask_types, 4) || misaligned(partial_idx_or_null, 4))
    return OMNI_ATTN_ERR_MISALIGNED;
  if (dtype != OMNI_ATTN_DTYPE_F16 && dtype != OMNI_ATTN_DTYPE_BF16)
    return OMNI_ATTN_ERR_UNSUPPORTED_DTYPE;
  if (D != 32 && D != 64 && D != 128) return OMNI_ATTN_ERR_UNSUPPORTED_HEAD_DIM;
  if ((QB != 64 && QB != 128) || (KB != 64 && KB != 128)) return OMNI_ATTN_ERR_UNSUPPORTED_BLOCK;
  if (B <= 0 || H <= 0 || S_pad <= 0 || Tq <= 0 || max_blocks <= 0 || seqlen_orig < 0 || num_partial < 0)
    return OMNI_ATTN_ERR_BAD_SHAPE;
  if (!(softcap >= 0.f) || std::isinf(softcap)) return OMNI_ATTN_ERR_BAD_SHAPE;  // also refuses NaN
  if (Tq != (S_pad + QB - 1) / QB) return OMNI_ATTN_ERR_BAD_SHAPE;
  const long long total = (long long)B * H * Tq;
  if ((long long)S_pad * D > 0x7fffffffLL || total > 0x7fffffffLL / 2 ||
      total * max_blocks > (1LL << 40))
    return OMNI_ATTN_ERR_TOO_LARGE;

  FwdParams p;
  p.q = static_cast<const uint16_t*>(q);
  p.k = static_cast<const uint16_t*>(k);
  p.v = static_cast<const uint16_t*>(v);
  p.o = static_cast<uint16_t*>(o);
  p.lse = lse_or_null;
  p.kv_num_blocks = kv_num_blocks;
  p.kv_indices = kv_indices;
  p.types = block_mask_types;
  if ((long long)num_partial * QB * KB > 0x7fffffffLL * 64) return OMNI_ATTN_ERR_TOO_LARGE;
  const bool has_partial = partial_idx_or_null != nullptr && num_partial > 0 &&
                           (partial_masks_or_null != nullptr || partial_bits_or_null != nullptr);
  p.partial_idx = has_partial ? partial_idx_or_null : nullptr;
  p.partial_masks = has_partial ? partial_masks_or_null : nullptr;
  p.partial_bits = has_partial ? partial_bits_or_null : nullptr;
  p.num_partial = has_partial ? num_partial : 0;
  p.S = S_pad;
  p.Tq = Tq;
  p.Tk = (S_pad + KB - 1) / KB;
  p.max_blocks = max_blocks;
  p.seqlen = seqlen_orig < S_pad ? seqlen_orig : S_pad;
  p.n_slabs = B * H;
  DeviceTopology topo;
  if (const int e = query_topology(&topo)) {
    g_last_hip_error = e;
    return OMNI_ATTN_ERR_LAUNCH;
  }
  p.n_xcd = topo.n_xcd;
  const int X = topo.n_xcd;
  // Slabs of one XCD that are walked together, longest query block first.  A CU holds two
  // workgroups of this kernel (a Q_BLOCK 64 workgroup is half the size, four fit): at
  // least enough slabs to fill the XCD's slots.  Beyond that, the heads of
  // one batch element that land on the XCD (heads of a batch element share their mask in
  // practice, so "query block index" orders their workgroups by length across heads and the
  // tail of one head is filled by the others; mixing batch elements with different masks in
  // one group measured 8 % slower, a group of one head 2-4 % slower) -- but no more heads
  // than have their K and V in the XCD's L2 (4 MiB on MI355X) together, when at least two
  // do: a bigger group was 2 % faster still on 4096-token slabs and doubled the L2 misses.
  const int slots_per_xcd = topo.cus_per_xcd * (QB == 128 ? 2 : 4);
  const int fill = slots_per_xcd / Tq > 1 ? slots_per_xcd / Tq : 1;
  int heads = (H % X == 0) ? H / X : 1;
  const long long slab_kv_bytes = 4LL * S_pad * D;  // K and V, 16-bit
  const long long fit = topo.l2_bytes / slab_kv_bytes;
  if (fit >= 2 && fit < heads) {
    heads = int(fit);
    while ((H / X) % heads != 0) --heads;  // whole batch elements per group sequence
  }
  p.slab_group = heads * ((fill + heads - 1) / heads);
  p.softcap = softcap;
  p.cap_c2 = softcap > 0.f ? float(2.0 * 1.4426950408889634 / (std::sqrt(double(D)) * double(softcap))) : 0.f;
  p.sl2 = softcap > 0.f ? float(1.4426950408889634) : float(1.4426950408889634 / std::sqrt(double(D)));

  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool bf = dtype == OMNI_ATTN_DTYPE_BF16;
  int err;
  switch (D) {
    case 32: err = bf ? launch_fwd_blocks<true, 32>(p, QB, KB, s) : launch_fwd_blocks<false, 32>(p, QB, KB, s); break;
    case 64: err = bf ? launch_fwd_blocks<true, 64>(p, QB, KB, s) : launch_fwd_blocks<false, 64>(p, QB, KB, s); break;
    default: err = bf ? launch_fwd_blocks<true, 128>(p, QB, KB, s) : launch_fwd_blocks<false, 128>(p, QB, KB, s); break;
  }
  if (err != 0) {
    g_last_hip_error = err;
    return OMNI_ATTN_ERR_LAUNCH;
  }
  return OMNI_ATTN_OK;
}
}  // namespace

extern "C" int omni_attn_fwd_gfx950(const void* q, const void* k, const void* v, void* o,
                                    float* lse_or_null, const int32_t* kv_num_blocks,
                                    const int32_t* kv_indices, const int32_t* block_mask_types,
                                    const int32_t* partial_idx_or_null,
                                    const uint8_t* partial_masks_or_null, int B, int H, int S_pad,
                                    int D, int Tq, int max_blocks, int QB, int KB, int num_partial,
                                    int seqlen_orig, int dtype, float softcap, void* stream) {
  return forward(q, k, v, o, lse_or_null, kv_num_blocks, kv_indices, block_mask_types, partial_idx_or_null,
                 partial_masks_or_null, nullptr, B, H, S_pad, D, Tq, max_blocks, QB, KB, num_partial,
                 seqlen_orig, dtype, softcap, stream);
}

extern "C" int omni_attn_fwd_packed_gfx950(const void* q, const void* k, const void* v, void* o,
                                           float* lse_or_null, const int32_t* kv_num_blocks,
                                           const int32_t* kv_indices, const int32_t* block_mask_types,
                                           const int32_t* partial_idx_or_null,
                                           const uint32_t* partial_bits_or_null, int B, int H, int S_pad,
                                           int D, int Tq, int max_blocks, int QB, int KB, int num_partial,
                                           int seqlen_orig, int dtype, float softcap, void* stream) {
  return forward(q, k, v, o, lse_or_null, kv_num_blocks, kv_indices, block_mask_types, partial_idx_or_null,
                 nullptr, partial_bits_or_null, B, H, S_pad, D, Tq, max_blocks, QB, KB, num_partial,
                 seqlen_orig, dtype, softcap, stream);
}

extern "C" size_t omni_attn_bwd_workspace_bytes(int B, int H, int S_pad) {
  if (B <= 0 || H <= 0 || S_pad <= 0) return 0;
  // two floats per row: -rowsum(dO . O) and the row's exponent offset
  return size_t(B) * size_t(H) * size_t(S_pad) * 2 * sizeof(float);
}

namespace {
// The backward with the workspace already chosen (caller's, or the library's static one).
int backward(const void* q, const void* k, const void* v, const void* o, const void* dout,
             const float* lse, void* dq, void* dk, void* dv, const int32_t* kv_num_blocks,
             const int32_t* kv_indices, const int32_t* block_mask_types,
             const int32_t* partial_idx_or_null, const uint8_t* partial_masks_or_null,
             const uint32_t* partial_bits_or_null, float* delta_workspace, int B, int H, int S_pad,
             int D, int Tq, int max_blocks, int QB, int KB, int num_partial, int seqlen_orig, int dtype,
             float softcap, void* stream) {
  using namespace omni_attn;
  if (!(softcap >= 0.f) || std::isinf(softcap)) return OMNI_ATTN_ERR_BAD_SHAPE;
  if (!q || !k || !v || !o || !dout || !lse || !dq || !dk || !dv || !kv_num_blocks || !kv_indices ||
      !block_mask_types || !delta_workspace)
    return OMNI_ATTN_ERR_NULL_POINTER;
  const auto misaligned = [](const void* ptr, uintptr_t a) { return (reinterpret_cast<uintptr_t>(ptr) & (a - 1)) != 0; };
  if (misaligned(q, 16) || misaligned(k, 16) || misaligned(v, 16) || misaligned(o, 16) || misaligned(dout, 16) ||
      misaligned(dq, 16) || misaligned(dk, 16) || misaligned(dv, 16) || misaligned(partial_masks_or_null, 16) ||
      misaligned(partial_bits_or_null, 4) || misaligned(lse, 4) || misaligned(delta_workspace, 4) ||
      misaligned(kv_num_blocks, 4) || misaligned(kv_indices, 4) || misaligned(block_mask_types, 4) ||
      misaligned(partial_idx_or_null, 4))
    return OMNI_ATTN_ERR_MISALIGNED;
  if (dtype != OMNI_ATTN_DTYPE_F16 && dtype != OMNI_ATTN_DTYPE_BF16) return OMNI_ATTN_ERR_UNSUPPORTED_DTYPE;
  if (D != 32 && D != 64 && D != 128) return OMNI_ATTN_ERR_UNSUPPORTED_HEAD_DIM;
  if ((QB != 64 && QB != 128) || (KB != 64 && KB != 128)) return OMNI_ATTN_ERR_UNSUPPORTED_BLOCK;
  if (B <= 0 || H <= 0 || S_pad <= 0 || Tq <= 0 || max_blocks <= 0 || seqlen_orig < 0 || num_partial < 0)
    return OMNI_ATTN_ERR_BAD_SHAPE;
  if (Tq != (S_pad + QB - 1) / QB) return OMNI_ATTN_ERR_BAD_SHAPE;
  const long long total = (long long)B * H * Tq;
  const int Tk = (S_pad + KB - 1) / KB;
  if ((long long)S_pad * D > 0x7fffffffLL || total > 0x7fffffffLL / 2 || (long long)B * H * Tk > 0x7fffffffLL / 2 ||
      total * max_blocks > (1LL << 40) || (long long)num_partial * QB * KB > 0x7fffffffLL * 64)
    return OMNI_ATTN_ERR_TOO_LARGE;
  // the dK/dV kernel numbers the 64-slot words of a slab's metadata with an int
  if ((long long)Tq * ((max_blocks + 63) / 64) > 0x7fffffffLL) return OMNI_ATTN_ERR_TOO_LARGE;

  BwdParams p;
  p.q = static_cast<const uint16_t*>(q);
  p.k = static_cast<const uint16_t*>(k);
  p.v = static_cast<const uint16_t*>(v);
  p.o = static_cast<const uint16_t*>(o);
  p.dout = static_cast<const uint16_t*>(dout);
  p.lse = lse;
  p.dq = static_cast<uint16_t*>(dq);
  p.dk = static_cast<uint16_t*>(dk);
  p.dv = static_cast<uint16_t*>(dv);
  p.ws = delta_workspace;
  p.kv_num_blocks = kv_num_blocks;
  p.kv_indices = kv_indices;
  p.types = block_mask_types;
  const bool has_partial = partial_idx_or_null != nullptr && num_partial > 0 &&
                           (partial_masks_or_null != nullptr || partial_bits_or_null != nullptr);
  p.partial_idx = has_partial ? partial_idx_or_null : nullptr;
  p.partial_masks = has_partial && partial_bits_or_null == nullptr ? partial_masks_or_null : nullptr;
  p.partial_bits = has_partial ? partial_bits_or_null : nullptr;
  p.num_partial = has_partial ? num_partial : 0;
  p.S = S_pad;
  p.Tq = Tq;
  p.Tk = Tk;
  p.max_blocks = max_blocks;
  p.seqlen = seqlen_orig < S_pad ? seqlen_orig : S_pad;
  p.n_slabs = B * H;
  DeviceTopology topo;
  if (const int e = query_topology(&topo)) {
    g_last_hip_error = e;
    return OMNI_ATTN_ERR_LAUNCH;
  }
  p.n_xcd = topo.n_xcd;
  p.scale = float(1.0 / std::sqrt(double(D)));
  p.sl2 = float(1.4426950408889634 / std::sqrt(double(D)));
  p.softcap = softcap;
  p.cap_c2 = softcap > 0.f ? float(2.0 * 1.4426950408889634 / (std::sqrt(double(D)) * double(softcap))) : 0.f;

  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool bf = dtype == OMNI_ATTN_DTYPE_BF16;
  int err;
  switch (D) {
    case 32: err = bf ? launch_bwd_blocks<true, 32>(p, QB, KB, s) : launch_bwd_blocks<false, 32>(p, QB, KB, s); break;
    case 64: err = bf ? launch_bwd_blocks<true, 64>(p, QB, KB, s) : launch_bwd_blocks<false, 64>(p, QB, KB, s); break;
    default: err = bf ? launch_bwd_blocks<true, 128>(p, QB, KB, s) : launch_bwd_blocks<false, 128>(p, QB, KB, s); break;
  }
  if (err != 0) {
    g_last_hip_error = err;
    return OMNI_ATTN_ERR_LAUNCH;
  }
  return OMNI_ATTN_OK;
}
}  // namespace

extern "C" int omni_attn_bwd_gfx950(const void* q, const void* k, const void* v, const void* o,
                                    const void* dout, const float* lse, void* dq, void* dk, void* dv,
                                    const int32_t* kv_num_blocks, const int32_t* kv_indices,
                                    const int32_t* block_mask_types, const int32_t* partial_idx_or_null,
                                    const uint8_t* partial_masks_or_null,
                                    const uint32_t* partial_bits_or_null, void* workspace,
                                    size_t workspace_bytes, int B, int H, int S_pad, int D, int Tq,
                                    int max_blocks, int QB, int KB, int num_partial, int seqlen_orig,
                                    int dtype, float softcap, void* stream) {
  if (B > 0 && H > 0 && S_pad > 0 && workspace_bytes < omni_attn_bwd_workspace_bytes(B, H, S_pad))
    return OMNI_ATTN_ERR_WORKSPACE;
  return backward(q, k, v, o, dout, lse, dq, dk, dv, kv_num_blocks, kv_indices, block_mask_types,
                  partial_idx_or_null, partial_masks_or_null, partial_bits_or_null,
                  static_cast<float*>(workspace), B, H, S_pad, D, Tq, max_blocks, QB, KB, num_partial,
                  seqlen_orig, dtype, softcap, stream);
}

// ---- the backward for callers that cannot allocate -------------------------------------------
// Same kernels; the workspace (two floats per row) is this file-scope device array instead of
// caller memory.
// Every GPU the library runs on holds its own copy at its own address until the process ends.
constexpr size_t kScratchFloats = size_t(8) << 20;  // 32 MiB: B * H * S_pad up to 4 194 304 rows
static __device__ __align__(256) float scratch[kScratchFloats];

namespace {
float* g_scratch_ptr[kMaxDevices];
std::atomic<bool> g_scratch_known[kMaxDevices];

// Device address of `scratch` on the current device (looked up once per device: in host code the
// array's name is only a handle for this lookup, never an address a kernel can use).
int scratch_address(float** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return int(e);
  if (dev < 0 || dev >= kMaxDevices) return int(hipErrorInvalidDevice);
  if (!g_scratch_known[dev].load(std::memory_order_acquire)) {
    float* ptr = nullptr;
    e = hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch));
    if (e != hipSuccess) return int(e);
    if (ptr == nullptr) return int(hipErrorInvalidSymbol);
    g_scratch_ptr[dev] = ptr;
    g_scratch_known[dev].store(true, std::memory_order_release);
  }
  *out = g_scratch_ptr[dev];
  return 0;
}
}  // namespace

extern "C" size_t omni_attn_bwd_noalloc_max_rows(void) { return kScratchFloats / 2; }

extern "C" int omni_attn_bwd_noalloc_gfx950(const void* q, const void* k, const void* v, const void* o,
                                            const void* dout, const float* lse, void* dq, void* dk,
                                            void* dv, const int32_t* kv_num_blocks,
                                            const int32_t* kv_indices, const int32_t* block_mask_types,
                                            const int32_t* partial_idx_or_null,
                                            const uint8_t* partial_masks_or_null,
                                            const uint32_t* partial_bits_or_null, int B, int H, int S_pad,
                                            int D, int Tq, int max_blocks, int QB, int KB, int num_partial,
                                            int seqlen_orig, int dtype, float softcap, void* stream) {
  if (B <= 0 || H <= 0 || S_pad <= 0) return OMNI_ATTN_ERR_BAD_SHAPE;
  if ((unsigned long long)B * (unsigned long long)H * (unsigned long long)S_pad > kScratchFloats / 2)
    return OMNI_ATTN_ERR_SCRATCH_LIMIT;
  float* delta = nullptr;
  if (const int e = scratch_address(&delta)) {
    g_last_hip_error = e;
    return OMNI_ATTN_ERR_LAUNCH;
  }
  // Nothing in the array has to start at zero: the dQ kernel writes both floats of every row of
  // every slab before the dK/dV kernel, which runs after it on the same stream, reads any of them.
  return backward(q, k, v, o, dout, lse, dq, dk, dv, kv_num_blocks, kv_indices, block_mask_types,
                  partial_idx_or_null, partial_masks_or_null, partial_bits_or_null, delta, B, H, S_pad, D,
                  Tq, max_blocks, QB, KB, num_partial, seqlen_orig, dtype, softcap, stream);
}

extern "C" const char* omni_attn_status_string(int status) {
  switch (status) {
    case OMNI_ATTN_OK: return "ok";
    case OMNI_ATTN_ERR_NULL_POINTER: return "a required pointer is NULL";
    case OMNI_ATTN_ERR_BAD_SHAPE: return "bad shape: sizes must be positive and Tq == ceil(S_pad / Q_BLOCK_SIZE)";
    case OMNI_ATTN_ERR_UNSUPPORTED_HEAD_DIM: return "unsupported head_dim (supported: 32, 64, 128)";
    case OMNI_ATTN_ERR_UNSUPPORTED_BLOCK: return "unsupported Q_BLOCK_SIZE / KV_BLOCK_SIZE (supported: 64, 128)";
    case OMNI_ATTN_ERR_UNSUPPORTED_DTYPE: return "unsupported dtype (supported: fp16, bf16)";
    case OMNI_ATTN_ERR_LAUNCH: return "HIP kernel launch failed";
    case OMNI_ATTN_ERR_TOO_LARGE: return "tensor too large for 32-bit slab indexing";
    case OMNI_ATTN_ERR_MISALIGNED: return "misaligned pointer: q, k, v, o and partial masks need 16 bytes, 32-bit arrays 4";
    case OMNI_ATTN_ERR_WORKSPACE: return "workspace too small (see omni_attn_bwd_workspace_bytes)";
    case OMNI_ATTN_ERR_SCRATCH_LIMIT:
      return "B * H * S_pad exceeds the built-in scratch of omni_attn_bwd_noalloc_gfx950 (4 194 304 rows); "
             "use omni_attn_bwd_gfx950 with a workspace";
    default: return "unknown status";
  }
}

extern "C" int omni_attn_last_hip_error(void) { return g_last_hip_error; }

extern "C" int omni_attn_abi_version(void) { return 4; }
