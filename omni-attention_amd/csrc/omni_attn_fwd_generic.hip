// The scalar-semantics forward for shapes the MFMA kernel has no instance for.
//
// The reference's correctness kernel omni_attn_simple_kernel_impl
// (omni-attn-mma/mma/attn_naive.cu:21-302, launcher :305-408) takes any Q_BLOCK / KV_BLOCK and
// any head_dim up to 256 (`float out[256]`, :189-190); its MMA kernels take only
// {64, 128}^2 x {32, 64, 128}.  This kernel keeps that generality: same two-pass fp32 softmax
// per query row (row maximum over all listed keys first, then exp / sum / weighted V), same
// slot rules, plus the row logsumexp.  One wave per query row: in the score passes a lane owns
// a key (64 keys at a time), in the weighted-V pass a lane owns head dimensions d, d + 64, ...
// and the wave walks the 64 weights with readlane.  Not a performance path.
#include "../../include/omni_attn_gfx950.h"

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cmath>

namespace omni_attn {
// Keeps the hipError_t behind an OMNI_ATTN_ERR_LAUNCH for omni_attn_last_hip_error() (defined
// beside that function).
void record_hip_error(int hip_error);
}  // namespace omni_attn

namespace {

enum : int { kMasked = 0, kCausal = 1, kFull = 2, kPartial = 3 };

struct GenericParams {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  uint16_t* o;
  float* lse;
  const int32_t* kv_num_blocks;
  const int32_t* kv_indices;
  const int32_t* types;
  const int32_t* partial_idx;
  const uint8_t* partial_masks;
  int num_partial;
  int S, D, Tq, Tk, max_blocks, QB, KB, seqlen;
  int k_rows_16b;  // every row of K starts on a 16-byte boundary (base aligned, D a multiple of 8)
  long long rows;  // B * H * S
  float scale, softcap;
};

template <bool BF16>
__device__ __forceinline__ float to_float(uint16_t x) {
  if constexpr (BF16) {
    const uint32_t u = uint32_t(x) << 16;
    return __builtin_bit_cast(float, u);
  } else {
    return float(__builtin_bit_cast(_Float16, x));
  }
}
template <bool BF16>
__device__ __forceinline__ uint16_t from_float(float x) {
  if constexpr (BF16) {
    const __bf16 b = (__bf16)x;
    return __builtin_bit_cast(uint16_t, b);
  } else {
    const _Float16 h = (_Float16)x;
    return __builtin_bit_cast(uint16_t, h);
  }
}
__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) x = fmaxf(x, __shfl_xor(x, m, 64));
  return x;
}
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) x += __shfl_xor(x, m, 64);
  return x;
}

constexpr int kRowsPerWorkgroup = 4;
constexpr int kMaxD = 256;

template <bool BF16>
__global__ void __launch_bounds__(64 * kRowsPerWorkgroup) fwd_generic_kernel(const GenericParams p) {
  __shared__ float sq[kRowsPerWorkgroup][kMaxD];
  const int lane = threadIdx.x & 63;
  const int w = threadIdx.x >> 6;
  const long long row = (long long)blockIdx.x * kRowsPerWorkgroup + w;
  if (row >= p.rows) return;
  const long long bh = row / p.S;
  const int q_idx = int(row - bh * p.S);
  const size_t slab = size_t(bh) * size_t(p.S) * p.D;
  uint16_t* orow = p.o + slab + size_t(q_idx) * p.D;
  const int ND = (p.D + 63) / 64;  // head dimensions per lane in the weighted-V pass (<= 4)

  auto write_empty = [&]() {
    for (int d = lane; d < p.D; d += 64) orow[d] = 0;
    if (lane == 0 && p.lse) p.lse[row] = -INFINITY;
  };
  if (q_idx >= p.seqlen) {  // padding row: zeros (attn_naive.cu:64-72)
    write_empty();
    return;
  }
  int q_block = q_idx / p.QB;
  if (q_block >= p.Tq) q_block = p.Tq - 1;  // :75-78
  const size_t mrow = size_t(bh) * p.Tq + q_block;
  int nb = p.kv_num_blocks[mrow];
  nb = nb < 0 ? 0 : (nb > p.max_blocks ? p.max_blocks : nb);
  const int32_t* idx = p.kv_indices + mrow * p.max_blocks;
  const int32_t* tys = p.types + mrow * p.max_blocks;
  const bool has_partial = p.partial_idx != nullptr && p.partial_masks != nullptr;
  const int32_t* pidx = has_partial ? p.partial_idx + mrow * p.max_blocks : nullptr;

  for (int d = lane; d < p.D; d += 64) sq[w][d] = to_float<BF16>(p.q[slab + size_t(q_idx) * p.D + d]);
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the row is in LDS before the wave reads it

  // key range of slot s for this row, after the slot rules; returns false for a skipped slot
  auto slot_range = [&](int s, int& kv_start, int& kv_end, int& pid, int& mode) {
    int kvb = idx[s];
    kvb = kvb < 0 ? 0 : (kvb >= p.Tk ? p.Tk - 1 : kvb);
    const int ty = tys[s];
    mode = (ty == kCausal || ty == kFull || ty == kPartial) ? ty : int(kMasked);
    pid = -1;
    if (mode == kPartial) {  // :119-131, plus the upper bound on the index
      pid = has_partial ? pidx[s] : -1;
      if (pid < 0 || pid >= p.num_partial) mode = kMasked;
    }
    if (mode == kMasked) return false;  // :108-110
    kv_start = kvb * p.KB;
    kv_end = kv_start + p.KB < p.seqlen ? kv_start + p.KB : p.seqlen;  // :113
    if (mode == kCausal) {  // :134-140
      if (q_idx < kv_start) return false;
      kv_end = kv_end < q_idx + 1 ? kv_end : q_idx + 1;
    }
    return kv_start < kv_end;
  };
  auto score_of = [&](int kv, int kv_start, int pid, int mode, bool& allowed) {
    allowed = true;
    if (mode == kPartial) {  // :143-154
      const int local_q = q_idx - q_block * p.QB, local_kv = kv - kv_start;
      allowed = p.partial_masks[(size_t(pid) * p.QB + local_q) * p.KB + local_kv] != 0;
    }
    const uint16_t* krow = p.k + slab + size_t(kv) * p.D;
    float s = 0.f;
    if (p.k_rows_16b) {  // rows of K start on 16-byte boundaries: eight elements per load
      typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
      const u32x4_t* k8 = reinterpret_cast<const u32x4_t*>(krow);
      for (int d8 = 0; d8 < p.D / 8; ++d8) {
        const u32x4_t kk = k8[d8];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t pair = kk[e];
          s = __builtin_fmaf(sq[w][8 * d8 + 2 * e], to_float<BF16>(uint16_t(pair & 0xffffu)), s);
          s = __builtin_fmaf(sq[w][8 * d8 + 2 * e + 1], to_float<BF16>(uint16_t(pair >> 16)), s);
        }
      }
    } else {
      for (int d = 0; d < p.D; ++d) s = __builtin_fmaf(sq[w][d], to_float<BF16>(krow[d]), s);
    }
    s *= p.scale;  // :88
    if (p.softcap > 0.f) s = tanhf(s / p.softcap) * p.softcap;
    return s;
  };

  // pass 0: row maximum
  float mx = -INFINITY;
  for (int s = 0; s < nb; ++s) {
    int kv_start, kv_end, pid, mode;
    if (!slot_range(s, kv_start, kv_end, pid, mode)) continue;
    for (int kv = kv_start + lane; kv < kv_end; kv += 64) {
      bool allowed;
      const float sc = score_of(kv, kv_start, pid, mode, allowed);
      if (allowed) mx = fmaxf(mx, sc);
    }
  }
  mx = wave_max(mx);
  if (mx == -INFINITY) {  // everything masked: zeros (:177-183)
    write_empty();
    return;
  }
  // pass 1: weights, their sum, weighted V
  float sum = 0.f;
  float acc[kMaxD / 64] = {0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < nb; ++s) {
    int kv_start, kv_end, pid, mode;
    if (!slot_range(s, kv_start, kv_end, pid, mode)) continue;
    for (int base = kv_start; base < kv_end; base += 64) {
      const int kv = base + lane;
      float wgt = 0.f;
      if (kv < kv_end) {
        bool allowed;
        const float sc = score_of(kv, kv_start, pid, mode, allowed);
        if (allowed) wgt = __expf(sc - mx);  // :270-272
      }
      sum += wgt;
      const int n = kv_end - base < 64 ? kv_end - base : 64;
      for (int j = 0; j < n; ++j) {
        const float wj = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wgt), j));
        if (wj == 0.f) continue;
        const uint16_t* vrow = p.v + slab + size_t(base + j) * p.D;
#pragma unroll
        for (int i = 0; i < kMaxD / 64; ++i) {
          const int d = lane + 64 * i;
          if (i < ND && d < p.D) acc[i] = __builtin_fmaf(wj, to_float<BF16>(vrow[d]), acc[i]);
        }
      }
    }
  }
  sum = wave_sum(sum);
  const float inv = sum > 0.f ? 1.f / sum : 0.f;  // :283-288
#pragma unroll
  for (int i = 0; i < kMaxD / 64; ++i) {
    const int d = lane + 64 * i;
    if (i < ND && d < p.D) orow[d] = from_float<BF16>(acc[i] * inv);
  }
  if (lane == 0 && p.lse) p.lse[row] = sum > 0.f ? mx + __logf(sum) : -INFINITY;
}

}  // namespace

extern "C" int omni_attn_fwd_generic_gfx950(const void* q, const void* k, const void* v, void* o,
                                            float* lse_or_null, const int32_t* kv_num_blocks,
                                            const int32_t* kv_indices, const int32_t* block_mask_types,
                                            const int32_t* partial_idx_or_null,
                                            const uint8_t* partial_masks_or_null, int B, int H, int S_pad,
                                            int D, int Tq, int max_blocks, int QB, int KB, int num_partial,
                                            int seqlen_orig, int dtype, float softcap, void* stream) {
  if (!q || !k || !v || !o || !kv_num_blocks || !kv_indices || !block_mask_types)
    return OMNI_ATTN_ERR_NULL_POINTER;
  const auto misaligned = [](const void* ptr, uintptr_t a) { return (reinterpret_cast<uintptr_t>(ptr) & (a - 1)) != 0; };
  if (misaligned(q, 2) || misaligned(k, 2) || misaligned(v, 2) || misaligned(o, 2) || misaligned(lse_or_null, 4) ||
      misaligned(kv_num_blocks, 4) || misaligned(kv_indices, 4) || misaligned(block_mask_types, 4) ||
      misaligned(partial_idx_or_null, 4))
    return OMNI_ATTN_ERR_MISALIGNED;
  if (dtype != OMNI_ATTN_DTYPE_F16 && dtype != OMNI_ATTN_DTYPE_BF16) return OMNI_ATTN_ERR_UNSUPPORTED_DTYPE;
  if (D <= 0 || D > kMaxD) return OMNI_ATTN_ERR_UNSUPPORTED_HEAD_DIM;  // the reference's bound, attn_naive.cu:189-190
  if (QB <= 0 || KB <= 0) return OMNI_ATTN_ERR_UNSUPPORTED_BLOCK;
  if (B <= 0 || H <= 0 || S_pad <= 0 || Tq <= 0 || max_blocks <= 0 || seqlen_orig < 0 || num_partial < 0 ||
      !(softcap >= 0.f) || std::isinf(softcap))
    return OMNI_ATTN_ERR_BAD_SHAPE;
  if (Tq != (S_pad + QB - 1) / QB) return OMNI_ATTN_ERR_BAD_SHAPE;
  const long long rows = (long long)B * H * S_pad;
  if ((long long)S_pad * D > 0x7fffffffLL || rows > (1LL << 33) || (long long)B * H * Tq * max_blocks > (1LL << 40))
    return OMNI_ATTN_ERR_TOO_LARGE;
  GenericParams p;
  p.q = static_cast<const uint16_t*>(q);
  p.k = static_cast<const uint16_t*>(k);
  p.v = static_cast<const uint16_t*>(v);
  p.o = static_cast<uint16_t*>(o);
  p.lse = lse_or_null;
  p.kv_num_blocks = kv_num_blocks;
  p.kv_indices = kv_indices;
  p.types = block_mask_types;
  const bool has_partial = partial_idx_or_null && partial_masks_or_null && num_partial > 0;
  p.partial_idx = has_partial ? partial_idx_or_null : nullptr;
  p.partial_masks = has_partial ? partial_masks_or_null : nullptr;
  p.num_partial = has_partial ? num_partial : 0;
  p.S = S_pad;
  p.D = D;
  p.Tq = Tq;
  p.Tk = (S_pad + KB - 1) / KB;
  p.max_blocks = max_blocks;
  p.QB = QB;
  p.KB = KB;
  p.seqlen = seqlen_orig < S_pad ? seqlen_orig : S_pad;
  p.rows = rows;
  p.scale = float(1.0 / std::sqrt(double(D)));
  p.softcap = softcap;
  p.k_rows_16b = (D % 8 == 0) && (reinterpret_cast<uintptr_t>(k) & 15) == 0;
  const unsigned grid = unsigned((rows + kRowsPerWorkgroup - 1) / kRowsPerWorkgroup);
  const void* kern = dtype == OMNI_ATTN_DTYPE_BF16 ? reinterpret_cast<const void*>(fwd_generic_kernel<true>)
                                                   : reinterpret_cast<const void*>(fwd_generic_kernel<false>);
  void* args[] = {&p};
  const hipError_t e = hipLaunchKernel(kern, dim3(grid), dim3(64 * kRowsPerWorkgroup), args, 0,
                                       static_cast<hipStream_t>(stream));
  if (e != hipSuccess) {
    omni_attn::record_hip_error(int(e));
    return OMNI_ATTN_ERR_LAUNCH;
  }
  return OMNI_ATTN_OK;
}
